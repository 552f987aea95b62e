// Kernel argument block shared by the bf16 / fp16 and fp32 block-GEMM kernels.
#pragma once

#include "cw_common.h"

namespace cw {

struct GemmArgs {
    const void* A[CW_MAX_KSTEPS];
    const void* B[CW_MAX_KSTEPS];
    const void* addend[CW_MAX_ADDENDS];
    const void* bias;
    void* C;
    void* preact;
    int64_t lda, ldb, ldc, ldp, ldadd;
    int M, N, K;  // K: reduction length of one step
    int n_steps, n_addends;
    // 1 when the operand's base and leading dimension allow 16-byte (bf16: 8
    // elements, fp32: 4 elements) row accesses; C/preact/addends/bias: 8-byte.
    int vec_a, vec_b, vec_c, vec_p, vec_add, vec_bias;
    // caller's scratch for split-k partial sums (may be NULL / 0)
    void* workspace;
    int64_t workspace_bytes;
};

// Compact argument block of the LDS-DMA kernel: few enough pointers that they
// all stay in scalar registers for the whole k loop.
constexpr int kRingMaxSteps = 4;
constexpr int kRingMaxAddends = 2;
struct RingArgs {
    const void* A[kRingMaxSteps];
    const void* B[kRingMaxSteps];
    const void* addend[kRingMaxAddends];
    const void* bias;
    void* C;
    void* preact;
    int64_t lda, ldb, ldc, ldp, ldadd;
    int M, N, K;
    int n_steps, n_addends;
    int vec_bias, vec_add;  // always 1 on this path; read by the shared epilogue
    // > 0: one more step follows the n_steps regular ones, with k extent k_tail and the operands
    // A[n_steps], B[n_steps] (how a reduction length that is not a multiple of the k tile is finished)
    int k_tail;
    float* partial;         // split-k only: [slices][M][N] fp32 partial sums
};

// Number of k slices the bf16 GEMM would split a problem into (1 = no split)
// when given scratch; the scratch it then needs is slices * M * N * 4 bytes.
int gemm_bf16_split_slices(int64_t M, int64_t N, int64_t K, int n_steps);
// Scratch for finishing a reduction length that is not a multiple of 32 on the LDS-DMA kernel (0: not used).
int64_t gemm_bf16_ktail_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps);

// bf16 (f16 = false) or fp16 (f16 = true) operands and outputs
int gemm_half_launch(const GemmArgs& args, int layout, int epilogue, bool f16, hipStream_t s);
int gemm_f32_launch(const GemmArgs& args, int layout, int epilogue, hipStream_t s);

}  // namespace cw
