// Measurement aid (libcubework_diag.so, loaded by bench.py only): the ring kernel of the block GEMM with one part
// taken out, so that the part's share of a launch - in time and, through the socket's energy counter, in joules -
// can be read as a difference against the whole kernel. Same source as the library's kernel (gemm_bf16_dma.h),
// another value of its ABL template parameter:
//   part 0  the whole kernel (the instantiation the library launches for this shape)
//   part 1  the k loop issues no operand loads: the four LDS stages are filled once and re-used
//   part 2  no epilogue: no bias / activation arithmetic, nothing stored
//   part 3  the k loop reads no fragments from LDS: the first tile's stay in the registers
// NN layout, bf16, bias + GeLU(tanh) epilogue, tile-aligned shapes with at least 128 tiles, 1 to 4 k-steps:
// the headline shape of the benchmark. Results of parts 1 to 3 are meaningless as numbers.
#include "gemm_bf16_dma.h"

namespace cw {
namespace {

template <int ABL>
int launch_part(const RingArgs& args, hipStream_t s) {
    auto kern = gemm_dma::gemm_bf16_dma_kernel<false, true, CW_EPI_BIAS_GELU_TANH, gemm_dma::kStages, false, bf16_t, ABL>;
    constexpr size_t lds = gemm_dma::lds_bytes_dma<gemm_dma::kStages>();
    if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)lds, "gemm_bf16_ring (measurement build)"); lrc != CW_OK)
        return lrc;
    const int tiles = (args.M / gemm_dma::kTile) * (args.N / gemm_dma::kTile);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(gemm_dma::kThreads), lds, s, args);
    return check_launch("gemm_bf16_dma_kernel (measurement build)");
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int cw_diag_gemm_part(int part, int64_t M, int64_t N, int64_t K, int n_steps, const void* const* A_steps,
                                 int64_t lda, const void* const* B_steps, int64_t ldb, const void* bias, void* C,
                                 int64_t ldc, void* stream) {
    if (part < 0 || part > 3) return fail(CW_ERR_INVALID, "cw_diag_gemm_part: part %d outside [0, 3]", part);
    if (n_steps < 1 || n_steps > kRingMaxSteps || A_steps == nullptr || B_steps == nullptr || bias == nullptr || C == nullptr)
        return fail(CW_ERR_INVALID, "cw_diag_gemm_part: 1 to %d k-steps, operands, bias and C are needed", kRingMaxSteps);
    if (M < 256 || N < 256 || K < 128 || (M % 256) != 0 || (N % 256) != 0 || (K % 64) != 0 || (M / 256) * (N / 256) < 128 ||
        M > (1 << 24) || N > (1 << 24) || K > (1 << 24))
        return fail(CW_ERR_UNSUPPORTED, "cw_diag_gemm_part: tile-aligned shapes with at least 128 tiles of 256 x 256 only");
    if (lda < K || ldb < N || ldc < N || (lda % 8) != 0 || (ldb % 8) != 0 || (ldc % 8) != 0)
        return fail(CW_ERR_ALIGNMENT, "cw_diag_gemm_part: leading dimensions must cover the rows and be multiples of 8");
    for (int i = 0; i < n_steps; ++i)
        if (A_steps[i] == nullptr || B_steps[i] == nullptr || !aligned16(A_steps[i]) || !aligned16(B_steps[i]))
            return fail(CW_ERR_ALIGNMENT, "cw_diag_gemm_part: step operands must be 16-byte aligned");
    if (!aligned16(C) || !aligned16(bias)) return fail(CW_ERR_ALIGNMENT, "cw_diag_gemm_part: C and bias must be 16-byte aligned");
    if (const int drc = require_gfx950("cw_diag_gemm_part"); drc != CW_OK) return drc;
    RingArgs args = {};
    for (int i = 0; i < n_steps; ++i) {
        args.A[i] = A_steps[i];
        args.B[i] = B_steps[i];
    }
    args.bias = bias;
    args.C = C;
    args.lda = lda;
    args.ldb = ldb;
    args.ldc = ldc;
    args.M = (int)M;
    args.N = (int)N;
    args.K = (int)K;
    args.n_steps = n_steps;
    args.vec_bias = 1;
    args.vec_add = 1;
    hipStream_t s = (hipStream_t)stream;
    switch (part) {
        case 0: return launch_part<0>(args, s);
        case 1: return launch_part<1>(args, s);
        case 2: return launch_part<2>(args, s);
        default: return launch_part<3>(args, s);
    }
}
