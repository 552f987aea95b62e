// bf16 / fp16 block GEMM: choice of kernel and tile configuration (the same for both element types).
//   - large tile-aligned problems (>= 128 tiles of 256x256, K a multiple of 64,
//     16-byte aligned rows, at most 4 k-steps and 2 addends): the LDS-DMA
//     kernel (gemm_bf16_dma.h);
//   - the same kernel split along k when the output has too few 256x256 tiles
//     to occupy the chip but the reduction is long (the weight-gradient shape
//     X^T dY), given scratch for the fp32 partial sums: `slices` blocks per
//     tile, then splitk_reduce_kernel adds them in slice order and applies the
//     epilogue;
//   - everything else: the register-staged kernel (gemm_bf16_kernel.h), with
//     256x256 or 128x128 tiles, guarded when the shape is ragged or unaligned.
// CW_GEMM_IMPL=staged in the environment forces the register-staged kernel.
#include <cstdlib>
#include <cstring>

#include "gemm_bf16_kernel.h"
#include "gemm_plan.h"

namespace cw {

int gemm_bf16_dma_launch_nn(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a, const void* tail_b);
int gemm_bf16_dma_launch_nt(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a, const void* tail_b);
int gemm_bf16_dma_launch_tn(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a, const void* tail_b);

int gemm_bf16_dma_split_launch_nn(const GemmArgs& args, int slices, hipStream_t s);
int gemm_bf16_dma_split_launch_nt(const GemmArgs& args, int slices, hipStream_t s);
int gemm_bf16_dma_split_launch_tn(const GemmArgs& args, int slices, hipStream_t s);

int gemm_f16_dma_launch_nn(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a, const void* tail_b);
int gemm_f16_dma_launch_nt(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a, const void* tail_b);
int gemm_f16_dma_launch_tn(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a, const void* tail_b);

int gemm_f16_dma_split_launch_nn(const GemmArgs& args, int slices, hipStream_t s);
int gemm_f16_dma_split_launch_nt(const GemmArgs& args, int slices, hipStream_t s);
int gemm_f16_dma_split_launch_tn(const GemmArgs& args, int slices, hipStream_t s);

int gemm_half_small_launch(const GemmArgs& args, int layout, int epilogue, bool f16, hipStream_t s);

namespace {

// C = epilogue(sum over slices of partial + addends + bias). One thread per 8
// consecutive columns of a row; slices are added in index order.
template <int EPI, typename E>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int slices, int64_t M,
                                                            int64_t N, const E* __restrict__ bias,
                                                            const E* __restrict__ add0, const E* __restrict__ add1,
                                                            int64_t ldadd, E* __restrict__ C, int64_t ldc,
                                                            E* __restrict__ preact, int64_t ldp) {
    const int64_t vec_per_row = N / 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= M * vec_per_row) return;
    const int64_t row = idx / vec_per_row, col = (idx - row * vec_per_row) * 8;
    const float* p = partial + row * N + col;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    for (int z = 0; z < slices; ++z) {
        float lo[4], hi[4];
        unpack_raw(load_raw_stream(p + (int64_t)z * M * N), lo, (const float*)nullptr);
        unpack_raw(load_raw_stream(p + (int64_t)z * M * N + 4), hi, (const float*)nullptr);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[e] += lo[e];
            v[4 + e] += hi[e];
        }
    }
    float t[8];
    if (EPI != CW_EPI_NONE && bias != nullptr) {
        unpack_raw(load_raw(bias + col), t, (const E*)nullptr);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
    }
    if (add0 != nullptr) {
        unpack_raw(load_raw_stream(add0 + row * ldadd + col), t, (const E*)nullptr);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
    }
    if (add1 != nullptr) {
        unpack_raw(load_raw_stream(add1 + row * ldadd + col), t, (const E*)nullptr);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
    }
    if (preact != nullptr) store_raw_stream(preact + row * ldp + col, pack_raw(v, (const E*)nullptr));
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = gemm_bf16::epi_act<EPI>(v[e]);
    store_raw_stream(C + row * ldc + col, pack_raw(v, (const E*)nullptr));
}

template <int EPI, typename E>
int launch_splitk_reduce(const GemmArgs& a, int slices, hipStream_t s) {
    const int64_t threads = (int64_t)a.M * (a.N / 8);
    hipLaunchKernelGGL((splitk_reduce_kernel<EPI, E>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,
                       (const float*)a.workspace, slices, (int64_t)a.M, (int64_t)a.N, (const E*)a.bias,
                       (const E*)(a.n_addends > 0 ? a.addend[0] : nullptr),
                       (const E*)(a.n_addends > 1 ? a.addend[1] : nullptr), a.ldadd, (E*)a.C, a.ldc, (E*)a.preact, a.ldp);
    return check_launch("splitk_reduce_kernel");
}

template <typename E>
int splitk_reduce(const GemmArgs& a, int slices, int epilogue, hipStream_t s) {
    switch (epilogue) {
        case CW_EPI_NONE: return launch_splitk_reduce<CW_EPI_NONE, E>(a, slices, s);
        case CW_EPI_BIAS: return launch_splitk_reduce<CW_EPI_BIAS, E>(a, slices, s);
        case CW_EPI_BIAS_GELU_TANH: return launch_splitk_reduce<CW_EPI_BIAS_GELU_TANH, E>(a, slices, s);
        case CW_EPI_BIAS_GELU_ERF: return launch_splitk_reduce<CW_EPI_BIAS_GELU_ERF, E>(a, slices, s);
        case CW_EPI_BIAS_RELU: return launch_splitk_reduce<CW_EPI_BIAS_RELU, E>(a, slices, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    }
}

}  // namespace

// Rows K-32 .. K-1 of a [K, N] operand (row pitch ld) into `out` (same pitch), the first `zero_rows` of
// them as zeros: the k-slow operand of the short extra step that finishes a reduction length K which is
// not a multiple of 32. The step covers k in [K-32, K); the part that overlaps the regular steps
// (zero_rows = 32 - K % 32 rows) must not count twice, and a zero row of this operand takes it out.
__global__ __launch_bounds__(256) void ktail_rows_kernel(const uint16_t* __restrict__ src, int64_t ld, int64_t K, int N,
                                                         int zero_rows, uint16_t* __restrict__ out) {
    const int vec_per_row = N / 8;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= 32 * vec_per_row) return;
    const int r = idx / vec_per_row, c = (idx - r * vec_per_row) * 8;
    raw16_t v = (raw16_t){0u, 0u, 0u, 0u};
    if (r >= zero_rows) v = load_raw(src + (K - 32 + r) * ld + c);
    *reinterpret_cast<raw16_t*>(out + (int64_t)r * ld + c) = v;
}

static bool dma_kernel_enabled() {
    static const bool enabled = [] {
        const char* v = std::getenv("CW_GEMM_IMPL");
        return !(v != nullptr && std::strcmp(v, "staged") == 0);
    }();
    return enabled;
}

// CW_GEMM_IMPL=onelaunch keeps a product whose last round of tiles is mostly empty in one launch (A/B measurements).
static bool strip_split_enabled() {
    static const bool enabled = [] {
        const char* v = std::getenv("CW_GEMM_IMPL");
        return !(v != nullptr && std::strcmp(v, "onelaunch") == 0);
    }();
    return enabled;
}

static int staged_launch(const GemmArgs& a, int layout, int epilogue, bool big, bool exact, bool f16, hipStream_t s) {
    switch (layout) {
        case CW_NN: return f16 ? gemm_f16_launch_nn(a, epilogue, big, exact, s) : gemm_bf16_launch_nn(a, epilogue, big, exact, s);
        case CW_NT: return f16 ? gemm_f16_launch_nt(a, epilogue, big, exact, s) : gemm_bf16_launch_nt(a, epilogue, big, exact, s);
        case CW_TN: return f16 ? gemm_f16_launch_tn(a, epilogue, big, exact, s) : gemm_bf16_launch_tn(a, epilogue, big, exact, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

static int dma_launch(const GemmArgs& a, int layout, int epilogue, bool f16, hipStream_t s, const void* tail_a = nullptr,
                      const void* tail_b = nullptr) {
    switch (layout) {
        case CW_NN:
            return f16 ? gemm_f16_dma_launch_nn(a, epilogue, s, tail_a, tail_b) : gemm_bf16_dma_launch_nn(a, epilogue, s, tail_a, tail_b);
        case CW_NT:
            return f16 ? gemm_f16_dma_launch_nt(a, epilogue, s, tail_a, tail_b) : gemm_bf16_dma_launch_nt(a, epilogue, s, tail_a, tail_b);
        case CW_TN:
            return f16 ? gemm_f16_dma_launch_tn(a, epilogue, s, tail_a, tail_b) : gemm_bf16_dma_launch_tn(a, epilogue, s, tail_a, tail_b);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

// f16: the operands, bias, addends and outputs are IEEE half instead of bfloat16; everything else is shared.
// The choice of kernel and the cuts are gemm_half_plan's (gemm_plan.hip); this function only launches.
int gemm_half_launch(const GemmArgs& args, int layout, int epilogue, bool f16, hipStream_t s) {
    const GemmPlan plan = gemm_half_plan(args, layout, dma_kernel_enabled(), strip_split_enabled());
    switch (plan.route) {
        case kRouteSmallRing: return gemm_half_small_launch(plan.head, layout, epilogue, f16, s);
        case kRouteRing: return dma_launch(plan.head, layout, epilogue, f16, s);
        case kRouteRingThenSmall: {
            if (const int rc = dma_launch(plan.head, layout, epilogue, f16, s); rc != CW_OK) return rc;
            return gemm_half_small_launch(plan.tail, layout, epilogue, f16, s);
        }
        case kRouteRingKTail: {
            uint16_t* tail_b = reinterpret_cast<uint16_t*>(args.workspace);
            const int vecs = 32 * (args.N / 8);
            hipLaunchKernelGGL(ktail_rows_kernel, dim3((vecs + 255) / 256), dim3(256), 0, s,
                               reinterpret_cast<const uint16_t*>(args.B[0]), args.ldb, (int64_t)args.K, args.N,
                               plan.ktail_zero_rows, tail_b);
            if (const int rc = check_launch("ktail_rows_kernel"); rc != CW_OK) return rc;
            return dma_launch(plan.head, layout, epilogue, f16, s, plan.ktail_a, tail_b);
        }
        case kRouteSplitK: {
            int rc;
            switch (layout) {
                case CW_NN: rc = f16 ? gemm_f16_dma_split_launch_nn(args, plan.slices, s) : gemm_bf16_dma_split_launch_nn(args, plan.slices, s); break;
                case CW_NT: rc = f16 ? gemm_f16_dma_split_launch_nt(args, plan.slices, s) : gemm_bf16_dma_split_launch_nt(args, plan.slices, s); break;
                case CW_TN: rc = f16 ? gemm_f16_dma_split_launch_tn(args, plan.slices, s) : gemm_bf16_dma_split_launch_tn(args, plan.slices, s); break;
                default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
            }
            if (rc != CW_OK) return rc;
            return f16 ? splitk_reduce<f16_t>(args, plan.slices, epilogue, s) : splitk_reduce<bf16_t>(args, plan.slices, epilogue, s);
        }
        default: return staged_launch(args, layout, epilogue, plan.big, plan.exact, f16, s);
    }
}

}  // namespace cw
