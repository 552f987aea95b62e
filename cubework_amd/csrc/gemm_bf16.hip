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

int gemm_bf16_split_slices(int64_t M, int64_t N, int64_t K, int n_steps) {
    if (M <= 0 || N <= 0 || K <= 0 || n_steps <= 0 || n_steps > kRingMaxSteps) return 1;
    if ((M % 256) != 0 || (N % 256) != 0 || (K % 64) != 0) return 1;
    const int64_t tiles = (M / 256) * (N / 256);
    if (tiles >= 128 || K * n_steps < 2048) return 1;  // enough tiles already, or a short reduction
    int slices = 8;
    while (slices > 1 && (tiles * slices > 256 || (K % (64 * slices)) != 0 || K / slices < 256)) slices >>= 1;
    return slices;
}

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

int64_t gemm_bf16_ktail_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps) {
    if (layout == CW_NT || n_steps != 1 || K < 64 || (K % 32) == 0 || (K % 8) != 0) return 0;
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    if (tiles < 128 || M < 256 || N < 256 || (N % 8) != 0) return 0;
    return 32 * N * (int64_t)sizeof(uint16_t);
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
int gemm_half_launch(const GemmArgs& args, int layout, int epilogue, bool f16, hipStream_t s) {
    // the unguarded kernels address operands with 32-bit byte offsets
    const int64_t max_dim = args.M > args.N ? (args.M > args.K ? args.M : args.K) : (args.N > args.K ? args.N : args.K);
    const bool fits32 = (max_dim + 64) * (args.lda > args.ldb ? args.lda : args.ldb) * 2 < ((int64_t)1 << 32);
    const bool all_vec = fits32 && args.vec_a && args.vec_b && args.vec_c && (args.preact == nullptr || args.vec_p) &&
                         (args.bias == nullptr || args.vec_bias) && (args.n_addends == 0 || args.vec_add);
    const int64_t tiles256 = (int64_t)((args.M + 255) / 256) * ((args.N + 255) / 256);
    const bool big = tiles256 >= 128;
    const int tile = big ? 256 : 128;
    const bool exact = all_vec && (args.M % tile) == 0 && (args.N % tile) == 0 && (args.K % gemm_bf16::kBK) == 0;
    const bool ring_ok = args.n_steps > 0 && args.n_steps <= kRingMaxSteps && args.n_addends <= kRingMaxAddends &&
                         dma_kernel_enabled();
    // The LDS-DMA kernel takes M and N that are not tile multiples (its last tiles overlap their
    // neighbours): a vocabulary slice of 12568 columns is 50 tiles instead of 49.1. What it needs is one
    // full tile in each direction and 16-byte steps wherever a tile origin moves along a contiguous
    // dimension (N always: the output and a [K, N] operand; M for a [K, M] operand).
    const bool edges_ok = args.M >= 256 && args.N >= 256 && (args.N % 8) == 0 && (layout != CW_TN || (args.M % 8) == 0);
    // Fewer than 160 tiles of 256 x 256 (at 128 .. 159 of them the large tiles leave 40 % of the compute units
    // idle, and four times as many small tiles fill them): the ring kernel with 128 x 128 tiles, unless a long
    // reduction over few tiles is better served by splitting k (below; measured on 2048 x 2048 outputs: the
    // small tiles win up to a reduction length of 8192, the split from 16384).
    const int slices = gemm_bf16_split_slices(args.M, args.N, args.K, args.n_steps);
    {
        const int64_t tiles128 = (int64_t)((args.M + 127) / 128) * ((args.N + 127) / 128);
        const bool splits = slices > 1 && args.workspace != nullptr && aligned16(args.workspace) &&
                            args.workspace_bytes >= (int64_t)slices * args.M * args.N * (int64_t)sizeof(float);
        if (tiles256 < 160 && all_vec && ring_ok && args.M >= 128 && args.N >= 128 && (args.N % 8) == 0 &&
            (layout != CW_TN || (args.M % 8) == 0) && args.K >= 64 && (args.K % 64) == 0 &&
            args.lda < ((int64_t)1 << 23) && args.ldb < ((int64_t)1 << 23) && ((tiles128 >= 192 && (int64_t)args.K * args.n_steps < 12288) || !splits))
            return gemm_half_small_launch(args, layout, epilogue, f16, s);
    }
    if (big && all_vec && ring_ok && edges_ok && (args.K % gemm_bf16::kBK) == 0) {
        // A last round of 256 x 256 tiles that is mostly empty (a vocabulary slice as N: 8192 x 12568 is 32 x 50 =
        // 1600 tiles, 6.25 rounds of the 256 compute units): when the partial round is whole tile columns (or whole
        // tile rows), at most 3/8 of a round, and that strip is at most one round of 128 x 128 tiles, it goes to the
        // small-tile kernel as a second launch and the rest is whole rounds.
        const int64_t tiles_m = (args.M + 255) / 256, tiles_n = (args.N + 255) / 256;
        const int64_t last_round = (tiles_m * tiles_n) % 256;
        const bool small_ok = (args.K % 64) == 0 && args.lda < ((int64_t)1 << 23) && args.ldb < ((int64_t)1 << 23);
        if (tiles_m * tiles_n > 256 && last_round > 0 && last_round <= 96 && small_ok && strip_split_enabled()) {
            auto shift = [&](const void* p, int64_t elems) -> const void* {
                return p == nullptr ? nullptr : reinterpret_cast<const uint16_t*>(p) + elems;
            };
            GemmArgs head = args, tail = args;
            bool split = false;
            if (last_round % tiles_m == 0) {  // whole tile columns
                const int64_t n0 = (tiles_n - last_round / tiles_m) * 256, strip = args.N - n0;
                if (n0 >= 256 && strip >= 128 && ((args.M + 127) / 128) * ((strip + 127) / 128) <= 256) {
                    head.N = (int)n0;
                    tail.N = (int)strip;
                    for (int i = 0; i < args.n_steps; ++i) tail.B[i] = shift(args.B[i], layout == CW_NT ? n0 * args.ldb : n0);
                    for (int k = 0; k < args.n_addends; ++k) tail.addend[k] = shift(args.addend[k], n0);
                    tail.bias = shift(args.bias, n0);
                    tail.C = const_cast<void*>(shift(args.C, n0));
                    tail.preact = const_cast<void*>(shift(args.preact, n0));
                    split = true;
                }
            }
            if (!split && last_round % tiles_n == 0) {  // whole tile rows
                const int64_t m0 = (tiles_m - last_round / tiles_n) * 256, strip = args.M - m0;
                if (m0 >= 256 && strip >= 128 && ((strip + 127) / 128) * ((args.N + 127) / 128) <= 256) {
                    head.M = (int)m0;
                    tail.M = (int)strip;
                    for (int i = 0; i < args.n_steps; ++i) tail.A[i] = shift(args.A[i], layout == CW_TN ? m0 : m0 * args.lda);
                    for (int k = 0; k < args.n_addends; ++k) tail.addend[k] = shift(args.addend[k], m0 * args.ldadd);
                    tail.C = const_cast<void*>(shift(args.C, m0 * args.ldc));
                    tail.preact = const_cast<void*>(shift(args.preact, m0 * args.ldp));
                    split = true;
                }
            }
            if (split) {
                if (const int rc = dma_launch(head, layout, epilogue, f16, s); rc != CW_OK) return rc;
                return gemm_half_small_launch(tail, layout, epilogue, f16, s);
            }
        }
        return dma_launch(args, layout, epilogue, f16, s);
    }
    // A reduction length that is not a multiple of the k tile (a vocabulary slice as K: 12568 = 392 x 32 +
    // 24), with B stored [K, N]: the regular step covers the first K - K % 32 columns, one more step of 32
    // covers [K-32, K) with a copy of B's last 32 rows whose overlapping rows are zero. The copy (64 bytes
    // per column) lives in the caller's scratch and has B's row pitch, which the steps share.
    if (big && all_vec && ring_ok && edges_ok && layout != CW_NT && args.n_steps == 1 && args.K >= 64 &&
        (args.K % 32) != 0 && (args.K % 8) == 0 && args.workspace != nullptr && aligned16(args.workspace) &&
        args.workspace_bytes >= 32 * args.ldb * (int64_t)sizeof(uint16_t)) {
        const int kr = args.K % 32;
        uint16_t* tail_b = reinterpret_cast<uint16_t*>(args.workspace);
        const int vecs = 32 * (args.N / 8);
        hipLaunchKernelGGL(ktail_rows_kernel, dim3((vecs + 255) / 256), dim3(256), 0, s,
                           reinterpret_cast<const uint16_t*>(args.B[0]), args.ldb, (int64_t)args.K, args.N, 32 - kr, tail_b);
        int rc = check_launch("ktail_rows_kernel");
        if (rc != CW_OK) return rc;
        // A's part of the step: columns (NN, A is [M, K]) or rows (TN, A is [K, M]) K-32 .. K-1, in place
        const uint16_t* a0 = reinterpret_cast<const uint16_t*>(args.A[0]);
        const void* tail_a = layout == CW_TN ? a0 + (int64_t)(args.K - 32) * args.lda : a0 + (args.K - 32);
        GemmArgs main_part = args;
        main_part.K = args.K - kr;
        return dma_launch(main_part, layout, epilogue, f16, s, tail_a, tail_b);
    }
    if (slices > 1 && all_vec && args.n_addends <= kRingMaxAddends && dma_kernel_enabled() &&
        args.workspace != nullptr && aligned16(args.workspace) &&
        args.workspace_bytes >= (int64_t)slices * args.M * args.N * (int64_t)sizeof(float)) {
        int rc;
        switch (layout) {
            case CW_NN: rc = f16 ? gemm_f16_dma_split_launch_nn(args, slices, s) : gemm_bf16_dma_split_launch_nn(args, slices, s); break;
            case CW_NT: rc = f16 ? gemm_f16_dma_split_launch_nt(args, slices, s) : gemm_bf16_dma_split_launch_nt(args, slices, s); break;
            case CW_TN: rc = f16 ? gemm_f16_dma_split_launch_tn(args, slices, s) : gemm_bf16_dma_split_launch_tn(args, slices, s); break;
            default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
        }
        if (rc != CW_OK) return rc;
        return f16 ? splitk_reduce<f16_t>(args, slices, epilogue, s) : splitk_reduce<bf16_t>(args, slices, epilogue, s);
    }
    return staged_launch(args, layout, epilogue, big, exact, f16, s);
}

}  // namespace cw
