// 16-bit block GEMM for outputs with too few 256x256 tiles for the chip (shards of a larger grid, small
// batches): 128x128 tiles, 2x2 wavefronts of 64x64, a ring of 4 LDS stages of k = 64 filled by the load
// unit, three tiles of prefetch. Where the register-staged kernel issues a tile's loads one tile ahead and
// waits out their latency in every trip (1.4 us per k tile of 64 for 0.25 us of MFMA work), this one has
// them in flight for three trips.
//
// Built from the tile images of the attention kernels (attention_common.h): an operand tile of 128 rows x
// 64 k is two 64 x 64 images, a k-contiguous operand as "row images" (read with ds_read_b128), a k-slow one
// as "transpose images" of its [64 k][64 rows] blocks (read with the transposing ds_read_b64_tr_b16); both
// are conflict free and written by global_load_lds_dwordx4 with the swizzle applied on the global side.
// One barrier per stage, after the first half of its products: it publishes the next stage, whose first
// fragments are read during the second half, and frees the previous one for the loads issued right behind it.
// The products go to the shared epilogue of gemm_bf16_kernel.h (bias, addends, pre-activation copy,
// activation, staging through LDS, whole-row stores).
#include "attention_common.h"
#include "gemm_bf16_kernel.h"

namespace cw {

namespace gemm_small {

using namespace attn;

constexpr int kBM = 128, kBN = 128, kBKs = 64, kNS = 4, kThreads = 256;
constexpr int kStageBytes = 4 * kImage;  // A rows 0..63, A rows 64..127, B rows 0..63, B rows 64..127
constexpr int kDmaPerTile = 8;           // per thread: 4 images x 512 chunk positions / 256 threads

// Transposing read of a transpose image that delivers the k order of a row image's ds_read_b128 (lane half
// h holds k = 8h .. 8h+7 of the 16-row block at R0), so that a k-slow operand can meet a k-contiguous one in
// one MFMA: the attention kernels' read_transposed pairs tile rows 4h + {0..3} with 8 + 4h + {0..3}, which
// is the order of their accumulators. Same bank pattern (row parity and swizzle term are unchanged).
struct TrOffsetsK8 {
    int tr[2];  // [dt]
    __device__ __forceinline__ void init(int lane) {
        const int grp = lane >> 4, i16 = lane & 15;
        const int ra = 8 * (grp >> 1) + (i16 >> 2);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) tr[dt] = ra * 128 + (((2 * dt + (grp & 1)) ^ (ra & 3)) << 5) + 8 * (i16 & 3);
    }
};
template <int R0>
__device__ __forceinline__ bf16x8_t read_transposed_k8(lds_char* img, const TrOffsetsK8& to, int dt) {
    static_assert(R0 % 16 == 0, "row offset must keep the swizzle");
    lds_char* p = img + to.tr[dt] + R0 * 128;
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)p);
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 4 * 128));
    return __builtin_bit_cast(bf16x8_t, (s16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

template <bool TRANS_A, bool TRANS_B, int EPI, typename E>
__global__ __launch_bounds__(kThreads) void gemm_half_small_kernel(const RingArgs args) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds_u16[];
    lds_char* lds = (lds_char*)lds_u16;
    const uint32_t lds_addr0 = (uint32_t)(uintptr_t)lds;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int M = args.M, N = args.N, K = args.K;
    // the last tile of a row or column of tiles is moved back to end at the edge (it overlaps its neighbour;
    // both compute the shared elements from the same operands in the same order)
    const int tiles_m = (M + kBM - 1) / kBM, tiles_n = (N + kBN - 1) / kBN;
    const int total = tiles_m * tiles_n;
    int tile;
    {
        const int pid = blockIdx.x;
        const int per_xcd = (total + 7) / 8;
        tile = (pid & 7) * per_xcd + (pid >> 3);
        if (tile >= total) return;
    }
    constexpr int GROUP_M = 8;
    const int group = tile / (GROUP_M * tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int in_group = tile - group * GROUP_M * tiles_n;
    int m0 = (first_m + in_group % gsz) * kBM;
    int n0 = (in_group / gsz) * kBN;
    m0 = m0 + kBM > M ? M - kBM : m0;
    n0 = n0 + kBN > N ? N - kBN : n0;

    const int kt_per_step = K / kBKs;
    const int KT = kt_per_step * args.n_steps;

    ReadOffsets ro;
    ro.init(lane);
    TrOffsetsK8 to;
    to.init(lane);
    TileDma<kThreads> dma;
    dma.init(tid);

    // the tile whose loads are issued next; past the last tile the position stays on it (harmless duplicate
    // loads into a free stage keep the load counting the same in every trip)
    int is_kt = 0, is_step = 0, is_k0 = 0, is_stage = 0;
    const uint16_t* is_a = reinterpret_cast<const uint16_t*>(args.A[0]);
    const uint16_t* is_b = reinterpret_cast<const uint16_t*>(args.B[0]);
    auto issue_tile = [&]() {
        const uint32_t st = lds_addr0 + is_stage * kStageBytes;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            // k-contiguous operand [rows][k]: tile rows are operand rows, its 64 columns are k0 .. k0+63;
            // k-slow operand [k][rows]: tile rows are k0 .. k0+63, its 64 columns are operand rows
            if constexpr (!TRANS_A) dma.template load<true, false>(is_a + is_k0, args.lda, m0 + 64 * p, M, st + p * kImage, 0);
            else dma.template load<false, true>(is_a + m0 + 64 * p, args.lda, is_k0, K, 0, st + p * kImage);
            if constexpr (!TRANS_B) dma.template load<true, false>(is_b + is_k0, args.ldb, n0 + 64 * p, N, st + (2 + p) * kImage, 0);
            else dma.template load<false, true>(is_b + n0 + 64 * p, args.ldb, is_k0, K, 0, st + (2 + p) * kImage);
        }
        if (is_kt + 1 < KT) {
            ++is_kt;
            is_k0 += kBKs;
            if (is_k0 >= K) {
                is_k0 = 0;
                ++is_step;
                is_a = reinterpret_cast<const uint16_t*>(gemm_bf16::pick_ptr(args.A, is_step));
                is_b = reinterpret_cast<const uint16_t*>(gemm_bf16::pick_ptr(args.B, is_step));
            }
        }
        is_stage = (is_stage + 1 == kNS) ? 0 : is_stage + 1;
    };

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // fragments of k block kb (16 values of k) of a stage: A blocks i = 0, 1 of this wavefront's 64 rows
    // (image wm), B blocks j = 0, 1 of its 64 columns (image 2 + wn)
    auto read_frags = [&](lds_char* st, auto kbc, bf16x8_t (&af)[2], bf16x8_t (&bfr)[2]) {
        constexpr int KB = decltype(kbc)::value;
        lds_char* ia = st + wm * kImage;
        lds_char* ib = st + (2 + wn) * kImage;
        if constexpr (!TRANS_A) {
            af[0] = read_rows<0>(ia, ro, KB);
            af[1] = read_rows<32>(ia, ro, KB);
        } else {
            af[0] = read_transposed_k8<16 * KB>(ia, to, 0);
            af[1] = read_transposed_k8<16 * KB>(ia, to, 1);
        }
        if constexpr (!TRANS_B) {
            bfr[0] = read_rows<0>(ib, ro, KB);
            bfr[1] = read_rows<32>(ib, ro, KB);
        } else {
            bfr[0] = read_transposed_k8<16 * KB>(ib, to, 0);
            bfr[1] = read_transposed_k8<16 * KB>(ib, to, 1);
        }
    };
    // the B fragment goes in as the first MFMA operand, so that a lane ends up with four consecutive output
    // columns per register quad (the layout the shared epilogue takes)
    auto products = [&](const bf16x8_t (&af)[2], const bf16x8_t (&bfr)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = mfma16<E>(bfr[j], af[i], acc[i][j]);
    };

    // prologue: tiles 0 .. NS-2 in flight; tile 0 complete before the first read
    for (int p = 0; p < kNS - 1; ++p) issue_tile();
    dma_wait<kDmaPerTile*(kNS - 2)>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    bf16x8_t af[2][2], bfr[2][2];
    read_frags(lds, std::integral_constant<int, 0>{}, af[0], bfr[0]);
    int cur = 0;
    for (int kt = 0; kt < KT; ++kt) {
        lds_char* st = lds + cur * kStageBytes;
        const int nxt = (cur + 1 == kNS) ? 0 : cur + 1;
        lds_char* ns = lds + nxt * kStageBytes;
        read_frags(st, std::integral_constant<int, 1>{}, af[1], bfr[1]);
        products(af[0], bfr[0]);
        read_frags(st, std::integral_constant<int, 2>{}, af[0], bfr[0]);
        products(af[1], bfr[1]);
        // tile kt+1 complete for everybody, the stage of tile kt-1 free: its next tenant's loads go out
        dma_wait<kDmaPerTile*(kNS - 3)>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue_tile();
        read_frags(st, std::integral_constant<int, 3>{}, af[1], bfr[1]);
        products(af[0], bfr[0]);
        read_frags(ns, std::integral_constant<int, 0>{}, af[0], bfr[0]);
        products(af[1], bfr[1]);
        cur = nxt;
    }
    dma_wait<0>();
    __syncthreads();
    gemm_bf16::gemm_epilogue<kBM, kBN, 2, 2, EPI, true, E>(acc, args, lds_u16, m0, n0, wm, wn, lane, tid);
}

template <bool TA, bool TB, int EPI, typename E>
int launch_cfg(const RingArgs& args, hipStream_t s) {
    auto kern = gemm_half_small_kernel<TA, TB, EPI, E>;
    constexpr size_t stages = (size_t)kNS * kStageBytes;
    constexpr size_t ctile = (size_t)kBM * gemm_bf16::c_pitch<kBN>() * sizeof(uint16_t);
    constexpr size_t lds = stages > ctile ? stages : ctile;
    static_assert(lds <= 160 * 1024, "LDS image does not fit the CU");
    if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)((int)lds), "gemm_half_small"); lrc != CW_OK) return lrc;
    const int tiles = ((args.M + kBM - 1) / kBM) * ((args.N + kBN - 1) / kBN);
    hipLaunchKernelGGL(kern, dim3(((tiles + 7) / 8) * 8), dim3(kThreads), lds, s, args);
    return check_launch("gemm_half_small_kernel");
}

template <bool TA, bool TB, typename E>
int launch_epi(const RingArgs& args, int epilogue, hipStream_t s) {
    switch (epilogue) {
        case CW_EPI_NONE: return launch_cfg<TA, TB, CW_EPI_NONE, E>(args, s);
        case CW_EPI_BIAS: return launch_cfg<TA, TB, CW_EPI_BIAS, E>(args, s);
        case CW_EPI_BIAS_GELU_TANH: return launch_cfg<TA, TB, CW_EPI_BIAS_GELU_TANH, E>(args, s);
        case CW_EPI_BIAS_GELU_ERF: return launch_cfg<TA, TB, CW_EPI_BIAS_GELU_ERF, E>(args, s);
        case CW_EPI_BIAS_RELU: return launch_cfg<TA, TB, CW_EPI_BIAS_RELU, E>(args, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    }
}

template <typename E>
int launch_layout(const RingArgs& args, int layout, int epilogue, hipStream_t s) {
    switch (layout) {
        case CW_NN: return launch_epi<false, true, E>(args, epilogue, s);
        case CW_NT: return launch_epi<false, false, E>(args, epilogue, s);
        case CW_TN: return launch_epi<true, true, E>(args, epilogue, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

}  // namespace gemm_small

// The caller has checked: every pointer and leading dimension good for 16-byte accesses, M, N >= 128, N a
// multiple of 8 (and M for CW_TN), K a multiple of 64, at most kRingMaxSteps steps and kRingMaxAddends
// addends, leading dimensions below 2^23 elements.
int gemm_half_small_launch(const GemmArgs& g, int layout, int epilogue, bool f16, hipStream_t s) {
    RingArgs r = {};
    for (int i = 0; i < g.n_steps && i < kRingMaxSteps; ++i) { r.A[i] = g.A[i]; r.B[i] = g.B[i]; }
    for (int i = 0; i < g.n_addends && i < kRingMaxAddends; ++i) r.addend[i] = g.addend[i];
    r.bias = g.bias; r.C = g.C; r.preact = g.preact;
    r.lda = g.lda; r.ldb = g.ldb; r.ldc = g.ldc; r.ldp = g.ldp; r.ldadd = g.ldadd;
    r.M = g.M; r.N = g.N; r.K = g.K; r.n_steps = g.n_steps; r.n_addends = g.n_addends;
    r.vec_bias = 1; r.vec_add = 1; r.k_tail = 0; r.partial = nullptr;
    return f16 ? gemm_small::launch_layout<f16_t>(r, layout, epilogue, s) : gemm_small::launch_layout<bf16_t>(r, layout, epilogue, s);
}

}  // namespace cw
