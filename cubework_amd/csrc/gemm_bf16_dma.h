// SUMMA block GEMM for gfx950, large tile-aligned problems.
//
//   - 256x256 tile of C per 256-thread block (4 wavefronts, 2x2, 128x128 each =
//     4x4 v_mfma_f32_32x32x16_bf16 (E = f16_t: _f16) tiles = 256 fp32 accumulators per lane);
//   - operands stream global -> LDS through the load unit itself
//     (global_load_lds_dwordx4): no staging registers, no LDS write
//     instructions, no transposition ALU work;
//   - a ring of NS LDS stages of k extent 32 (32 KB each): while tile kt is
//     multiplied, tile kt+1 is complete and tiles kt+2.. are in flight. One
//     barrier per tile, in the middle of the tile's MFMAs, both publishes tile
//     kt+1 and frees the stage of tile kt-1, so no wave ever waits at a tile
//     boundary: the first fragments of tile kt+1 are read during the last MFMAs
//     of tile kt;
//   - fragments are read with ds_read_b128 (operand stored with k contiguous)
//     or with two ds_read_b64_tr_b16 (operand stored with k as the slow index:
//     the LDS read transposes 4x4 blocks across 16 lanes);
//   - every load, LDS read and MFMA of the loop body is placed by hand (one
//     memory instruction behind each MFMA) and pinned with scheduling fences;
//   - the loop body has no branches: past the last tile it keeps re-issuing the
//     last tile's loads into a free stage, which keeps the load-counter
//     arithmetic identical in every iteration.
//
// LDS image of one stage, 16 KB per operand:
//   k-contiguous operand : [256 rows][32 k], 64 B per row, 16-byte chunk c of
//     row r stored at chunk position c ^ ((r >> 2) & 3);
//   k-slow operand       : [32 k][256 rows], 512 B per k row, chunk c of k row k
//     stored at position c ^ ((k & 3) << 2).
// Both make the fragment reads bank-conflict free (measured: SQ_LDS_BANK_CONFLICT
// = 0). A load instruction writes 1 KB of LDS linearly (lane l -> bytes
// [16l, 16l+16)), so the swizzle is applied on the global side: lane l fetches
// the chunk that belongs at its LDS position.
//
// The loads are issued through inline asm on purpose: the compiler cannot tell
// the transposing LDS reads apart from the load unit's LDS writes and would wait
// for every outstanding load before each of them; the kernel counts its own
// loads instead (dma_wait<N>).
#pragma once
#include "gemm_bf16_kernel.h"

namespace cw {
namespace gemm_dma {

using gemm_bf16::bf16x8_t;
using gemm_bf16::f32x16_t;
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) char lds_char;

constexpr int kTile = 256;
constexpr int kBK = 32;
constexpr int kThreads = 256;
constexpr int kOperBytes = kTile * kBK * 2;  // 16384
constexpr int kStageBytes = 2 * kOperBytes;  // 32768
constexpr int kDmaPerTile = 8;               // load instructions per wavefront per tile


template <bool TRANS>
__device__ __forceinline__ void dma_lane_offsets(int lane, int64_t ld, int row0, uint32_t& even, uint32_t& odd) {
    if constexpr (!TRANS) {
        // instruction = 16 rows x 64 B; lane -> row lane/4, chunk position lane%4; swizzle (row>>2)&3 = lane>>4
        const int r = lane >> 2, c = (lane & 3) ^ (lane >> 4);
        even = odd = (uint32_t)((((int64_t)(row0 + r)) * ld + c * 8) * 2);
    } else {
        const int kr = lane >> 5, cpos = lane & 31;
        even = (uint32_t)((((int64_t)kr) * ld + row0 + (cpos ^ (kr << 2)) * 8) * 2);
        odd = (uint32_t)((((int64_t)kr) * ld + row0 + (cpos ^ ((2 + kr) << 2)) * 8) * 2);
    }
}

// one of the wavefront's 4 load instructions (I) of an operand tile
template <bool TRANS, int I>
__device__ __forceinline__ void dma_one(const char* gbase, int64_t ld_bytes, int k0, uint32_t voff_even, uint32_t voff_odd,
                                        uint32_t lds_oper, int wave) {
    const uint32_t voff = (I & 1) ? voff_odd : voff_even;
    if constexpr (!TRANS) {
        const int row = wave * 64 + I * 16;
        dma16(gbase + ((int64_t)row * ld_bytes + (int64_t)k0 * 2), voff, lds_oper + row * 64);
    } else {
        const int k = wave * 8 + I * 2;
        dma16(gbase + (int64_t)(k0 + k) * ld_bytes, voff, lds_oper + k * 512);
    }
}

template <bool TRANS>
struct FragReader {
    uint32_t off[4];  // !TRANS: [ks] (2 used); TRANS: [t]
    __device__ __forceinline__ void init(int lane, int wrow) {
        if constexpr (!TRANS) {
            const int r = lane & 31, g = lane >> 5, swz = (r >> 2) & 3;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) off[ks] = (uint32_t)((wrow + r) * 64 + (((2 * ks + g) ^ swz) << 4));
            off[2] = off[3] = 0;
        } else {
            const int i = lane & 15, grp = lane >> 4, g = grp >> 1, kk = (i >> 2) & 3;
            const int lane_const = (8 * g + (i >> 2)) * 512 + (((wrow >> 3) + 2 * (grp & 1) + ((i & 3) >> 1)) << 4) + 8 * (i & 1);
#pragma unroll
            for (int t = 0; t < 4; ++t) off[t] = (uint32_t)(lane_const + 64 * (t ^ kk));
        }
    }
    template <int T, int KS>
    __device__ __forceinline__ bf16x8_t read(lds_char* oper) const {
        if constexpr (!TRANS) {
            return *(__attribute__((address_space(3))) const bf16x8_t*)(oper + off[KS] + T * 32 * 64);
        } else {
            lds_char* p = oper + off[T] + KS * 16 * 512;
            const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)p);
            const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 4 * 512));
            const s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(bf16x8_t, v);
        }
    }
};

#define CW_PIN() __builtin_amdgcn_sched_barrier(0)

// SPLIT: blockIdx.y selects one of gridDim.y equal slices of every step's k
// range; the block writes its fp32 partial tile to args.partial and
// splitk_reduce_kernel finishes the sum and the epilogue.
// ABL: 0 in every instantiation of the library. The measurement library instantiates the same kernel with one
// part taken out, to price that part (time and energy per launch against the whole kernel; the results of such
// a launch are meaningless): 1 = the k loop issues no operand loads (the ring's stages are filled once, in the
// prologue, and re-used), 2 = no epilogue (nothing is stored), 3 = the k loop reads no fragments from LDS (the
// first tile's stay in the registers).
template <bool TRANS_A, bool TRANS_B, int EPI, int NS, bool SPLIT, typename E, int ABL = 0>
__global__ __launch_bounds__(kThreads) void gemm_bf16_dma_kernel(const RingArgs args) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    lds_char* lds_base = (lds_char*)lds;
    const uint32_t lds_addr0 = (uint32_t)(uintptr_t)lds_base;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    const int M = args.M, N = args.N, K = args.K;
    // M and N need not be tile multiples (but are at least one tile): the last tile of a row or column of
    // tiles is moved back to end at the edge. It overlaps its neighbour, and both compute the shared
    // elements from the same operands in the same order, so the duplicate stores write identical bits.
    const int tiles_m = (M + kTile - 1) / kTile, tiles_n = (N + kTile - 1) / kTile;
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
    int m0 = (first_m + in_group % gsz) * kTile;
    int n0 = (in_group / gsz) * kTile;
    m0 = m0 + kTile > M ? M - kTile : m0;
    n0 = n0 + kTile > N ? N - kTile : n0;

    const int k_len = SPLIT ? K / (int)gridDim.y : K;  // k extent of this block within each step
    const int k_beg = SPLIT ? (int)blockIdx.y * k_len : 0;
    const int k_end = k_beg + k_len;
    const int kt_per_step = k_len / kBK;
    const int k_tail = SPLIT ? 0 : args.k_tail;
    const int KT = kt_per_step * args.n_steps + k_tail / kBK;

    uint32_t a_even, a_odd, b_even, b_odd;
    dma_lane_offsets<TRANS_A>(lane, args.lda, m0, a_even, a_odd);
    dma_lane_offsets<TRANS_B>(lane, args.ldb, n0, b_even, b_odd);
    const int64_t lda_bytes = args.lda * 2, ldb_bytes = args.ldb * 2;

    FragReader<TRANS_A> fa;
    FragReader<TRANS_B> fb;
    fa.init(lane, wm * 128);
    fb.init(lane, wn * 128);

    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // the lane's bias values, fetched ahead of every operand load so that the
    // epilogue finds them in registers
    gemm_bf16::u32x2_t bias_raw[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) bias_raw[j][g] = gemm_bf16::u32x2_t{0u, 0u};
    if (!SPLIT && EPI != CW_EPI_NONE && args.bias != nullptr) {
        const uint16_t* bp = reinterpret_cast<const uint16_t*>(args.bias) + n0 + wn * 128 + 4 * (lane >> 5);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) bias_raw[j][g] = *reinterpret_cast<const gemm_bf16::u32x2_t*>(bp + j * 32 + 8 * g);
    }

    // state of the tile whose loads are issued next. Past the last tile the
    // issue position stays on it: the loop keeps issuing (harmless duplicate
    // loads into a free stage) so that its body has no branches and the load
    // counter arithmetic is the same in every iteration.
    // The eight XCDs walk the flattened (step, k) range cyclically from starting points an eighth of it apart.
    // Walking in step, all 256 workgroups ask memory for the same k slice of B (and the same column slice of
    // A's rows) at the same moment, and when the operands come from HBM rather than from a cache that
    // concentrates the traffic on a few channels (measured: k loop 95 -> 78 us on operands that miss the
    // Infinity Cache). Workgroups of one XCD stay together, so they still share their panels through its L2.
    // The sum of a tile is taken in a rotated order, the same on every launch. Not done where tiles overlap
    // (M or N not a tile multiple): the duplicated elements must come out with identical bits from both tiles.
    const bool cyclic = !SPLIT && k_tail == 0 && (M % kTile) == 0 && (N % kTile) == 0;
    const int kt0 = cyclic ? (int)(((long long)KT * (blockIdx.x & 7)) >> 3) : 0;
    int is_kt = 0, is_step = kt0 / kt_per_step, is_k0 = k_beg + (kt0 % kt_per_step) * kBK, is_stage = 0, is_k_end = k_end;
    const char* is_a = reinterpret_cast<const char*>(gemm_bf16::pick_ptr(args.A, is_step));
    const char* is_b = reinterpret_cast<const char*>(gemm_bf16::pick_ptr(args.B, is_step));
    auto issue_advance = [&]() {
        if (is_kt + 1 < KT) {
            ++is_kt;
            is_k0 += kBK;
            if (is_k0 >= is_k_end) {
                is_k0 = k_beg;
                ++is_step;
                if (cyclic && is_step == args.n_steps) is_step = 0;
                is_a = reinterpret_cast<const char*>(gemm_bf16::pick_ptr(args.A, is_step));
                is_b = reinterpret_cast<const char*>(gemm_bf16::pick_ptr(args.B, is_step));
                if (is_step == args.n_steps) is_k_end = k_beg + k_tail;  // the short extra step
            }
        }
        is_stage = (is_stage + 1 == NS) ? 0 : is_stage + 1;
    };

    // prologue: tiles 0..NS-3 in flight, plus the A part of tile NS-2 (its B part
    // is issued by the first loop iteration, like every later tile's)
    for (int p = 0; p < (ABL == 1 ? NS : NS - 2); ++p) {
        const uint32_t st = lds_addr0 + is_stage * kStageBytes;
        gemm_bf16::static_for<4>([&](auto I) {
            dma_one<TRANS_A, I.value>(is_a, lda_bytes, is_k0, a_even, a_odd, st, wave);
            dma_one<TRANS_B, I.value>(is_b, ldb_bytes, is_k0, b_even, b_odd, st + kOperBytes, wave);
        });
        issue_advance();
    }
    if constexpr (ABL != 1) {
        const uint32_t st = lds_addr0 + is_stage * kStageBytes;
        gemm_bf16::static_for<4>([&](auto I) {
            dma_one<TRANS_A, I.value>(is_a, lda_bytes, is_k0, a_even, a_odd, st, wave);
        });
    }
    if constexpr (ABL == 1) dma_wait<0>();
    else dma_wait<kDmaPerTile*(NS - 3) + 4>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    bf16x8_t af[2][4], bfr[2][4];
    int cur = 0;
    gemm_bf16::static_for<4>([&](auto t) {
        af[0][t.value] = fa.template read<t.value, 0>(lds_base);
        bfr[0][t.value] = fb.template read<t.value, 0>(lds_base + kOperBytes);
        if constexpr (ABL == 3) {
            af[1][t.value] = fa.template read<t.value, 1>(lds_base);
            bfr[1][t.value] = fb.template read<t.value, 1>(lds_base + kOperBytes);
        }
    });

    for (int kt = 0; kt < KT; ++kt) {
        lds_char* sa = lds_base + cur * kStageBytes;
        lds_char* sb = sa + kOperBytes;
        const int nxt = (cur + 1 == NS) ? 0 : cur + 1;
        lds_char* na = lds_base + nxt * kStageBytes;
        lds_char* nb = na + kOperBytes;

        // ---- phase 1: MFMAs of k-step 0; between them the reads of k-step 1 and
        //      the B part of the tile whose A part went out in the previous phase 2
        CW_PIN();
        {
            const uint32_t st = lds_addr0 + is_stage * kStageBytes;
            gemm_bf16::static_for<4>([&](auto i) {
                gemm_bf16::static_for<4>([&](auto j) {
                    constexpr int I = i.value, J = j.value, Q = I * 4 + J;
                    // the 4 x 4 products in serpentine order: consecutive instructions differ in one operand only
                    // (measurably less power than row by row, where every fourth changes both)
                    constexpr int JS = (I & 1) ? 3 - J : J;
                    acc[I][JS] = gemm_bf16::mfma_32x32x16<E>(bfr[0][JS], af[0][I], acc[I][JS]);
                    if constexpr (Q < 4) { if constexpr (ABL != 3) af[1][Q] = fa.template read<Q, 1>(sa); }
                    else if constexpr (Q < 8) { if constexpr (ABL != 3) bfr[1][Q - 4] = fb.template read<Q - 4, 1>(sb); }
                    else if constexpr ((Q & 1) == 0 && ABL != 1) dma_one<TRANS_B, (Q - 8) / 2>(is_b, ldb_bytes, is_k0, b_even, b_odd, st + kOperBytes, wave);
                    CW_PIN();
                });
            });
            issue_advance();
        }

        // ---- mid: tile kt+1 complete for everybody, stage of tile kt-1 free
        dma_wait<kDmaPerTile*(NS - 3)>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        CW_PIN();
        // ---- phase 2: MFMAs of k-step 1; A part of tile kt+NS-1 and reads of (kt+1, k-step 0) between them
        {
            const uint32_t st = lds_addr0 + is_stage * kStageBytes;
            gemm_bf16::static_for<4>([&](auto i) {
                gemm_bf16::static_for<4>([&](auto j) {
                    constexpr int I = i.value, J = j.value, Q = I * 4 + J;
                    constexpr int JS = (I & 1) ? 3 - J : J;
                    acc[I][JS] = gemm_bf16::mfma_32x32x16<E>(bfr[1][JS], af[1][I], acc[I][JS]);
                    if constexpr (Q < 8 && (Q & 1) == 0) { if constexpr (ABL != 1) dma_one<TRANS_A, Q / 2>(is_a, lda_bytes, is_k0, a_even, a_odd, st, wave); }
                    else if constexpr (Q >= 8 && Q < 12) { if constexpr (ABL != 3) af[0][Q - 8] = fa.template read<Q - 8, 0>(na); }
                    else if constexpr (Q >= 12) { if constexpr (ABL != 3) bfr[0][Q - 12] = fb.template read<Q - 12, 0>(nb); }
                    CW_PIN();
                });
            });
        }
        cur = nxt;
    }
    dma_wait<0>();
    __syncthreads();
    if constexpr (SPLIT) {
        // accumulator element 4g+e of tile (i, j): row (lane & 31) + 32 i, column 4 (lane >> 5) + 32 j + 8 g + e
        float* part = args.partial + (int64_t)blockIdx.y * M * N + (int64_t)(m0 + wm * 128 + (lane & 31)) * N + n0 +
                      wn * 128 + 4 * (lane >> 5);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    raw16_t u;
                    u.x = __float_as_uint(acc[i][j][4 * g]);
                    u.y = __float_as_uint(acc[i][j][4 * g + 1]);
                    u.z = __float_as_uint(acc[i][j][4 * g + 2]);
                    u.w = __float_as_uint(acc[i][j][4 * g + 3]);
                    *reinterpret_cast<raw16_t*>(part + (int64_t)i * 32 * N + j * 32 + 8 * g) = u;
                }
    } else if constexpr (ABL == 2) {
        // never true for a launch that got this far: keeps the products alive without storing them
        if (args.n_steps < 0) gemm_bf16::gemm_epilogue_slabs<EPI, E>(acc, args, bias_raw, lds, m0, n0, wm, wn, lane, tid);
    } else {
        gemm_bf16::gemm_epilogue_slabs<EPI, E>(acc, args, bias_raw, lds, m0, n0, wm, wn, lane, tid);
    }
}

template <int NS>
constexpr size_t lds_bytes_dma() {
    const size_t stages = (size_t)NS * kStageBytes;
    const size_t ctile = (size_t)kTile * gemm_bf16::c_pitch<kTile>() * sizeof(uint16_t);
    return stages > ctile ? stages : ctile;
}

inline RingArgs to_ring_args(const GemmArgs& g) {
    RingArgs r = {};
    for (int i = 0; i < g.n_steps && i < kRingMaxSteps; ++i) { r.A[i] = g.A[i]; r.B[i] = g.B[i]; }
    r.k_tail = 0;
    for (int i = 0; i < g.n_addends && i < kRingMaxAddends; ++i) r.addend[i] = g.addend[i];
    r.bias = g.bias; r.C = g.C; r.preact = g.preact;
    r.lda = g.lda; r.ldb = g.ldb; r.ldc = g.ldc; r.ldp = g.ldp; r.ldadd = g.ldadd;
    r.M = g.M; r.N = g.N; r.K = g.K; r.n_steps = g.n_steps; r.n_addends = g.n_addends;
    r.vec_bias = 1; r.vec_add = 1;
    r.partial = nullptr;
    return r;
}

// tail_a / tail_b != nullptr: the extra short step (k extent kBK) that finishes a reduction length which is
// not a multiple of the k tile; gargs.K is then the part covered by the regular steps.
template <bool TA, bool TB, int EPI, int NS, typename E>
int launch_dma_cfg(const GemmArgs& gargs, hipStream_t s, const void* tail_a = nullptr, const void* tail_b = nullptr) {
    RingArgs args = to_ring_args(gargs);
    if (tail_a != nullptr && tail_b != nullptr && gargs.n_steps < kRingMaxSteps) {
        args.A[gargs.n_steps] = tail_a;
        args.B[gargs.n_steps] = tail_b;
        args.k_tail = kBK;
    }
    auto kern = gemm_bf16_dma_kernel<TA, TB, EPI, NS, false, E>;
    constexpr size_t lds = lds_bytes_dma<NS>();
    static_assert(lds <= 160 * 1024, "LDS image does not fit the CU");
    if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)((int)lds), "gemm_bf16_ring"); lrc != CW_OK) return lrc;
    const int tiles = ((args.M + kTile - 1) / kTile) * ((args.N + kTile - 1) / kTile);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, s, args);
    return check_launch("gemm_bf16_dma_kernel");
}

constexpr int kStages = 4;

// Split-k launch: `slices` blocks per output tile, partial sums to the
// caller's scratch. The epilogue is left to splitk_reduce.
template <bool TA, bool TB, typename E>
int launch_dma_split(const GemmArgs& gargs, int slices, hipStream_t s) {
    RingArgs args = to_ring_args(gargs);
    args.partial = reinterpret_cast<float*>(gargs.workspace);
    auto kern = gemm_bf16_dma_kernel<TA, TB, CW_EPI_NONE, kStages, true, E>;
    constexpr size_t lds = lds_bytes_dma<kStages>();
    if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)((int)lds), "gemm_bf16_ring, split"); lrc != CW_OK) return lrc;
    const int tiles = ((args.M + kTile - 1) / kTile) * ((args.N + kTile - 1) / kTile);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid, slices), dim3(kThreads), lds, s, args);
    return check_launch("gemm_bf16_dma_kernel (split k)");
}

template <bool TA, bool TB, typename E>
int launch_dma(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a = nullptr, const void* tail_b = nullptr) {
    switch (epilogue) {
        case CW_EPI_NONE: return launch_dma_cfg<TA, TB, CW_EPI_NONE, kStages, E>(args, s, tail_a, tail_b);
        case CW_EPI_BIAS: return launch_dma_cfg<TA, TB, CW_EPI_BIAS, kStages, E>(args, s, tail_a, tail_b);
        case CW_EPI_BIAS_GELU_TANH: return launch_dma_cfg<TA, TB, CW_EPI_BIAS_GELU_TANH, kStages, E>(args, s, tail_a, tail_b);
        case CW_EPI_BIAS_GELU_ERF: return launch_dma_cfg<TA, TB, CW_EPI_BIAS_GELU_ERF, kStages, E>(args, s, tail_a, tail_b);
        case CW_EPI_BIAS_RELU: return launch_dma_cfg<TA, TB, CW_EPI_BIAS_RELU, kStages, E>(args, s, tail_a, tail_b);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    }
}

}  // namespace gemm_dma
}  // namespace cw
