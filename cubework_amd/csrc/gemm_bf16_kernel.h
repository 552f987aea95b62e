// SUMMA block GEMM for gfx950: C = act(sum_i op(A_i) op(B_i) + addends + bias),
// 16-bit operands (bf16, or fp16 with E = f16_t: the same kernels, another MFMA opcode and conversion),
// fp32 accumulation in v_mfma_f32_32x32x16_bf16 / _f16.
//
// Shape of the kernel
//   - one 256-thread block (4 wavefronts, 2x2) per BM x BN tile of C; a
//     wavefront owns a (BM/2) x (BN/2) sub-tile as TM x TN MFMA tiles of 32x32
//     (256x256 block: 4x4 tiles = 256 fp32 accumulators per lane);
//   - the k loop runs over (step, k) flattened into tiles of 64, so the software
//     pipeline does not drain where one k-step's operands end and the next
//     step's (a different allocation) begin;
//   - global -> registers -> LDS with the next tile's loads in flight during the
//     current tile's MFMAs, two LDS stages, one barrier per tile;
//   - both operands sit in LDS as [row][k] with k contiguous (pitch 72 elements
//     = 144 bytes, which spreads eight consecutive rows over all banks for the
//     16-byte fragment reads). An operand whose memory has k as the slow index
//     (B of NN, both of TN) is transposed in registers on its way to LDS: each
//     thread owns an 8x8 block;
//   - the MFMA is issued with the B fragment as srcA and the A fragment as
//     srcB, so a lane ends up with four consecutive output COLUMNS per register
//     quad; the epilogue packs them and stages the tile through LDS so that
//     global stores are whole rows of the tile;
//   - workgroup ids are remapped so that the 8 XCDs (ids are dealt round-robin
//     to them) each work on a compact patch of tiles and share A/B panels in
//     their own L2.
#pragma once

#include <type_traits>
#include <utility>

#include "cw_common.h"
#include "gemm.h"

namespace cw {

namespace gemm_bf16 {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
// Staging registers use the native vector type: struct uint4 copies between
// address spaces become memcpy calls that keep the array in scratch memory.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

// acc += a b for the element type E; fragments travel as 8 x 16 bits whatever the type.
template <typename E>
__device__ __forceinline__ f32x16_t mfma_32x32x16(bf16x8_t a, bf16x8_t b, f32x16_t acc) {
    if constexpr (std::is_same<E, f16_t>::value)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), acc, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}

// Compile-time loop: f(std::integral_constant<int, I>) for I in [0, N).
template <int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// tab[idx] without dynamic indexing: a dynamically indexed member keeps the
// whole kernel-argument struct in scratch memory, and then every field (the
// leading dimensions, the operand pointers) is read back through vector
// loads and counts as lane-varying.
template <int N>
__device__ __forceinline__ const void* pick_ptr(const void* const (&tab)[N], int idx) {
    const void* p = tab[0];
    static_for<N>([&](auto i) {
        if (idx == i.value) p = tab[i.value];
    });
    return p;
}

constexpr int kBK = 64;         // k extent of an LDS tile
constexpr int kPitch = 72;      // elements per LDS row (64 + 8 padding)
constexpr int kThreads = 256;

// Eight consecutive bf16 of row r starting at column c of a row-major
// [rmax][cmax] operand; zero outside. vec_ok: rows are 16-byte aligned.
__device__ __forceinline__ u32x4_t load8_guarded(const uint16_t* __restrict__ base, int64_t ld, int r, int c, int rmax,
                                               int cmax, bool vec_ok) {
    u32x4_t out = {0u, 0u, 0u, 0u};
    if (r >= rmax || c >= cmax) return out;
    const uint16_t* p = base + (int64_t)r * ld + c;
    if (vec_ok && c + 8 <= cmax) return *reinterpret_cast<const u32x4_t*>(p);
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < 8; ++e)
        if (c + e < cmax) w[e >> 1] |= (uint32_t)p[e] << ((e & 1) * 16);
    return u32x4_t{w[0], w[1], w[2], w[3]};
}

// Global -> registers for a ROWS x 64 operand tile.
//   TRANS == false: memory is [rows][k] (k contiguous). 16-byte chunk c of the
//     tile is (row c/8, k-chunk c%8); thread handles chunks tid, tid+256, ...
//   TRANS == true : memory is [k][rows] (rows contiguous). Thread owns the 8x8
//     block (k-block tid%8, row-block tid/8) and loads its 8 k-rows.
template <int ROWS, bool TRANS, bool GUARD>
__device__ __forceinline__ void tile_g2r(u32x4_t (&reg)[8], const uint16_t* __restrict__ base, int64_t ld, int row0,
                                         int k0, int rmax, int kmax, int tid, bool vec_ok) {
    if constexpr (!TRANS) {
        constexpr int CH = ROWS * 8 / kThreads;
#pragma unroll
        for (int it = 0; it < CH; ++it) {
            const int c = it * kThreads + tid;
            const int row = row0 + (c >> 3);
            const int k = k0 + (c & 7) * 8;
            if constexpr (GUARD)
                reg[it] = load8_guarded(base, ld, row, k, rmax, kmax, vec_ok);
            else
                reg[it] = *reinterpret_cast<const u32x4_t*>(base + (int64_t)row * ld + k);
        }
    } else {
        const int kb = tid & 7;
        const int rb = tid >> 3;
        if (rb < ROWS / 8) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int k = k0 + kb * 8 + j;
                const int row = row0 + rb * 8;
                if constexpr (GUARD)
                    reg[j] = load8_guarded(base, ld, k, row, kmax, rmax, vec_ok);
                else
                    reg[j] = *reinterpret_cast<const u32x4_t*>(base + (int64_t)k * ld + row);
            }
        }
    }
}

// Fast-path variant of tile_g2r for in-bounds, 16-byte aligned tiles: the
// address is (uniform base of the tile row block) + (one 32-bit per-thread byte
// offset `voff`, invariant over the k loop), so the loads use the scalar-base
// addressing form and need no per-load address registers.
//   TRANS == false: voff = ((row0 + tid/8) * ld + (tid%8)*8) * 2
//   TRANS == true : voff = (((tid%8)*8) * ld + row0 + (tid/8)*8) * 2
template <int ROWS, bool TRANS>
__device__ __forceinline__ void tile_g2r_fast(u32x4_t (&reg)[8], const char* __restrict__ base, uint32_t voff,
                                              int64_t ld_bytes, int k0, int tid) {
    if constexpr (!TRANS) {
        constexpr int CH = ROWS * 8 / kThreads;
        static_for<CH>([&](auto it) {
            const char* p = base + ((int64_t)it.value * 32 * ld_bytes + (int64_t)k0 * 2);
            reg[it.value] = *reinterpret_cast<const u32x4_t*>(p + voff);
        });
    } else {
        if ((tid >> 3) < ROWS / 8) {
            static_for<8>([&](auto j) {
                const char* p = base + (int64_t)(k0 + j.value) * ld_bytes;
                reg[j.value] = *reinterpret_cast<const u32x4_t*>(p + voff);
            });
        }
    }
}

__device__ __forceinline__ uint32_t pick_lo(uint32_t a, uint32_t b) { return (a & 0xffffu) | (b << 16); }
__device__ __forceinline__ uint32_t pick_hi(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xffff0000u); }

// Registers -> LDS tile [ROWS][kPitch].
template <int ROWS, bool TRANS>
__device__ __forceinline__ void tile_r2s(const u32x4_t (&reg)[8], uint16_t* __restrict__ lds, int tid) {
    if constexpr (!TRANS) {
        constexpr int CH = ROWS * 8 / kThreads;
        static_for<CH>([&](auto it) {
            const int c = it.value * kThreads + tid;
            *reinterpret_cast<u32x4_t*>(lds + (c >> 3) * kPitch + (c & 7) * 8) = reg[it.value];
        });
    } else {
        const int kb = tid & 7;
        const int rb = tid >> 3;
        if (rb < ROWS / 8) {
            // reg[j] = 8 rows' values at k-row j; dword d of it = rows (2d, 2d+1).
            // out(row i) dword d' = (k = 2d', 2d'+1) of row i.
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                uint32_t w[4];
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const u32x4_t ra = reg[2 * d];
                    const u32x4_t rb4 = reg[2 * d + 1];
                    const uint32_t a = (i >> 1) == 0 ? ra.x : (i >> 1) == 1 ? ra.y : (i >> 1) == 2 ? ra.z : ra.w;
                    const uint32_t b = (i >> 1) == 0 ? rb4.x : (i >> 1) == 1 ? rb4.y : (i >> 1) == 2 ? rb4.z : rb4.w;
                    w[d] = (i & 1) ? pick_hi(a, b) : pick_lo(a, b);
                }
                *reinterpret_cast<u32x4_t*>(lds + (rb * 8 + i) * kPitch + kb * 8) = u32x4_t{w[0], w[1], w[2], w[3]};
            }
        }
    }
}

template <int EPI>
__device__ __forceinline__ float epi_act(float x) {
    if constexpr (EPI == CW_EPI_BIAS_GELU_TANH) return gelu_tanh(x);
    if constexpr (EPI == CW_EPI_BIAS_GELU_ERF) return gelu_erf(x);
    if constexpr (EPI == CW_EPI_BIAS_RELU) return x < 0.0f ? 0.0f : x;  // NaN stays NaN, as torch.relu leaves it
    return x;
}

template <typename E>
__device__ __forceinline__ void load4_half(const uint16_t* __restrict__ p, int n_valid, bool vec_ok, float (&v)[4]) {
    if (vec_ok && n_valid >= 4) {
        const u32x2_t u = *reinterpret_cast<const u32x2_t*>(p);
        v[0] = half_conv<E>::lo(u.x);
        v[1] = half_conv<E>::hi(u.x);
        v[2] = half_conv<E>::lo(u.y);
        v[3] = half_conv<E>::hi(u.y);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = e < n_valid ? half_conv<E>::one(p[e]) : 0.0f;
    }
}

// LDS image of the output tile: [BM][BN + 8] bf16. The 528-byte (BN = 256)
// pitch keeps rows 16-byte aligned for the row-wise readout and spreads the
// 8-byte writes of 16 consecutive rows over 16 different 16-byte bank groups.
template <int BN>
constexpr int c_pitch() { return BN + 8; }

// Write the staged tile out row by row: 16 bytes per lane, a wavefront covers
// whole 512-byte rows (BN = 256), so global stores are full cache lines.
template <int BM, int BN, bool FAST>
__device__ __forceinline__ void tile_store(const uint16_t* __restrict__ lds_c, uint16_t* __restrict__ C, int64_t ldc,
                                           int m0, int n0, int M, int N, int tid) {
    constexpr int CP = c_pitch<BN>();
    constexpr int CHUNKS_PER_ROW = BN / 8;
    constexpr int TOTAL = BM * CHUNKS_PER_ROW;
    if constexpr (FAST) {
        // whole tile in bounds, rows 16-byte aligned: thread -> (row q/32.., chunk q%32), no checks
        uint16_t* base = C + (int64_t)(m0 + tid / CHUNKS_PER_ROW) * ldc + n0 + (tid % CHUNKS_PER_ROW) * 8;
        const uint16_t* src = lds_c + (tid / CHUNKS_PER_ROW) * CP + (tid % CHUNKS_PER_ROW) * 8;
        constexpr int ROWS_PER_PASS = kThreads / CHUNKS_PER_ROW;
#pragma unroll 8
        for (int pass = 0; pass < BM / ROWS_PER_PASS; ++pass)
            *reinterpret_cast<u32x4_t*>(base + (int64_t)pass * ROWS_PER_PASS * ldc) =
                *reinterpret_cast<const u32x4_t*>(src + pass * ROWS_PER_PASS * CP);
        return;
    }
    const bool vec16 = ((reinterpret_cast<uintptr_t>(C) & 15u) == 0) && ((ldc & 7) == 0);
#pragma unroll 4
    for (int q = tid; q < TOTAL; q += kThreads) {
        const int r = q / CHUNKS_PER_ROW;
        const int cq = q % CHUNKS_PER_ROW;
        const int row = m0 + r;
        const int col = n0 + cq * 8;
        if (row < M && col < N) {
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(lds_c + r * CP + cq * 8);
            uint16_t* dst = C + (int64_t)row * ldc + col;
            if (vec16 && col + 8 <= N) {
                *reinterpret_cast<u32x4_t*>(dst) = v;
            } else {
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (col + i < N) dst[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
            }
        }
    }
}

// Epilogue shared by the block-GEMM kernels: value = acc + addends + bias,
// optionally stored as the pre-activation, then activation, bf16 packing,
// staging of the tile in LDS (which must be free: all waves past their last
// operand read) and row-wise stores. The accumulators are only read (one
// 32x32 MFMA tile at a time), never written back.
// acc[i][j][v]: row  m = m0 + wm*(BM/2) + i*32 + (lane & 31)
//               col  n = n0 + wn*(BN/2) + j*32 + 8*(v/4) + 4*(lane>>5) + (v%4)
// FAST: the tile is entirely in bounds and every pointer / leading dimension
// allows the vector accesses (checked on the host): no per-element guards.
template <int BM, int BN, int TM, int TN, int EPI, bool FAST, typename E, typename Args>
__device__ __forceinline__ void gemm_epilogue(f32x16_t (&acc)[TM][TN], const Args& args, uint16_t* lds, int m0,
                                              int n0, int wm, int wn, int lane, int tid) {
    constexpr int WTM = BM / 2, WTN = BN / 2;
    constexpr int CP = c_pitch<BN>();
    const int M = args.M, N = args.N;
    uint16_t* lds_c = lds;
    const int row_l = wm * WTM + (lane & 31);
    const int col_l = wn * WTN + 4 * (lane >> 5);
    const uint16_t* bias = reinterpret_cast<const uint16_t*>(args.bias);
    const bool use_bias = (EPI != CW_EPI_NONE) && bias != nullptr;

    auto stage_tile = [&](auto activated) {
        constexpr bool ACT = decltype(activated)::value;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            float bv[4][4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int ncol = n0 + col_l + j * 32 + 8 * g;
                if (use_bias && (FAST || ncol < N)) {
                    load4_half<E>(bias + ncol, FAST ? 4 : N - ncol, FAST || args.vec_bias != 0, bv[g]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) bv[g][e] = 0.0f;
                }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int mrow = m0 + row_l + i * 32;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int ncol = n0 + col_l + j * 32 + 8 * g;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * g + e] + bv[g][e];
                    if (args.n_addends > 0 && (FAST || (mrow < M && ncol < N))) {
#pragma unroll 1
                        for (int a = 0; a < args.n_addends; ++a) {
                            float t[4];
                            load4_half<E>(reinterpret_cast<const uint16_t*>(pick_ptr(args.addend, a)) + (int64_t)mrow * args.ldadd + ncol,
                                          FAST ? 4 : N - ncol, FAST || args.vec_add != 0, t);
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] += t[e];
                        }
                    }
                    if constexpr (ACT) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = epi_act<EPI>(v[e]);
                    }
                    u32x2_t p;
                    p.x = half_conv<E>::pack2(v[0], v[1]);
                    p.y = half_conv<E>::pack2(v[2], v[3]);
                    *reinterpret_cast<u32x2_t*>(lds_c + (row_l + i * 32) * CP + col_l + j * 32 + 8 * g) = p;
                }
            }
        }
    };

    if (args.preact != nullptr) {
        stage_tile(std::false_type{});
        __syncthreads();
        tile_store<BM, BN, FAST>(lds_c, reinterpret_cast<uint16_t*>(args.preact), args.ldp, m0, n0, M, N, tid);
        __syncthreads();
    }
    stage_tile(std::true_type{});
    __syncthreads();
    tile_store<BM, BN, FAST>(lds_c, reinterpret_cast<uint16_t*>(args.C), args.ldc, m0, n0, M, N, tid);
}

// Epilogue of the 256x256 LDS-DMA kernel (whole tile in bounds, aligned): the
// tile goes out in four slabs of 2 x 32 rows (accumulator row index i of both
// wavefront rows), staged through two alternating LDS buffers. The global
// stores of slab i drain while slab i+1 is computed, and one barrier per slab
// is enough: a buffer is rewritten two slabs after it was read.
// bias_raw[j][g]: the lane's 4 bias values (bf16 pairs) for accumulator
// columns j*32 + 8g .. +3, loaded by the caller ahead of the k loop.
template <int EPI, typename E, typename Args>
__device__ __forceinline__ void gemm_epilogue_slabs(f32x16_t (&acc)[4][4], const Args& args,
                                                    const u32x2_t (&bias_raw)[4][4], uint16_t* lds, int m0, int n0,
                                                    int wm, int wn, int lane, int tid) {
    constexpr int CP = c_pitch<256>();
    constexpr int BUF = 64 * CP;  // elements per staging buffer
    const int lrow = wm * 32 + (lane & 31);
    const int col_l = wn * 128 + 4 * (lane >> 5);
    int buf = 0;

    auto stage = [&](auto slab, auto activated) {
        constexpr int I = decltype(slab)::value;
        constexpr bool ACT = decltype(activated)::value;
        const int mrow = m0 + wm * 128 + I * 32 + (lane & 31);
        uint16_t* dst = lds + buf * BUF + lrow * CP + col_l;
        // the first addend's 16 pieces of this slab are requested together, ahead of the arithmetic (a load in
        // front of each use would expose its latency sixteen times); further addends, rare, are read where used
        u32x2_t add0[4][4];
        if (args.n_addends > 0) {
            const uint16_t* ap = reinterpret_cast<const uint16_t*>(pick_ptr(args.addend, 0)) + (int64_t)mrow * args.ldadd + n0 + col_l;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) add0[j][g] = *reinterpret_cast<const u32x2_t*>(ap + j * 32 + 8 * g);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x2_t b = bias_raw[j][g];
                float v[4];
                v[0] = acc[I][j][4 * g] + half_conv<E>::lo(b.x);
                v[1] = acc[I][j][4 * g + 1] + half_conv<E>::hi(b.x);
                v[2] = acc[I][j][4 * g + 2] + half_conv<E>::lo(b.y);
                v[3] = acc[I][j][4 * g + 3] + half_conv<E>::hi(b.y);
                if (args.n_addends > 0) {
                    const int ncol = n0 + col_l + j * 32 + 8 * g;
                    v[0] += half_conv<E>::lo(add0[j][g].x);
                    v[1] += half_conv<E>::hi(add0[j][g].x);
                    v[2] += half_conv<E>::lo(add0[j][g].y);
                    v[3] += half_conv<E>::hi(add0[j][g].y);
#pragma unroll 1
                    for (int a = 1; a < args.n_addends; ++a) {
                        float t[4];
                        load4_half<E>(reinterpret_cast<const uint16_t*>(pick_ptr(args.addend, a)) + (int64_t)mrow * args.ldadd + ncol,
                                      4, true, t);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] += t[e];
                    }
                }
                if constexpr (ACT) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = epi_act<EPI>(v[e]);
                }
                u32x2_t p;
                p.x = half_conv<E>::pack2(v[0], v[1]);
                p.y = half_conv<E>::pack2(v[2], v[3]);
                *reinterpret_cast<u32x2_t*>(dst + j * 32 + 8 * g) = p;
            }
        }
    };
    // 64 staged rows x 32 chunks of 16 bytes: 8 per thread, whole 512-byte rows per wavefront pass
    auto store = [&](int slab, uint16_t* out, int64_t ld) {
        const int r = tid >> 5, cq = tid & 31;
        const uint16_t* src = lds + buf * BUF + r * CP + cq * 8;
#pragma unroll
        for (int pass = 0; pass < 8; ++pass) {
            const int lr = r + 8 * pass;
            const int grow = m0 + (lr >= 32 ? 128 : 0) + slab * 32 + (lr & 31);
            *reinterpret_cast<u32x4_t*>(out + (int64_t)grow * ld + n0 + cq * 8) =
                *reinterpret_cast<const u32x4_t*>(src + pass * 8 * CP);
        }
    };
    static_for<4>([&](auto slab) {
        if (args.preact != nullptr) {
            stage(slab, std::false_type{});
            __syncthreads();
            store(decltype(slab)::value, reinterpret_cast<uint16_t*>(args.preact), args.ldp);
            buf ^= 1;
        }
        stage(slab, std::true_type{});
        __syncthreads();
        store(decltype(slab)::value, reinterpret_cast<uint16_t*>(args.C), args.ldc);
        buf ^= 1;
    });
}

template <int BM, int BN, bool TRANS_A, bool TRANS_B, bool GUARD, int EPI, typename E>
__global__ __launch_bounds__(kThreads) void gemm_bf16_kernel(const GemmArgs args) {
    constexpr int WTM = BM / 2, WTN = BN / 2;  // wavefront sub-tile
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_ELEMS = BM * kPitch, B_ELEMS = BN * kPitch;
    constexpr int STAGE = A_ELEMS + B_ELEMS;
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const int M = args.M, N = args.N, K = args.K;
    const int tiles_m = (M + BM - 1) / BM;
    const int tiles_n = (N + BN - 1) / BN;
    const int total = tiles_m * tiles_n;
    // XCD-aware remap: ids pid, pid+8, ... share an XCD; give each XCD a
    // contiguous range of tile ids, and order tile ids in groups of 8 tile rows.
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
    const int tile_m = first_m + in_group % gsz;
    const int tile_n = in_group / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int kt_per_step = (K + kBK - 1) / kBK;
    const int KT = kt_per_step * args.n_steps;
    const bool vec_a = args.vec_a != 0, vec_b = args.vec_b != 0;

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    u32x4_t ra[8], rb[8];
    // fragment read offsets (elements) within a stage
    const int a_frag = (wm * WTM + (lane & 31)) * kPitch + (lane >> 5) * 8;
    const int b_frag = A_ELEMS + (wn * WTN + (lane & 31)) * kPitch + (lane >> 5) * 8;

    // fast path: per-thread byte offsets that do not change over the k loop
    const uint32_t a_voff =
        TRANS_A ? (uint32_t)((((tid & 7) * 8) * args.lda + m0 + (tid >> 3) * 8) * 2)
                : (uint32_t)(((m0 + (tid >> 3)) * args.lda + (tid & 7) * 8) * 2);
    const uint32_t b_voff =
        TRANS_B ? (uint32_t)((((tid & 7) * 8) * args.ldb + n0 + (tid >> 3) * 8) * 2)
                : (uint32_t)(((n0 + (tid >> 3)) * args.ldb + (tid & 7) * 8) * 2);

    auto issue_loads = [&](int kt) {
        const int step = kt / kt_per_step;
        const int k0 = (kt - step * kt_per_step) * kBK;
        if constexpr (GUARD) {
            const uint16_t* Ap = reinterpret_cast<const uint16_t*>(args.A[step]);
            const uint16_t* Bp = reinterpret_cast<const uint16_t*>(args.B[step]);
            tile_g2r<BM, TRANS_A, true>(ra, Ap, args.lda, m0, k0, M, K, tid, vec_a);
            tile_g2r<BN, TRANS_B, true>(rb, Bp, args.ldb, n0, k0, N, K, tid, vec_b);
        } else {
            tile_g2r_fast<BM, TRANS_A>(ra, reinterpret_cast<const char*>(args.A[step]), a_voff, args.lda * 2, k0, tid);
            tile_g2r_fast<BN, TRANS_B>(rb, reinterpret_cast<const char*>(args.B[step]), b_voff, args.ldb * 2, k0, tid);
        }
    };
    auto commit_loads = [&](int stage) {
        uint16_t* s = lds + stage * STAGE;
        tile_r2s<BM, TRANS_A>(ra, s, tid);
        tile_r2s<BN, TRANS_B>(rb, s + A_ELEMS, tid);
    };

    if (KT > 0) {
        issue_loads(0);
        commit_loads(0);
    }
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) issue_loads(kt + 1);
        const uint16_t* s = lds + cur * STAGE;
        // fragments of k-step ks+1 are read from LDS while the MFMAs of step ks run
        bf16x8_t af[2][TM], bfr[2][TN];
        auto read_frags = [&](int ks, int set) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[set][i] = *reinterpret_cast<const bf16x8_t*>(s + a_frag + i * 32 * kPitch + ks * 16);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bfr[set][j] = *reinterpret_cast<const bf16x8_t*>(s + b_frag + j * 32 * kPitch + ks * 16);
        };
        read_frags(0, 0);
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            if (ks + 1 < kBK / 16) read_frags(ks + 1, (ks + 1) & 1);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = mfma_32x32x16<E>(bfr[ks & 1][j], af[ks & 1][i], acc[i][j]);
        }
        if (kt + 1 < KT) commit_loads(cur ^ 1);
        __syncthreads();
    }

    gemm_epilogue<BM, BN, TM, TN, EPI, !GUARD, E>(acc, args, lds, m0, n0, wm, wn, lane, tid);
}

template <int BM, int BN>
constexpr size_t lds_bytes() {
    const size_t stages = 2u * (BM + BN) * kPitch * sizeof(uint16_t);
    const size_t ctile = (size_t)BM * c_pitch<BN>() * sizeof(uint16_t);
    return stages > ctile ? stages : ctile;
}

template <int BM, int BN, bool TA, bool TB, bool GUARD, int EPI, typename E>
int launch_cfg(const GemmArgs& args, hipStream_t s) {
    auto kern = gemm_bf16_kernel<BM, BN, TA, TB, GUARD, EPI, E>;
    constexpr size_t lds = lds_bytes<BM, BN>();
    static_assert(lds <= 160 * 1024, "LDS tile does not fit the CU");
    if (lds > 48 * 1024) {
        if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)((int)lds), "gemm_bf16"); lrc != CW_OK) return lrc;
    }
    const int tiles = ((args.M + BM - 1) / BM) * ((args.N + BN - 1) / BN);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, s, args);
    return check_launch("gemm_bf16_kernel");
}

template <int BM, int BN, bool TA, bool TB, bool GUARD, typename E>
int launch_epi(const GemmArgs& args, int epilogue, hipStream_t s) {
    switch (epilogue) {
        case CW_EPI_NONE: return launch_cfg<BM, BN, TA, TB, GUARD, CW_EPI_NONE, E>(args, s);
        case CW_EPI_BIAS: return launch_cfg<BM, BN, TA, TB, GUARD, CW_EPI_BIAS, E>(args, s);
        case CW_EPI_BIAS_GELU_TANH: return launch_cfg<BM, BN, TA, TB, GUARD, CW_EPI_BIAS_GELU_TANH, E>(args, s);
        case CW_EPI_BIAS_GELU_ERF: return launch_cfg<BM, BN, TA, TB, GUARD, CW_EPI_BIAS_GELU_ERF, E>(args, s);
        case CW_EPI_BIAS_RELU: return launch_cfg<BM, BN, TA, TB, GUARD, CW_EPI_BIAS_RELU, E>(args, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    }
}

// All tile configurations of one operand orientation. `big` selects 256x256
// tiles, `exact` the unguarded kernels (tile-multiple, 16-byte aligned shapes).
template <bool TA, bool TB, typename E>
int launch_orientation(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s) {
    if (big)
        return exact ? launch_epi<256, 256, TA, TB, false, E>(args, epilogue, s)
                     : launch_epi<256, 256, TA, TB, true, E>(args, epilogue, s);
    return exact ? launch_epi<128, 128, TA, TB, false, E>(args, epilogue, s)
                 : launch_epi<128, 128, TA, TB, true, E>(args, epilogue, s);
}

}  // namespace gemm_bf16

// One translation unit per orientation and element type (gemm_bf16_nn/nt/tn.hip, gemm_f16_nn/nt/tn.hip).
int gemm_bf16_launch_nn(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s);
int gemm_bf16_launch_nt(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s);
int gemm_bf16_launch_tn(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s);
int gemm_f16_launch_nn(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s);
int gemm_f16_launch_nt(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s);
int gemm_f16_launch_tn(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s);

}  // namespace cw
