// Backward of the fused attention core for gfx950 (head size 64, bf16):
// given Q, K, V, O, dO and the forward's log-sum-exp L (natural log),
//   P_ij  = exp(scale q_i.k_j - L_i)              (recomputed, never stored)
//   D_i   = sum_d dO_id O_id
//   dV_j  = sum_i P_ij dO_i
//   dS_ij = P_ij (dO_i.v_j - D_i)
//   dQ_i  = scale sum_j dS_ij k_j,   dK_j = scale sum_i dS_ij q_i
// which is what autograd derives for benchmark/opt/opt.py:84-117 of the
// reference (scaled bmm, mask, softmax, bmm).
//
// Three kernels, no atomics (results are bit-reproducible):
//   attn_delta_kernel : D_i.
//   attn_dq_kernel    : a block owns 256 query rows (64 per wavefront, Q and dO
//                       fragments in registers) and walks the K/V tiles; all
//                       products are formed transposed (lane = query row), so
//                       L_i and D_i are per-lane scalars.
//   attn_dkdv_kernel  : a block owns 256 key rows (64 per wavefront, K and V
//                       fragments in registers) and walks the Q/dO tiles;
//                       products are formed with lane = key row.
// In both, the fp32 probabilities / score gradients of a lane, rounded to
// bf16, are directly the B operand of the next MFMA, and the A operand of
// that MFMA (K^T, Q^T or dO^T) comes from a transposing LDS read of the tile
// that is also read row-wise; the tile is kept in LDS in two images, each
// swizzled for its own read pattern.
#include "cw_common.h"

namespace cw {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) char lds_char;

constexpr int kHead = 64;
constexpr int kThreads = 256;
constexpr int kRowsPerWave = 64;
constexpr int kRowsPerBlock = 4 * kRowsPerWave;
constexpr int kTile = 64;                    // rows of a streamed tile
constexpr int kImage = kTile * kHead * 2;    // 8 KB: one LDS image of a tile
constexpr float kNegBig = -__builtin_huge_valf();

struct BwdArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    const uint16_t* o;
    const uint16_t* d_o;
    const float* lse;
    float* delta;
    uint16_t* dq;
    uint16_t* dk;
    uint16_t* dv;
    int64_t sb, ss, sh;  // q/k/v strides (elements): batch, token, head
    int64_t ob, os, oh;  // o / dO strides
    int64_t gb, gs, gh;  // dq/dk/dv strides
    int S, H, BH, n_blocks;
    float scale, scale_log2e;
    int causal;
};

// Row-image: row r (128 B) holds its 16-byte chunk c at position c ^ ((r >> 1) & 7); read with ds_read_b128.
__device__ __forceinline__ int row_image_offset(int r, int c) { return r * 128 + ((c ^ ((r >> 1) & 7)) << 4); }
// Transpose-image: chunk c of row r inside 32-byte unit (c >> 1) ^ (r & 3); read with ds_read_b64_tr_b16.
__device__ __forceinline__ int tr_image_offset(int r, int c) { return r * 128 + ((((c >> 1) ^ (r & 3)) << 5) | ((c & 1) << 4)); }

// MFMA operand "row = tile row r0 + lane % 32, 8 consecutive d at 16 kb + 8 (lane / 32)" from a row-image.
__device__ __forceinline__ bf16x8_t read_rows(lds_char* img, int r0, int kb, int lane) {
    return *(__attribute__((address_space(3))) const bf16x8_t*)(img + row_image_offset(r0 + (lane & 31), 2 * kb + (lane >> 5)));
}
// MFMA operand "row = d 32 dt + lane % 32, k slots = tile rows r0 + 4 (lane / 32) + {0..3} and + 8" from a
// transpose-image: the transpose of a 16-row slab of the tile.
__device__ __forceinline__ bf16x8_t read_transposed(lds_char* img, int r0, int dt, int lane) {
    const int grp = lane >> 4, i16 = lane & 15;
    const int ra = r0 + 4 * (grp >> 1) + (i16 >> 2);
    const int rb = ra + 8;
    const int unit = 2 * dt + (grp & 1);
    const int off_a = ra * 128 + ((unit ^ (ra & 3)) << 5) + 8 * (i16 & 3);
    const int off_b = rb * 128 + ((unit ^ (rb & 3)) << 5) + 8 * (i16 & 3);
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(img + off_a));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(img + off_b));
    return __builtin_bit_cast(bf16x8_t, (s16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// bf16 B operand from 8 consecutive accumulator elements (k slots j <-> element 8 blk + j).
__device__ __forceinline__ bf16x8_t pack_slots(const float (&x)[16], int blk) {
    bf16x8_t r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (__bf16)x[8 * blk + j];
    return r;
}

// Lane (row = lane % 32, half = lane / 32) holds acc element e = row-major index d = 32 dt + 8 (e / 4) + 4 half + e % 4
// of tile row `row`: write the 64 values of the lane's two accumulators, times `mul`, as bf16.
__device__ __forceinline__ void store_row_pieces(uint16_t* rowp, const f32x16_t (&acc)[2], float mul, int half) {
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint2 w = make_uint2(pack_bf16x2(acc[dt][4 * g] * mul, acc[dt][4 * g + 1] * mul),
                                       pack_bf16x2(acc[dt][4 * g + 2] * mul, acc[dt][4 * g + 3] * mul));
            *reinterpret_cast<uint2*>(rowp + 32 * dt + 8 * g + 4 * half) = w;
        }
}

// ---- D_i = sum_d dO_id O_id : one 8-lane group per (b, h, i) row ------------
__global__ __launch_bounds__(256) void attn_delta_kernel(const BwdArgs a) {
    const int64_t row = (int64_t)blockIdx.x * 32 + (threadIdx.x >> 3);  // (bh, i) flattened
    const int sub = threadIdx.x & 7;
    const int64_t total = (int64_t)a.BH * a.S;
    const int64_t rc = row < total ? row : total - 1;
    const int bh = (int)(rc / a.S);
    const int i = (int)(rc - (int64_t)bh * a.S);
    const int b = bh / a.H, h = bh - b * a.H;
    const int64_t off = b * a.ob + (int64_t)i * a.os + h * a.oh + sub * 8;
    float x[8], y[8];
    unpack_raw(load_raw(a.o + off), x, (const bf16_t*)nullptr);
    unpack_raw(load_raw(a.d_o + off), y, (const bf16_t*)nullptr);
    float s = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s += x[e] * y[e];
    s += dpp_move<kDppXor1>(s);
    s += dpp_move<kDppXor2>(s);
    s += dpp_move<kDppHalfMirror>(s);
    if (sub == 0 && row < total) a.delta[row] = s;
}

// Loader of one 64-row tile: 512 chunks of 16 bytes, two per thread.
struct TileRegs {
    raw16_t r[2];
};
__device__ __forceinline__ void tile_g2r(TileRegs& t, const uint16_t* base, int64_t row_stride, int row0, int S, int tid) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int id = tid + u * kThreads;
        int row = row0 + (id >> 3);
        row = row < S ? row : S - 1;
        t.r[u] = load_raw(base + (int64_t)row * row_stride + (id & 7) * 8);
    }
}
template <bool ROW_IMAGE, bool TR_IMAGE>
__device__ __forceinline__ void tile_r2s(const TileRegs& t, lds_char* row_img, lds_char* tr_img, int tid) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int id = tid + u * kThreads;
        const int r = id >> 3, c = id & 7;
        if (ROW_IMAGE) *(__attribute__((address_space(3))) raw16_t*)(row_img + row_image_offset(r, c)) = t.r[u];
        if (TR_IMAGE) *(__attribute__((address_space(3))) raw16_t*)(tr_img + tr_image_offset(r, c)) = t.r[u];
    }
}

// ---- dQ ---------------------------------------------------------------------
// LDS per stage: K row-image, K transpose-image, V row-image.
__global__ __launch_bounds__(kThreads, 2) void attn_dq_kernel(const BwdArgs a) {
    __shared__ __attribute__((aligned(16))) char lds_raw[2 * 3 * kImage];
    lds_char* lds = (lds_char*)lds_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int S = a.S;
    const int bh = (int)(blockIdx.x % (unsigned)a.BH);
    const int b = bh / a.H, h = bh - b * a.H;
    const int qblk = a.n_blocks - 1 - (int)(blockIdx.x / (unsigned)a.BH);  // longest blocks first
    const int q0 = qblk * kRowsPerBlock;
    const int qw0 = q0 + wave * kRowsPerWave;

    const uint16_t* kp = a.k + b * a.sb + h * a.sh;
    const uint16_t* vp = a.v + b * a.sb + h * a.sh;

    bf16x8_t qf[2][4], dof[2][4];
    float lse2[2], dlt[2];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        int row = qw0 + 32 * qt + l32;
        row = row < S ? row : S - 1;
        const uint16_t* p = a.q + b * a.sb + (int64_t)row * a.ss + h * a.sh + 8 * half;
        const uint16_t* g = a.d_o + b * a.ob + (int64_t)row * a.os + h * a.oh + 8 * half;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            qf[qt][kb] = __builtin_bit_cast(bf16x8_t, load_raw(p + 16 * kb));
            dof[qt][kb] = __builtin_bit_cast(bf16x8_t, load_raw(g + 16 * kb));
        }
        lse2[qt] = a.lse[(int64_t)bh * S + row] * kLog2e;
        dlt[qt] = a.delta[(int64_t)bh * S + row];
    }
    f32x16_t dq[2][2];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) dq[qt][dt][e] = 0.0f;

    int q_hi = q0 + kRowsPerBlock;
    q_hi = q_hi < S ? q_hi : S;
    const int kv_end = a.causal ? q_hi : S;
    const int n_tiles = (kv_end + kTile - 1) / kTile;

    TileRegs kr, vr;
    tile_g2r(kr, kp, a.ss, 0, S, tid);
    tile_g2r(vr, vp, a.ss, 0, S, tid);
    tile_r2s<true, true>(kr, lds, lds + kImage, tid);
    tile_r2s<true, false>(vr, lds + 2 * kImage, nullptr, tid);
    __syncthreads();

    for (int t = 0; t < n_tiles; ++t) {
        lds_char* st_base = lds + (t & 1) * 3 * kImage;
        lds_char* k_rows = st_base;
        lds_char* k_tr = st_base + kImage;
        lds_char* v_rows = st_base + 2 * kImage;
        const int kv0 = t * kTile;
        if (t + 1 < n_tiles) {
            tile_g2r(kr, kp, a.ss, kv0 + kTile, S, tid);
            tile_g2r(vr, vp, a.ss, kv0 + kTile, S, tid);
        }
        const bool active = !a.causal || kv0 <= qw0 + kRowsPerWave - 1;
        if (active) {
            const bool need_mask = (a.causal && kv0 + kTile - 1 > qw0) || kv0 + kTile > S;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                f32x16_t st[2], dpt[2];
#pragma unroll
                for (int qt = 0; qt < 2; ++qt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        st[qt][e] = 0.0f;
                        dpt[qt][e] = 0.0f;
                    }
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) {
                    const bf16x8_t kf = read_rows(k_rows, 32 * kt, kb, lane);
                    const bf16x8_t vf = read_rows(v_rows, 32 * kt, kb, lane);
                    st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[0][kb], st[0], 0, 0, 0);
                    st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[1][kb], st[1], 0, 0, 0);
                    dpt[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, dof[0][kb], dpt[0], 0, 0, 0);
                    dpt[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, dof[1][kb], dpt[1], 0, 0, 0);
                }
                bf16x8_t dsb[2][2];
#pragma unroll
                for (int qt = 0; qt < 2; ++qt) {
                    // element e: key kv0 + 32 kt + 8 (e / 4) + 4 half + e % 4, query qw0 + 32 qt + l32
                    const int qi = qw0 + 32 * qt + l32;
                    float ds[16];
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[qt][e], a.scale_log2e, -lse2[qt]));
                        if (need_mask) {
                            const int kvi = kv0 + 32 * kt + 8 * (e >> 2) + 4 * half + (e & 3);
                            p = ((a.causal && kvi > qi) || kvi >= S) ? 0.0f : p;
                        }
                        ds[e] = p * (dpt[qt][e] - dlt[qt]);
                    }
                    dsb[qt][0] = pack_slots(ds, 0);
                    dsb[qt][1] = pack_slots(ds, 1);
                }
#pragma unroll
                for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt) {
                        const bf16x8_t ktf = read_transposed(k_tr, 32 * kt + 16 * kvb, dt, lane);
                        dq[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf, dsb[0][kvb], dq[0][dt], 0, 0, 0);
                        dq[1][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf, dsb[1][kvb], dq[1][dt], 0, 0, 0);
                    }
            }
        }
        if (t + 1 < n_tiles) {
            lds_char* nx = lds + ((t + 1) & 1) * 3 * kImage;
            tile_r2s<true, true>(kr, nx, nx + kImage, tid);
            tile_r2s<true, false>(vr, nx + 2 * kImage, nullptr, tid);
        }
        __syncthreads();
    }
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        const int qi = qw0 + 32 * qt + l32;
        if (qi < S) store_row_pieces(a.dq + b * a.gb + (int64_t)qi * a.gs + h * a.gh, dq[qt], a.scale, half);
    }
}

// ---- dK, dV -----------------------------------------------------------------
// LDS per stage: Q row-image, Q transpose-image, dO row-image, dO transpose-image, L*log2e and D of the 64 rows.
constexpr int kDkdvStage = 4 * kImage + 2 * kTile * 4;

__global__ __launch_bounds__(kThreads, 1) void attn_dkdv_kernel(const BwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) char lds_dyn[];
    lds_char* lds = (lds_char*)lds_dyn;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int S = a.S;
    const int bh = (int)(blockIdx.x % (unsigned)a.BH);
    const int b = bh / a.H, h = bh - b * a.H;
    const int kvblk = (int)(blockIdx.x / (unsigned)a.BH);  // under the causal mask the first key block is the longest
    const int kvb0 = kvblk * kRowsPerBlock;
    const int kw0 = kvb0 + wave * kRowsPerWave;

    const uint16_t* qp = a.q + b * a.sb + h * a.sh;
    const uint16_t* gp = a.d_o + b * a.ob + h * a.oh;
    const float* lsep = a.lse + (int64_t)bh * S;
    const float* dltp = a.delta + (int64_t)bh * S;

    // K, V fragments of the wavefront's 2 x 32 key rows (B operands: column = key row)
    bf16x8_t kf[2][4], vf[2][4];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
        int row = kw0 + 32 * kt + l32;
        row = row < S ? row : S - 1;
        const uint16_t* pk = a.k + b * a.sb + (int64_t)row * a.ss + h * a.sh + 8 * half;
        const uint16_t* pv = a.v + b * a.sb + (int64_t)row * a.ss + h * a.sh + 8 * half;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            kf[kt][kb] = __builtin_bit_cast(bf16x8_t, load_raw(pk + 16 * kb));
            vf[kt][kb] = __builtin_bit_cast(bf16x8_t, load_raw(pv + 16 * kb));
        }
    }
    f32x16_t dk[2][2], dv[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                dk[kt][dt][e] = 0.0f;
                dv[kt][dt][e] = 0.0f;
            }

    // query tiles: under the causal mask only queries >= the block's first key take part
    const int first_tile = a.causal ? kvb0 / kTile : 0;
    const int n_tiles = (S + kTile - 1) / kTile;

    TileRegs qr, gr;
    float stat = 0.0f;  // threads 0..63: L*log2e of tile row tid; 64..127: D of tile row tid - 64
    auto load_stats = [&](int q0) {
        if (tid < 2 * kTile) {
            int row = q0 + (tid & (kTile - 1));
            row = row < S ? row : S - 1;
            stat = tid < kTile ? lsep[row] * kLog2e : dltp[row];
        }
    };
    auto store_stats = [&](lds_char* stage) {
        if (tid < 2 * kTile) *(__attribute__((address_space(3))) float*)(stage + 4 * kImage + tid * 4) = stat;
    };
    tile_g2r(qr, qp, a.ss, first_tile * kTile, S, tid);
    tile_g2r(gr, gp, a.os, first_tile * kTile, S, tid);
    load_stats(first_tile * kTile);
    tile_r2s<true, true>(qr, lds, lds + kImage, tid);
    tile_r2s<true, true>(gr, lds + 2 * kImage, lds + 3 * kImage, tid);
    store_stats(lds);
    __syncthreads();

    for (int t = first_tile; t < n_tiles; ++t) {
        lds_char* stg = lds + ((t - first_tile) & 1) * kDkdvStage;
        lds_char* q_rows = stg;
        lds_char* q_tr = stg + kImage;
        lds_char* g_rows = stg + 2 * kImage;
        lds_char* g_tr = stg + 3 * kImage;
        const int q0 = t * kTile;
        if (t + 1 < n_tiles) {
            tile_g2r(qr, qp, a.ss, q0 + kTile, S, tid);
            tile_g2r(gr, gp, a.os, q0 + kTile, S, tid);
            load_stats(q0 + kTile);
        }
        // the wavefront's keys kw0 .. kw0+63 see queries >= kw0 only
        const bool active = !a.causal || q0 + kTile - 1 >= kw0;
        if (active) {
            const bool need_mask = (a.causal && q0 < kw0 + kRowsPerWave - 1) || q0 + kTile > S;
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                // row-wise fragments of the 32 query rows (A operands of S and dP)
                bf16x8_t qa[4], ga[4];
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) {
                    qa[kb] = read_rows(q_rows, 32 * qt, kb, lane);
                    ga[kb] = read_rows(g_rows, 32 * qt, kb, lane);
                }
                // L*log2e and D of the lane's 16 query rows: element e <-> row 32 qt + 8 (e / 4) + 4 half + e % 4
                float l2[16], dl[16];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int r = 32 * qt + 8 * g + 4 * half;
                    const f32x4_t x = *(__attribute__((address_space(3))) const f32x4_t*)(stg + 4 * kImage + r * 4);
                    const f32x4_t y = *(__attribute__((address_space(3))) const f32x4_t*)(stg + 4 * kImage + (kTile + r) * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        l2[4 * g + e] = x[e];
                        dl[4 * g + e] = y[e];
                    }
                }
                // transposed fragments of the same rows (A operands of dV^T and dK^T), two 16-row slabs
                bf16x8_t qtf[2][2], gtf[2][2];  // [slab][dt]
#pragma unroll
                for (int sl = 0; sl < 2; ++sl)
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt) {
                        qtf[sl][dt] = read_transposed(q_tr, 32 * qt + 16 * sl, dt, lane);
                        gtf[sl][dt] = read_transposed(g_tr, 32 * qt + 16 * sl, dt, lane);
                    }
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    f32x16_t s_acc, dp_acc;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        s_acc[e] = 0.0f;
                        dp_acc[e] = 0.0f;
                    }
#pragma unroll
                    for (int kb = 0; kb < 4; ++kb) {
                        s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[kb], kf[kt][kb], s_acc, 0, 0, 0);
                        dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ga[kb], vf[kt][kb], dp_acc, 0, 0, 0);
                    }
                    // element e: query q0 + 32 qt + 8 (e / 4) + 4 half + e % 4, key kw0 + 32 kt + l32
                    const int kvi = kw0 + 32 * kt + l32;
                    float p[16], ds[16];
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[e], a.scale_log2e, -l2[e]));
                        if (need_mask) {
                            const int qi = q0 + 32 * qt + 8 * (e >> 2) + 4 * half + (e & 3);
                            pe = ((a.causal && kvi > qi) || qi >= S) ? 0.0f : pe;
                        }
                        p[e] = pe;
                        ds[e] = pe * (dp_acc[e] - dl[e]);
                    }
#pragma unroll
                    for (int sl = 0; sl < 2; ++sl) {
                        const bf16x8_t pb = pack_slots(p, sl);
                        const bf16x8_t dsb = pack_slots(ds, sl);
#pragma unroll
                        for (int dt = 0; dt < 2; ++dt) {
                            dv[kt][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gtf[sl][dt], pb, dv[kt][dt], 0, 0, 0);
                            dk[kt][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qtf[sl][dt], dsb, dk[kt][dt], 0, 0, 0);
                        }
                    }
                }
            }
        }
        if (t + 1 < n_tiles) {
            lds_char* nx = lds + ((t + 1 - first_tile) & 1) * kDkdvStage;
            tile_r2s<true, true>(qr, nx, nx + kImage, tid);
            tile_r2s<true, true>(gr, nx + 2 * kImage, nx + 3 * kImage, tid);
            store_stats(nx);
        }
        __syncthreads();
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
        const int kvi = kw0 + 32 * kt + l32;
        if (kvi < S) {
            store_row_pieces(a.dk + b * a.gb + (int64_t)kvi * a.gs + h * a.gh, dk[kt], a.scale, half);
            store_row_pieces(a.dv + b * a.gb + (int64_t)kvi * a.gs + h * a.gh, dv[kt], 1.0f, half);
        }
    }
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int64_t cw_attn_bwd_workspace_bytes(int64_t B, int64_t H, int64_t S) {
    if (B < 0 || H < 0 || S < 0) return 0;
    return B * H * S * (int64_t)sizeof(float);
}

extern "C" int cw_attn_bwd(int64_t B, int64_t H, int64_t S, int64_t D, const void* q, const void* k, const void* v,
                           int64_t stride_b, int64_t stride_s, int64_t stride_h, const void* out, const void* d_out,
                           int64_t out_stride_b, int64_t out_stride_s, int64_t out_stride_h, const float* lse,
                           float scale, int causal, void* dq, void* dk, void* dv, int64_t grad_stride_b,
                           int64_t grad_stride_s, int64_t grad_stride_h, void* workspace, int64_t workspace_bytes,
                           int io_dtype, void* stream) {
    if (B < 0 || H < 0 || S < 0 || D <= 0)
        return fail(CW_ERR_INVALID, "cw_attn_bwd: bad shape B=%lld H=%lld S=%lld D=%lld", (long long)B, (long long)H, (long long)S, (long long)D);
    if (io_dtype != CW_BF16) return fail(CW_ERR_UNSUPPORTED, "cw_attn_bwd: only bf16 is provided");
    if (D != kHead) return fail(CW_ERR_UNSUPPORTED, "cw_attn_bwd: head size %lld is not provided (64 only)", (long long)D);
    if (B == 0 || H == 0 || S == 0) return CW_OK;
    if (q == nullptr || k == nullptr || v == nullptr || out == nullptr || d_out == nullptr || lse == nullptr ||
        dq == nullptr || dk == nullptr || dv == nullptr || workspace == nullptr)
        return fail(CW_ERR_INVALID, "cw_attn_bwd: null pointer");
    if (workspace_bytes < cw_attn_bwd_workspace_bytes(B, H, S))
        return fail(CW_ERR_INVALID, "cw_attn_bwd: workspace too small (%lld bytes)", (long long)workspace_bytes);
    const int64_t nblk = (S + kRowsPerBlock - 1) / kRowsPerBlock;
    if (S > INT32_MAX / 2 || B * H > (1 << 20) || nblk * B * H > INT32_MAX)
        return fail(CW_ERR_INVALID, "cw_attn_bwd: S or B*H too large");
    const bool aligned = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out) && aligned16(d_out) &&
                         stride_b % 8 == 0 && stride_s % 8 == 0 && stride_h % 8 == 0 && out_stride_b % 8 == 0 &&
                         out_stride_s % 8 == 0 && out_stride_h % 8 == 0 &&
                         ((reinterpret_cast<uintptr_t>(dq) | reinterpret_cast<uintptr_t>(dk) | reinterpret_cast<uintptr_t>(dv)) & 7u) == 0 &&
                         grad_stride_b % 4 == 0 && grad_stride_s % 4 == 0 && grad_stride_h % 4 == 0 &&
                         (reinterpret_cast<uintptr_t>(workspace) & 3u) == 0;
    if (!aligned) return fail(CW_ERR_ALIGNMENT, "cw_attn_bwd: inputs need 16-byte aligned rows, gradients 8-byte aligned rows");
    BwdArgs a;
    a.q = (const uint16_t*)q; a.k = (const uint16_t*)k; a.v = (const uint16_t*)v;
    a.o = (const uint16_t*)out; a.d_o = (const uint16_t*)d_out;
    a.lse = lse; a.delta = (float*)workspace;
    a.dq = (uint16_t*)dq; a.dk = (uint16_t*)dk; a.dv = (uint16_t*)dv;
    a.sb = stride_b; a.ss = stride_s; a.sh = stride_h;
    a.ob = out_stride_b; a.os = out_stride_s; a.oh = out_stride_h;
    a.gb = grad_stride_b; a.gs = grad_stride_s; a.gh = grad_stride_h;
    a.S = (int)S; a.H = (int)H; a.BH = (int)(B * H); a.n_blocks = (int)nblk;
    a.scale = scale; a.scale_log2e = scale * kLog2e;
    a.causal = causal ? 1 : 0;
    hipStream_t s = (hipStream_t)stream;
    const int64_t rows = B * H * S;
    hipLaunchKernelGGL(attn_delta_kernel, dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, s, a);
    int rc = check_launch("attn_delta_kernel");
    if (rc != CW_OK) return rc;
    hipLaunchKernelGGL(attn_dq_kernel, dim3((unsigned)(nblk * B * H)), dim3(kThreads), 0, s, a);
    rc = check_launch("attn_dq_kernel");
    if (rc != CW_OK) return rc;
    constexpr int lds_bytes = 2 * kDkdvStage;
    hipError_t e = hipFuncSetAttribute((const void*)attn_dkdv_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail(CW_ERR_LAUNCH, "hipFuncSetAttribute(attn_dkdv_kernel): %s", hipGetErrorString(e));
    hipLaunchKernelGGL(attn_dkdv_kernel, dim3((unsigned)(nblk * B * H)), dim3(kThreads), lds_bytes, s, a);
    return check_launch("attn_dkdv_kernel");
}
