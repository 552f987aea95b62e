// Fused causal attention core for gfx950, head size 64, bf16:
//   O = softmax(scale * Q K^T + causal mask) V        per (batch, head)
// (benchmark/opt/opt.py:81-117 of the reference: scaled bmm, additive mask,
// softmax, bmm). One pass over K/V per block of queries with a running
// (max, sum) per query row; the score matrix never leaves registers.
//
// Everything is computed transposed so that a lane owns ONE query row:
//   S^T[kv, q] = K[kv, :] . Q[q, :]      v_mfma_f32_32x32x16_bf16, A = K, B = Q
//   O^T[d, q] += V^T[d, kv] . P^T[kv, q]                           A = V^T, B = P^T
// The MFMA result layout puts query q = lane % 32 in every lane: row maxima
// and sums are in-lane reductions over the lane's 16 kv values plus one
// exchange with lane ^ 32, the rescaling of O^T is a per-lane multiply, and
// the fp32 scores of a lane, rounded to bf16, are exactly the B operand of
// the second product (the reduction index kv may be permuted freely as long
// as the A operand uses the same permutation, which the transposing LDS
// read of V provides).
//
// Block = 4 wavefronts x 64 query rows; K/V tiles of 64 rows are staged in
// LDS (two stages, register prefetch of the next tile), K as [kv][d] read with
// ds_read_b128, V as [kv][d] read with ds_read_b64_tr_b16. Two blocks are
// resident per compute unit so that one wavefront's softmax arithmetic
// overlaps another's MFMAs.
#include "cw_common.h"

namespace cw {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) char lds_char;

constexpr int kHead = 64;            // head size
constexpr int kAttnThreads = 256;    // 4 wavefronts
constexpr int kQPerWave = 64;        // two 32-row query tiles per wavefront
constexpr int kQPerBlock = 4 * kQPerWave;
constexpr int kKvTile = 64;          // K/V rows per LDS stage
constexpr int kTileBytes = kKvTile * kHead * 2;  // 8 KB per operand per stage
constexpr float kNegBig = -__builtin_huge_valf();

struct AttnArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* o;
    float* lse;
    int64_t sb, ss, sh;     // q/k/v strides (elements): batch, token, head
    int64_t ob, os, oh;     // output strides
    int S, H, BH, n_qblocks;
    float scale_log2e;      // scale * log2(e)
    int causal;
};

// K tile in LDS: row r (128 B) holds its 16-byte chunk c at position c ^ ((r >> 1) & 7).
__device__ __forceinline__ int k_lds_offset(int r, int c) { return r * 128 + ((c ^ ((r >> 1) & 7)) << 4); }
// V tile in LDS: row r holds its 16-byte chunk c inside 32-byte unit (c >> 1) ^ (r & 3).
__device__ __forceinline__ int v_lds_offset(int r, int c) { return r * 128 + ((((c >> 1) ^ (r & 3)) << 5) | ((c & 1) << 4)); }

__device__ __forceinline__ float xchg32(float v) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute((int)(((threadIdx.x & 63) ^ 32) << 2), __float_as_int(v)));
}

__global__ __launch_bounds__(kAttnThreads, 2) void attn_fwd_kernel(const AttnArgs a) {
    __shared__ __attribute__((aligned(16))) char lds_raw[2 * 2 * kTileBytes];
    lds_char* lds = (lds_char*)lds_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int half = lane >> 5;
    const int l32 = lane & 31;
    const int S = a.S;
    // 1-D grid, all (batch, head) pairs of the last query block first: under the causal mask a block's
    // work grows with its query position, and the longest blocks must not be the last to start
    const int bh = (int)(blockIdx.x % (unsigned)a.BH);
    const int b = bh / a.H, h = bh - b * a.H;
    const int qblk = a.n_qblocks - 1 - (int)(blockIdx.x / (unsigned)a.BH);
    const int q0 = qblk * kQPerBlock;
    const int qw0 = q0 + wave * kQPerWave;

    const uint16_t* qp = a.q + b * a.sb + h * a.sh;
    const uint16_t* kp = a.k + b * a.sb + h * a.sh;
    const uint16_t* vp = a.v + b * a.sb + h * a.sh;

    // Q fragments (B operand): lane = query row l32 of tile qt, 8 d-values at 16 kb + 8 half
    bf16x8_t qf[2][4];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        int row = qw0 + 32 * qt + l32;
        row = row < S ? row : S - 1;
        const uint16_t* p = qp + (int64_t)row * a.ss + 8 * half;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) qf[qt][kb] = __builtin_bit_cast(bf16x8_t, load_raw(p + 16 * kb));
    }

    f32x16_t oacc[2][2];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[qt][dt][e] = 0.0f;
    float m_run[2] = {kNegBig, kNegBig};  // running maximum of scale*log2e*s
    float l_run[2] = {0.0f, 0.0f};        // this lane's share of the running sum

    int q_hi = q0 + kQPerBlock;
    q_hi = q_hi < S ? q_hi : S;
    const int kv_end = a.causal ? q_hi : S;
    const int n_tiles = (kv_end + kKvTile - 1) / kKvTile;

    // K/V tile loader: 512 chunks of 16 bytes per operand, two per thread
    raw16_t kreg[2], vreg[2];
    auto g2r = [&](int tile) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int id = tid + u * kAttnThreads;
            int row = tile * kKvTile + (id >> 3);
            row = row < S ? row : S - 1;
            const int64_t off = (int64_t)row * a.ss + (id & 7) * 8;
            kreg[u] = load_raw(kp + off);
            vreg[u] = load_raw(vp + off);
        }
    };
    auto r2s = [&](int stage) {
        lds_char* ks = lds + stage * 2 * kTileBytes;
        lds_char* vs = ks + kTileBytes;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int id = tid + u * kAttnThreads;
            const int r = id >> 3, c = id & 7;
            *(__attribute__((address_space(3))) raw16_t*)(ks + k_lds_offset(r, c)) = kreg[u];
            *(__attribute__((address_space(3))) raw16_t*)(vs + v_lds_offset(r, c)) = vreg[u];
        }
    };

    // per-lane LDS read offsets
    // K fragment (kt, kb): row 32 kt + l32, chunk 2 kb + half
    // V^T fragment (dt, kvb): rows 16 kvb + 4 hh + {0..3} and + 8, columns 32 dt + 16 (grp & 1) + ...
    const int grp = lane >> 4, i16 = lane & 15;
    const int v_hh = grp >> 1;  // which half of the k slots this lane feeds (= lane >> 5)

    g2r(0);
    r2s(0);
    __syncthreads();

    for (int t = 0; t < n_tiles; ++t) {
        const int stage = t & 1;
        const int kv0 = t * kKvTile;
        if (t + 1 < n_tiles) g2r(t + 1);

        const bool active = !a.causal || kv0 <= qw0 + kQPerWave - 1;
        if (active) {
            lds_char* ks = lds + stage * 2 * kTileBytes;
            lds_char* vs = ks + kTileBytes;
            const bool need_mask = (a.causal && kv0 + kKvTile - 1 > qw0) || kv0 + kKvTile > S;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                // S^T tiles for both query tiles against kv rows 32 kt .. +31
                f32x16_t st[2];
#pragma unroll
                for (int qt = 0; qt < 2; ++qt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) st[qt][e] = 0.0f;
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) {
                    const bf16x8_t kf = *(__attribute__((address_space(3))) const bf16x8_t*)(ks + k_lds_offset(32 * kt + l32, 2 * kb + half));
                    st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[0][kb], st[0], 0, 0, 0);
                    st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[1][kb], st[1], 0, 0, 0);
                }
                bf16x8_t pb[2][2];
#pragma unroll
                for (int qt = 0; qt < 2; ++qt) {
                    // element e: kv = kv0 + 32 kt + 8 (e / 4) + 4 half + e % 4, query = qw0 + 32 qt + l32
                    if (need_mask) {
                        const int qi = qw0 + 32 * qt + l32;
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const int kvi = kv0 + 32 * kt + 8 * (e >> 2) + 4 * half + (e & 3);
                            const bool dead = (a.causal && kvi > qi) || kvi >= S;
                            st[qt][e] = dead ? kNegBig : st[qt][e];
                        }
                    }
                    float mx = st[qt][0];
#pragma unroll
                    for (int e = 1; e < 16; ++e) mx = fmaxf(mx, st[qt][e]);
                    mx = fmaxf(mx, xchg32(mx));
                    const float m_new = fmaxf(m_run[qt], mx * a.scale_log2e);
                    const float m_use = (m_new == kNegBig) ? 0.0f : m_new;  // a row with no live key yet
                    const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_use);
                    float psum = 0.0f;
                    float p[16];
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[qt][e], a.scale_log2e, -m_use));
                        psum += p[e];
                    }
                    m_run[qt] = m_new;
                    l_run[qt] = l_run[qt] * alpha + psum;
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                        for (int e = 0; e < 16; ++e) oacc[qt][dt][e] *= alpha;
                    // k slot j of 16-block kvb: e = 8 kvb + j  (kv = 16 kvb + 4 half + j for j < 4, + 8 + 4 half + j - 4 above)
#pragma unroll
                    for (int kvb = 0; kvb < 2; ++kvb) {
                        bf16x8_t v8;
#pragma unroll
                        for (int j = 0; j < 8; ++j) v8[j] = (__bf16)p[8 * kvb + j];
                        pb[qt][kvb] = v8;
                    }
                }
                // O^T += V^T P^T over the 32 kv rows of this half tile
#pragma unroll
                for (int kvb = 0; kvb < 2; ++kvb) {
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt) {
                        const int r0 = 32 * kt + 16 * kvb + 4 * v_hh + (i16 >> 2);
                        const int unit = 2 * dt + (grp & 1);  // 32-byte unit = 16 columns
                        const int off_lo = r0 * 128 + ((unit ^ (r0 & 3)) << 5) + 8 * (i16 & 3);
                        const int r1 = r0 + 8;
                        const int off_hi = r1 * 128 + ((unit ^ (r1 & 3)) << 5) + 8 * (i16 & 3);
                        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(vs + off_lo));
                        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(vs + off_hi));
                        const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, (s16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                        oacc[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb[0][kvb], oacc[0][dt], 0, 0, 0);
                        oacc[1][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb[1][kvb], oacc[1][dt], 0, 0, 0);
                    }
                }
            }
        }
        if (t + 1 < n_tiles) r2s(stage ^ 1);
        __syncthreads();
    }

    // finish: combine the two halves' sums, normalise, store. Lane holds
    // O^T[d = 32 dt + 8 (e / 4) + 4 half + e % 4][q = l32] of query tile qt.
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        const int qi = qw0 + 32 * qt + l32;
        const float l_tot = l_run[qt] + xchg32(l_run[qt]);
        const float inv = l_tot > 0.0f ? __builtin_amdgcn_rcpf(l_tot) : 0.0f;
        if (qi < S) {
            uint16_t* op = a.o + b * a.ob + (int64_t)qi * a.os + h * a.oh;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint32_t w0 = pack_bf16x2(oacc[qt][dt][4 * g] * inv, oacc[qt][dt][4 * g + 1] * inv);
                    uint32_t w1 = pack_bf16x2(oacc[qt][dt][4 * g + 2] * inv, oacc[qt][dt][4 * g + 3] * inv);
                    uint2 w = make_uint2(w0, w1);
                    *reinterpret_cast<uint2*>(op + 32 * dt + 8 * g + 4 * half) = w;
                }
            if (half == 0 && a.lse != nullptr)
                a.lse[(int64_t)bh * S + qi] = (m_run[qt] + __builtin_amdgcn_logf(l_tot)) * kLn2;  // natural-log LSE of scale*s
        }
    }
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int cw_attn_fwd(int64_t B, int64_t H, int64_t S, int64_t D, const void* q, const void* k, const void* v,
                           int64_t stride_b, int64_t stride_s, int64_t stride_h, float scale, int causal, void* out,
                           int64_t out_stride_b, int64_t out_stride_s, int64_t out_stride_h, float* lse,
                           int io_dtype, void* stream) {
    if (B < 0 || H < 0 || S < 0 || D <= 0) return fail(CW_ERR_INVALID, "cw_attn_fwd: bad shape B=%lld H=%lld S=%lld D=%lld", (long long)B, (long long)H, (long long)S, (long long)D);
    if (io_dtype != CW_BF16) return fail(CW_ERR_UNSUPPORTED, "cw_attn_fwd: only bf16 is provided");
    if (D != kHead) return fail(CW_ERR_UNSUPPORTED, "cw_attn_fwd: head size %lld is not provided (64 only)", (long long)D);
    if (B == 0 || H == 0 || S == 0) return CW_OK;
    if (q == nullptr || k == nullptr || v == nullptr || out == nullptr) return fail(CW_ERR_INVALID, "cw_attn_fwd: null pointer");
    if (S > INT32_MAX / 2 || B * H > (1 << 20) || ((S + kQPerBlock - 1) / kQPerBlock) * B * H > INT32_MAX)
        return fail(CW_ERR_INVALID, "cw_attn_fwd: S or B*H too large");
    const bool aligned = aligned16(q) && aligned16(k) && aligned16(v) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0 &&
                         stride_b % 8 == 0 && stride_s % 8 == 0 && stride_h % 8 == 0 && out_stride_b % 4 == 0 &&
                         out_stride_s % 4 == 0 && out_stride_h % 4 == 0;
    if (!aligned) return fail(CW_ERR_ALIGNMENT, "cw_attn_fwd: q/k/v need 16-byte aligned rows, out 8-byte aligned rows");
    AttnArgs a;
    a.q = (const uint16_t*)q;
    a.k = (const uint16_t*)k;
    a.v = (const uint16_t*)v;
    a.o = (uint16_t*)out;
    a.lse = lse;
    a.sb = stride_b; a.ss = stride_s; a.sh = stride_h;
    a.ob = out_stride_b; a.os = out_stride_s; a.oh = out_stride_h;
    a.S = (int)S; a.H = (int)H; a.BH = (int)(B * H);
    a.scale_log2e = scale * kLog2e;
    a.causal = causal ? 1 : 0;
    a.n_qblocks = (int)((S + kQPerBlock - 1) / kQPerBlock);
    hipLaunchKernelGGL(attn_fwd_kernel, dim3((unsigned)(a.n_qblocks * B * H)), dim3(kAttnThreads), 0,
                       (hipStream_t)stream, a);
    return check_launch("attn_fwd_kernel");
}
