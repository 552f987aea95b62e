// Fused causal attention core for gfx950, head sizes 64 and 128, bf16 (or fp16: E = f16_t):
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
// Block = 8 wavefronts x 32 query rows; K/V tiles of 64 rows are staged in
// LDS (two stages, the next tile loaded straight into LDS while this one is
// used), K as [kv][d] read with ds_read_b128, V as [kv][d] read with
// ds_read_b64_tr_b16. At head size 64 two blocks are resident per compute
// unit (four wavefronts per SIMD); the softmax arithmetic (one v_exp_f32 per
// score) weighs about as much as the matrix products there.
#include "attention_common.h"

namespace cw {

namespace {

using namespace attn;

constexpr int kQT = 1;                    // 32-row query tiles per wavefront
constexpr int kWaves = 8;                 // wavefronts per block
constexpr int kThreads = kWaves * 64;
constexpr int kQPerWave = 32 * kQT;
constexpr float kLazy = 8.0f;             // log2 of the largest probability taken against a stale reference
constexpr float kNoKey = -1.0e30f;        // reference of a row that has met no live key yet (finite on purpose)
constexpr int kQPerBlock = kWaves * kQPerWave;

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

// NP: head size / 64. A tile of NP x 64 columns is NP images side by side ("panels"); everything that
// runs over the head dimension runs over NP times as many 16-wide k blocks (scores) or 32-wide output
// blocks (O^T). Head size 64 keeps two blocks per compute unit, 128 has the registers and LDS of one.
template <int NP, typename E>
__global__ __launch_bounds__(kThreads, NP == 1 ? 2 : 1) void attn_fwd_kernel(const AttnArgs a) {
    constexpr int kStage = 2 * NP * kImage;  // K panels (row images), then V panels (transpose images)
    __shared__ __attribute__((aligned(16))) char lds_raw[2 * kStage];
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
    // Under the causal mask a wavefront's work grows with its query position, and wavefront w always runs on
    // SIMD w % 4: half of the blocks deal the query tiles in reverse so that no SIMD collects the long ones
    // (blocks 256 apart, which share a compute unit when the launch starts, differ in bit 8).
    const int wq = (a.causal && (((blockIdx.x >> 8) ^ blockIdx.x) & 1)) ? kWaves - 1 - wave : wave;
    const int qw0 = q0 + wq * kQPerWave;

    const uint16_t* qp = a.q + b * a.sb + h * a.sh;
    const uint16_t* kp = a.k + b * a.sb + h * a.sh;
    const uint16_t* vp = a.v + b * a.sb + h * a.sh;

    // Q fragments (B operand): lane = query row l32 of tile qt, 8 d-values at 16 kb + 8 half
    bf16x8_t qf[kQT][4 * NP];
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        int row = qw0 + 32 * qt + l32;
        row = row < S ? row : S - 1;
        const uint16_t* p = qp + (int64_t)row * a.ss + 8 * half;
#pragma unroll
        for (int kb = 0; kb < 4 * NP; ++kb) qf[qt][kb] = __builtin_bit_cast(bf16x8_t, load_raw(p + 16 * kb));
    }

    f32x16_t oacc[kQT][2 * NP];
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt)
#pragma unroll
        for (int dt = 0; dt < 2 * NP; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[qt][dt][e] = 0.0f;
    // reference of the exponentials (scale*log2e*s units), the raw score above which it moves, this lane's share
    // of the running sum
    float m_run[kQT], m_thr[kQT], l_run[kQT];
    const float inv_scale_log2e = 1.0f / a.scale_log2e;
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        m_run[qt] = kNoKey;
        m_thr[qt] = (kNoKey + kLazy) * inv_scale_log2e;
        l_run[qt] = 0.0f;
    }

    int q_hi = q0 + kQPerBlock;
    q_hi = q_hi < S ? q_hi : S;
    const int kv_end = a.causal ? q_hi : S;
    const int n_tiles = (kv_end + kTile - 1) / kTile;

    TileDma<kThreads> dma;
    dma.init(tid);
    const uint32_t lds_addr = (uint32_t)(uintptr_t)lds;
    ReadOffsets ro;
    ro.init(lane);
    // stage = K row image, V transpose image, filled by the load unit
    auto load_stage = [&](int row0, uint32_t stage_addr) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            dma.template load<true, false>(kp + 64 * p, a.ss, row0, S, stage_addr + p * kImage, 0);
            dma.template load<false, true>(vp + 64 * p, a.ss, row0, S, 0, stage_addr + (NP + p) * kImage);
        }
    };
    load_stage(0, lds_addr);
    dma_wait<0>();
    __syncthreads();
    // The Q fragments must have arrived before the loop. Left pending, the compiler waits for them
    // inside the loop in every trip, and such a wait also covers the younger loads in flight: the next
    // tile's prefetch, whose latency the trip is there to hide.
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt)
#pragma unroll
        for (int kb = 0; kb < 4 * NP; ++kb) asm volatile("" : "+v"(qf[qt][kb]));

    // One tile of 64 key rows out of LDS stage STAGE (a compile-time constant, so that every fragment read is
    // lane offset + immediate: no address arithmetic in the loop); the loop below alternates the two stages.
    auto tile_step = [&](int t, auto stage_c) {
        constexpr int STAGE = decltype(stage_c)::value;
        lds_char* ks = lds + STAGE * kStage;
        lds_char* vs = ks + NP * kImage;
        const int kv0 = t * kTile;
        if (t + 1 < n_tiles) {
            // the other stage was last read in the previous trip, which ended with a barrier
            load_stage(kv0 + kTile, lds_addr + (1 - STAGE) * kStage);
        }

        const bool active = !a.causal || kv0 <= qw0 + kQPerWave - 1;
        if (active) {
            const bool need_mask = (a.causal && kv0 + kTile - 1 > qw0) || kv0 + kTile > S;
            // Only tiles on the diagonal or past the end of the sequence need the mask: a scalar branch
            // around the compare/select work, which interior tiles skip.
            const bool masked = __builtin_amdgcn_readfirstlane((int)need_mask) != 0;
            auto half_tile = [&](auto kt_c) {
                constexpr int kt = decltype(kt_c)::value;
                // S^T tiles for both query tiles against kv rows 32 kt .. +31
                f32x16_t st[kQT];
#pragma unroll
                for (int qt = 0; qt < kQT; ++qt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) st[qt][e] = 0.0f;
#pragma unroll
                for (int kb = 0; kb < 4 * NP; ++kb) {
                    const bf16x8_t kf = read_rows<32 * kt>(ks + (kb >> 2) * kImage, ro, kb & 3);
#pragma unroll
                    for (int qt = 0; qt < kQT; ++qt)
                        st[qt] = mfma16<E>(kf, qf[qt][kb], st[qt]);
                }
                bf16x8_t pb[kQT][2];
#pragma unroll
                for (int qt = 0; qt < kQT; ++qt) {
                    // element e: kv = kv0 + 32 kt + 8 (e / 4) + 4 half + e % 4, query = qw0 + 32 qt + l32
                    if (masked) {
                        // live <=> kv <= min(query, S-1) <=> 32 kt + 8 (e/4) + e%4 <= lim
                        const int qi = qw0 + 32 * qt + l32;
                        const int last = a.causal ? (qi < S - 1 ? qi : S - 1) : S - 1;
                        const int lim = last - kv0 - 4 * half;
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            st[qt][e] = (32 * kt + 8 * (e >> 2) + (e & 3) > lim) ? kNegBig : st[qt][e];
                    }
                    float mx = st[qt][0];
#pragma unroll
                    for (int e = 1; e < 16; ++e) mx = fmaxf(mx, st[qt][e]);
                    mx = max_halves(mx);
                    // m_run is the reference the exponentials are taken against, not necessarily the maximum so
                    // far: it moves (and the running sum and O^T are rescaled, 34 vector instructions) only
                    // when some row's maximum exceeds it by more than kLazy, i.e. a probability would pass
                    // 2^kLazy. With the true maximum as reference some row of the 32 moves in most tiles. The
                    // quotient O / l does not depend on the reference, and bf16 / fp16 keep their relative
                    // precision at 2^kLazy. The test is one compare against m_thr = (m_run + kLazy) / (scale
                    // log2 e), in the units of the raw scores. A row without a live key so far has the finite
                    // reference kNoKey: its maximum, once it has one, is always above the threshold, and until
                    // then its scores are -inf and its probabilities exp2(-inf - kNoKey) = 0.
                    if (__builtin_amdgcn_ballot_w64(mx > m_thr[qt]) != 0) {
                        const float m_new = fmaxf(m_run[qt], mx * a.scale_log2e);
                        const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_new);
                        l_run[qt] *= alpha;
#pragma unroll
                        for (int dt = 0; dt < 2 * NP; ++dt)
#pragma unroll
                            for (int e = 0; e < 16; ++e) oacc[qt][dt][e] *= alpha;
                        m_run[qt] = m_new;
                        m_thr[qt] = (m_new + kLazy) * inv_scale_log2e;
                    }
                    const float m_use = m_run[qt];
                    float p[16];
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[qt][e], a.scale_log2e, -m_use));
                    // k slot j of 16-block kvb <-> e = 8 kvb + j. The row sum is taken over the rounded
                    // probabilities, the values the second product uses.
                    pb[qt][0] = pack_slots<E>(p, 0);
                    pb[qt][1] = pack_slots<E>(p, 1);
                    l_run[qt] = sum_slots<E>(pb[qt][1], sum_slots<E>(pb[qt][0], l_run[qt]));
                }
                // O^T += V^T P^T over the 32 kv rows of this half tile
#pragma unroll
                for (int dt = 0; dt < 2 * NP; ++dt) {
                    const bf16x8_t vf0 = read_transposed<32 * kt>(vs + (dt >> 1) * kImage, ro, dt & 1);
                    const bf16x8_t vf1 = read_transposed<32 * kt + 16>(vs + (dt >> 1) * kImage, ro, dt & 1);
#pragma unroll
                    for (int qt = 0; qt < kQT; ++qt) {
                        oacc[qt][dt] = mfma16<E>(vf0, pb[qt][0], oacc[qt][dt]);
                        oacc[qt][dt] = mfma16<E>(vf1, pb[qt][1], oacc[qt][dt]);
                    }
                }
            };
            half_tile(std::integral_constant<int, 0>{});
            // the second 32 key rows of a tile that starts on the wavefront's diagonal are wholly masked
            if (!a.causal || kv0 + 32 <= qw0 + kQPerWave - 1) half_tile(std::integral_constant<int, 1>{});
        }
        dma_wait<0>();  // the next tile has landed (a third stage and loads two tiles ahead gained nothing)
        __syncthreads();
    };
    int t = 0;
    for (; t + 1 < n_tiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{});
        tile_step(t + 1, std::integral_constant<int, 1>{});
    }
    if (t < n_tiles) tile_step(t, std::integral_constant<int, 0>{});

    // finish: combine the two halves' sums, normalise, store
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        const int qi = qw0 + 32 * qt + l32;
        const float l_tot = sum_halves(l_run[qt]);
        const float inv = l_tot > 0.0f ? __builtin_amdgcn_rcpf(l_tot) : 0.0f;
        if (qi < S) {
            uint16_t* orow = a.o + b * a.ob + (int64_t)qi * a.os + h * a.oh;
#pragma unroll
            for (int p = 0; p < NP; ++p) store_row_pieces<E>(orow + 64 * p, oacc[qt] + 2 * p, inv, half);
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
    if (io_dtype != CW_BF16 && io_dtype != CW_F16) return fail(CW_ERR_UNSUPPORTED, "cw_attn_fwd: only bf16 and fp16 are provided");
    if (D != 64 && D != 128) return fail(CW_ERR_UNSUPPORTED, "cw_attn_fwd: head size %lld is not provided (64 and 128)", (long long)D);
    if (B == 0 || H == 0 || S == 0) return CW_OK;
    if (q == nullptr || k == nullptr || v == nullptr || out == nullptr) return fail(CW_ERR_INVALID, "cw_attn_fwd: null pointer");
    if (S > INT32_MAX / 2 || B * H > (1 << 20) || ((S + kQPerBlock - 1) / kQPerBlock) * B * H > INT32_MAX)
        return fail(CW_ERR_INVALID, "cw_attn_fwd: S or B*H too large");
    const bool aligned = aligned16(q) && aligned16(k) && aligned16(v) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0 &&
                         stride_b % 8 == 0 && stride_s % 8 == 0 && stride_h % 8 == 0 && out_stride_b % 4 == 0 &&
                         out_stride_s % 4 == 0 && out_stride_h % 4 == 0;
    if (!aligned) return fail(CW_ERR_ALIGNMENT, "cw_attn_fwd: q/k/v need 16-byte aligned rows, out 8-byte aligned rows");
    if (stride_s <= 0 || stride_s >= (1 << 23))
        return fail(CW_ERR_INVALID, "cw_attn_fwd: token stride %lld outside (0, 2^23) elements", (long long)stride_s);
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
    const dim3 grid((unsigned)(a.n_qblocks * B * H));
    if (const int drc = require_gfx950("cw_attn_fwd"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (io_dtype == CW_F16) {
        if (D == 64) hipLaunchKernelGGL((attn_fwd_kernel<1, f16_t>), grid, dim3(kThreads), 0, s, a);
        else hipLaunchKernelGGL((attn_fwd_kernel<2, f16_t>), grid, dim3(kThreads), 0, s, a);
    } else {
        if (D == 64) hipLaunchKernelGGL((attn_fwd_kernel<1, bf16_t>), grid, dim3(kThreads), 0, s, a);
        else hipLaunchKernelGGL((attn_fwd_kernel<2, bf16_t>), grid, dim3(kThreads), 0, s, a);
    }
    return check_launch("attn_fwd_kernel");
}
