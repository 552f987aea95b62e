// Backward of the fused attention core for gfx950 (head sizes 64 and 128; bf16, or fp16 with E = f16_t):
// given Q, K, V, O, dO and the forward's log-sum-exp L (natural log),
//   P_ij  = exp(scale q_i.k_j - L_i)              (recomputed, never stored)
//   D_i   = sum_d dO_id O_id
//   dV_j  = sum_i P_ij dO_i
//   dS_ij = P_ij (dO_i.v_j - D_i)
//   dQ_i  = scale sum_j dS_ij k_j,   dK_j = scale sum_i dS_ij q_i
// which is what autograd derives for benchmark/opt/opt.py:84-117 of the
// reference (scaled bmm, mask, softmax, bmm).
//
// Two kernels, no atomics (results are bit-reproducible):
//   attn_dq_kernel    : a block owns 256 query rows (32 per wavefront, Q and dO
//                       fragments in registers; D_i from them and the same rows
//                       of O, also left in scratch for the second kernel) and
//                       walks the K/V tiles; all
//                       products are formed transposed (lane = query row), so
//                       L_i and D_i are per-lane scalars.
//   attn_dkdv_kernel  : a block owns 256 key rows (32 per wavefront, K and V
//                       fragments in registers) and walks the Q/dO tiles;
//                       products are formed with lane = key row.
// In both, the fp32 probabilities / score gradients of a lane, rounded to
// bf16, are directly the B operand of the next MFMA, and the A operand of
// that MFMA (K^T, Q^T or dO^T) comes from a transposing LDS read of the tile
// that is also read row-wise; the tile is kept in LDS in two images, each
// swizzled for its own read pattern.
#include "attention_common.h"

namespace cw {

namespace {

using namespace attn;

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kRowsPerWave = 32;
constexpr int kRowsPerBlock = kWaves * kRowsPerWave;
// dK/dV kernel: 4 wavefronts (128 keys) per workgroup. At head size 64 a wavefront needs 218 registers and two
// workgroups share a compute unit (two wavefronts per SIMD, 2 x 65 KB of LDS): they run out of step, so that one's
// MFMA groups overlap the other's vector work, where the 8 wavefronts of one workgroup met at a barrier per tile
// and ran the same phase at the same time (302 -> 291 us for the whole backward at batch 4 x 32 heads x 2048
// tokens). At head size 128 a wavefront needs more than 256 registers and a unit holds one workgroup. Two groups
// of 32 keys per wavefront (every LDS operand read feeding two MFMAs, 510 registers) ran 278 us against 190 us.
constexpr int kDkdvWaves = 4;

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
    int S, H, BH, n_blocks;  // n_blocks: query blocks of the dQ kernel
    int D;                   // head size (64 or 128)
    float scale, scale_log2e;
    int causal;
};

// ---- dQ ---------------------------------------------------------------------
// LDS per stage: K row images, K transpose images, V row images (NP = head size / 64 panels of each).
template <int NP, typename E>
__global__ __launch_bounds__(kThreads, 1) void attn_dq_kernel(const BwdArgs a) {
    constexpr int kStage = 3 * NP * kImage;
    __shared__ __attribute__((aligned(16))) char lds_raw[2 * kStage];
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

    // the lane's query row: Q and dO fragments (B operands), L*log2e and D
    const int qi = qw0 + l32;
    const int qrow = qi < S ? qi : S - 1;
    bf16x8_t qf[4 * NP], dof[4 * NP];
    // D of the lane's row, from the dO pieces it holds anyway and the same pieces of O: the two lanes of a row
    // (half 0 and 1) add their parts. The dK/dV launch, which follows on the stream, reads it from a.delta.
    float dlt_ld = 0.0f;
    {
        const uint16_t* p = a.q + b * a.sb + (int64_t)qrow * a.ss + h * a.sh + 8 * half;
        const uint16_t* g = a.d_o + b * a.ob + (int64_t)qrow * a.os + h * a.oh + 8 * half;
        const uint16_t* o = a.o + b * a.ob + (int64_t)qrow * a.os + h * a.oh + 8 * half;
#pragma unroll
        for (int kb = 0; kb < 4 * NP; ++kb) {
            qf[kb] = __builtin_bit_cast(bf16x8_t, load_raw(p + 16 * kb));
            const raw16_t graw = load_raw(g + 16 * kb);
            dof[kb] = __builtin_bit_cast(bf16x8_t, graw);
            float x[8], y[8];
            unpack_raw(load_raw(o + 16 * kb), x, (const E*)nullptr);
            unpack_raw(graw, y, (const E*)nullptr);
#pragma unroll
            for (int e = 0; e < 8; ++e) dlt_ld = __builtin_fmaf(x[e], y[e], dlt_ld);
        }
        dlt_ld += __shfl_xor(dlt_ld, 32, 64);
        if (half == 0 && qi < S) a.delta[(int64_t)bh * S + qi] = dlt_ld;
    }
    const float lse2_ld = a.lse[(int64_t)bh * S + qrow] * kLog2e;
    f32x16_t dq[2 * NP];
#pragma unroll
    for (int dt = 0; dt < 2 * NP; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) dq[dt][e] = 0.0f;

    int q_hi = q0 + kRowsPerBlock;
    q_hi = q_hi < S ? q_hi : S;
    const int kv_end = a.causal ? q_hi : S;
    const int n_tiles = (kv_end + kTile - 1) / kTile;

    ReadOffsets ro;
    ro.init(lane);
    TileDma<kThreads> dma;
    dma.init(tid);
    const uint32_t lds_addr = (uint32_t)(uintptr_t)lds;
    // stage = K row images, K transpose images, V row images, filled by the load unit
    auto load_stage = [&](int row0, uint32_t st) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            dma.template load<true, true>(kp + 64 * p, a.ss, row0, S, st + p * kImage, st + (NP + p) * kImage);
            dma.template load<true, false>(vp + 64 * p, a.ss, row0, S, st + (2 * NP + p) * kImage, 0);
        }
    };
    load_stage(0, lds_addr);
    dma_wait<0>();
    __syncthreads();
    // Everything loaded so far must have arrived before the loop: a wait for it inside the loop would
    // also cover the younger loads in flight there, the next tile's prefetch.
    float lse2 = lse2_ld, dlt = dlt_ld;
    asm volatile("" : "+v"(lse2), "+v"(dlt));
#pragma unroll
    for (int kb = 0; kb < 4 * NP; ++kb) asm volatile("" : "+v"(qf[kb]), "+v"(dof[kb]));

    // One tile of 64 key rows out of LDS stage STAGE, a compile-time constant so that every fragment read is lane
    // offset + immediate (no address arithmetic in the loop); the loop below alternates the two stages.
    auto tile_step = [&](int t, auto stage_c) {
        constexpr int STAGE = decltype(stage_c)::value;
        lds_char* k_rows = lds + STAGE * kStage;
        lds_char* k_tr = k_rows + NP * kImage;
        lds_char* v_rows = k_rows + 2 * NP * kImage;
        const int kv0 = t * kTile;
        if (t + 1 < n_tiles) {
            // the other stage was last read in the previous trip, which ended with a barrier
            load_stage(kv0 + kTile, lds_addr + (1 - STAGE) * kStage);
        }
        const bool active = !a.causal || kv0 <= qw0 + kRowsPerWave - 1;
        if (active) {
            const bool need_mask = (a.causal && kv0 + kTile - 1 > qw0) || kv0 + kTile > S;
            const bool masked = __builtin_amdgcn_readfirstlane((int)need_mask) != 0;  // scalar branch
            const int last = a.causal ? (qi < S - 1 ? qi : S - 1) : S - 1;
            const int lim = last - kv0 - 4 * half;  // key element e of half tile kt is live <=> 32 kt + 8 (e/4) + e%4 <= lim
            auto half_tile = [&](auto kt_c) {
                constexpr int kt = decltype(kt_c)::value;
                f32x16_t st, dpt;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    st[e] = 0.0f;
                    dpt[e] = 0.0f;
                }
#pragma unroll
                for (int kb = 0; kb < 4 * NP; ++kb) {
                    st = mfma16<E>(read_rows<32 * kt>(k_rows + (kb >> 2) * kImage, ro, kb & 3), qf[kb], st);
                    dpt = mfma16<E>(read_rows<32 * kt>(v_rows + (kb >> 2) * kImage, ro, kb & 3), dof[kb], dpt);
                }
                // element e: key kv0 + 32 kt + 8 (e / 4) + 4 half + e % 4, query qi
                float ds[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[e], a.scale_log2e, -lse2));
                    ds[e] = p * (dpt[e] - dlt);
                }
                if (masked) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) ds[e] = (32 * kt + 8 * (e >> 2) + (e & 3) > lim) ? 0.0f : ds[e];
                }
                const bf16x8_t dsb0 = pack_slots<E>(ds, 0), dsb1 = pack_slots<E>(ds, 1);
#pragma unroll
                for (int dt = 0; dt < 2 * NP; ++dt) {
                    lds_char* kt_img = k_tr + (dt >> 1) * kImage;
                    dq[dt] = mfma16<E>(read_transposed<32 * kt>(kt_img, ro, dt & 1), dsb0, dq[dt]);
                    dq[dt] = mfma16<E>(read_transposed<32 * kt + 16>(kt_img, ro, dt & 1), dsb1, dq[dt]);
                }
            };
            half_tile(std::integral_constant<int, 0>{});
            // the second 32 key rows of a tile that starts on the wavefront's diagonal are wholly masked
            if (!a.causal || kv0 + 32 <= qw0 + kRowsPerWave - 1) half_tile(std::integral_constant<int, 1>{});
        }
        dma_wait<0>();
        __syncthreads();
    };
    {
        int t = 0;
        for (; t + 1 < n_tiles; t += 2) {
            tile_step(t, std::integral_constant<int, 0>{});
            tile_step(t + 1, std::integral_constant<int, 1>{});
        }
        if (t < n_tiles) tile_step(t, std::integral_constant<int, 0>{});
    }
    if (qi < S) {
        uint16_t* grow = a.dq + b * a.gb + (int64_t)qi * a.gs + h * a.gh;
#pragma unroll
        for (int p = 0; p < NP; ++p) store_row_pieces<E>(grow + 64 * p, dq + 2 * p, a.scale, half);
    }
}

// ---- dK, dV -----------------------------------------------------------------
// LDS per stage: Q row images, Q transpose images, dO row images, dO transpose images (NP = head size / 64
// panels of each), L*log2e and -D of the 64 rows. NW wavefronts of 32 key rows.
template <int NP>
constexpr int dkdv_stage_bytes() { return 4 * NP * kImage + 2 * kTile * 4; }

// KG: groups of 32 key rows per wavefront. With two, every A operand read from LDS (Q, dO, their
// transposes) feeds two MFMAs instead of one.
template <int NP, int NW, int KG, typename E>
__global__ __launch_bounds__(NW * 64, NP == 1 ? 2 : 1) void attn_dkdv_kernel(const BwdArgs a) {
    constexpr int kKeysPerWave = KG * kRowsPerWave;
    constexpr int kDkdvStage = dkdv_stage_bytes<NP>();
    constexpr int kStatsAt = 4 * NP * kImage;
    extern __shared__ __attribute__((aligned(16))) char lds_dyn[];
    lds_char* lds = (lds_char*)lds_dyn;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int S = a.S;
    const int bh = (int)(blockIdx.x % (unsigned)a.BH);
    const int b = bh / a.H, h = bh - b * a.H;
    const int kvblk = (int)(blockIdx.x / (unsigned)a.BH);  // under the causal mask the first key block is the longest
    const int kvb0 = kvblk * (NW * kKeysPerWave);
    const int kw0 = kvb0 + wave * kKeysPerWave;

    const uint16_t* qp = a.q + b * a.sb + h * a.sh;
    const uint16_t* gp = a.d_o + b * a.ob + h * a.oh;
    const float* lsep = a.lse + (int64_t)bh * S;
    const float* dltp = a.delta + (int64_t)bh * S;

    // the lane's key rows (one per group): K and V fragments (B operands)
    bf16x8_t kf[KG][4 * NP], vf[KG][4 * NP];
#pragma unroll
    for (int kg = 0; kg < KG; ++kg) {
        const int kvi = kw0 + 32 * kg + l32;
        const int kvrow = kvi < S ? kvi : S - 1;
        const uint16_t* pk = a.k + b * a.sb + (int64_t)kvrow * a.ss + h * a.sh + 8 * half;
        const uint16_t* pv = a.v + b * a.sb + (int64_t)kvrow * a.ss + h * a.sh + 8 * half;
#pragma unroll
        for (int kb = 0; kb < 4 * NP; ++kb) {
            kf[kg][kb] = __builtin_bit_cast(bf16x8_t, load_raw(pk + 16 * kb));
            vf[kg][kb] = __builtin_bit_cast(bf16x8_t, load_raw(pv + 16 * kb));
        }
    }
    f32x16_t dk[KG][2 * NP], dv[KG][2 * NP];
#pragma unroll
    for (int kg = 0; kg < KG; ++kg)
#pragma unroll
        for (int dt = 0; dt < 2 * NP; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                dk[kg][dt][e] = 0.0f;
                dv[kg][dt][e] = 0.0f;
            }

    // query tiles: under the causal mask only queries >= the block's first key take part
    const int first_tile = a.causal ? kvb0 / kTile : 0;
    const int n_tiles = (S + kTile - 1) / kTile;

    ReadOffsets ro;
    ro.init(lane);
    TileDma<NW * 64> dma;
    dma.init(tid);
    const uint32_t lds_addr = (uint32_t)(uintptr_t)lds;
    // threads 0..63: L of tile row tid (stored times log2e); 64..127: D of tile row tid - 64 (stored negated). Every thread
    // loads (no branch around the load: the value is not needed before the tile it belongs to is stored,
    // and a wait inside a branch would cover the tile prefetch issued just before); the rest discard.
    float stat = 0.0f;
    const float* statp = tid < kTile ? lsep : dltp;
    const float stat_mul = tid < kTile ? kLog2e : -1.0f;  // D is stored negated: it starts the dP accumulators
    auto load_stats = [&](int q0) {
        int row = q0 + (tid & (kTile - 1));
        row = row < S ? row : S - 1;
        stat = statp[row];
    };
    auto store_stats = [&](lds_char* stage) {
        if (tid < 2 * kTile) *(__attribute__((address_space(3))) float*)(stage + kStatsAt + tid * 4) = stat * stat_mul;
    };
    // stage = Q row and transpose images, dO row and transpose images (filled by the load unit), row statistics
    auto load_stage = [&](int row0, uint32_t st) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            dma.template load<true, true>(qp + 64 * p, a.ss, row0, S, st + p * kImage, st + (NP + p) * kImage);
            dma.template load<true, true>(gp + 64 * p, a.os, row0, S, st + (2 * NP + p) * kImage, st + (3 * NP + p) * kImage);
        }
    };
    load_stage(first_tile * kTile, lds_addr);
    load_stats(first_tile * kTile);
    store_stats(lds);
    dma_wait<0>();
    __syncthreads();
#pragma unroll
    for (int kg = 0; kg < KG; ++kg)
#pragma unroll
        for (int kb = 0; kb < 4 * NP; ++kb) asm volatile("" : "+v"(kf[kg][kb]), "+v"(vf[kg][kb]));  // arrived before the loop

    // One tile of 64 query rows out of LDS stage STAGE (compile-time: fragment reads are lane offset + immediate)
    auto tile_step = [&](int t, auto stage_c) {
        constexpr int STAGE = decltype(stage_c)::value;
        lds_char* stg = lds + STAGE * kDkdvStage;
        lds_char* q_rows = stg;
        lds_char* q_tr = stg + NP * kImage;
        lds_char* g_rows = stg + 2 * NP * kImage;
        lds_char* g_tr = stg + 3 * NP * kImage;
        lds_char* stats = stg + kStatsAt + 16 * half;  // + 4 bytes x (4 half): the lane's rows start at 8 g + 4 half
        const int q0 = t * kTile;
        if (t + 1 < n_tiles) {
            // the other stage was last read in the previous trip, which ended with a barrier
            load_stage(q0 + kTile, lds_addr + (1 - STAGE) * kDkdvStage);
            load_stats(q0 + kTile);
        }
        // the wavefront's keys kw0 .. kw0 + kKeysPerWave - 1 see queries >= kw0 only
        const bool active = !a.causal || q0 + kTile - 1 >= kw0;
        if (active) {
            const bool need_mask = (a.causal && q0 < kw0 + kKeysPerWave - 1) || q0 + kTile > S;
            const bool masked = __builtin_amdgcn_readfirstlane((int)need_mask) != 0;  // scalar branch
            // query element e of query tile qt (row q0 + 32 qt + 8 (e/4) + 4 half + e%4) is live for the
            // key of group kg <=> row >= key (causal) and row < S  <=>  lo + 32 kg <= 32 qt + 8 (e/4) + e%4 < hi
            const int lo = a.causal ? kw0 + l32 - q0 - 4 * half : -(1 << 30);
            const int hi = S - q0 - 4 * half;
            auto q_tile = [&](auto qt_c) {
                constexpr int qt = decltype(qt_c)::value;
                // the dP accumulators start at -D of their query rows (32 qt + 8 g + 4 half + {0..3}), so that the
                // products leave dP - D
                f32x16_t s_acc[KG], dp_acc[KG];
#pragma unroll
                for (int kg = 0; kg < KG; ++kg) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) s_acc[kg][e] = 0.0f;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4_t dl = *(__attribute__((address_space(3))) const f32x4_t*)(stats + (kTile + 32 * qt + 8 * g) * 4);
#pragma unroll
                        for (int i = 0; i < 4; ++i) dp_acc[kg][4 * g + i] = dl[i];
                    }
                }
#pragma unroll
                for (int kb = 0; kb < 4 * NP; ++kb) {
                    const bf16x8_t qa = read_rows<32 * qt>(q_rows + (kb >> 2) * kImage, ro, kb & 3);
                    const bf16x8_t ga = read_rows<32 * qt>(g_rows + (kb >> 2) * kImage, ro, kb & 3);
#pragma unroll
                    for (int kg = 0; kg < KG; ++kg) {
                        s_acc[kg] = mfma16<E>(qa, kf[kg][kb], s_acc[kg]);
                        dp_acc[kg] = mfma16<E>(ga, vf[kg][kb], dp_acc[kg]);
                    }
                }
                bf16x8_t pb[KG][2], dsb[KG][2];
#pragma unroll
                for (int kg = 0; kg < KG; ++kg) {
                    float p[16], ds[16];
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        // L*log2e of query rows 32 qt + 8 g + 4 half + {0..3}
                        const f32x4_t l2 = *(__attribute__((address_space(3))) const f32x4_t*)(stats + (32 * qt + 8 * g) * 4);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int e = 4 * g + i;
                            p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kg][e], a.scale_log2e, -l2[i]));
                            ds[e] = p[e] * dp_acc[kg][e];
                        }
                    }
                    if (masked) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const int r = 32 * qt + 8 * (e >> 2) + (e & 3);
                            const bool dead = r < lo + 32 * kg || r >= hi;
                            p[e] = dead ? 0.0f : p[e];
                            ds[e] = dead ? 0.0f : ds[e];
                        }
                    }
#pragma unroll
                    for (int sl = 0; sl < 2; ++sl) {
                        pb[kg][sl] = pack_slots<E>(p, sl);
                        dsb[kg][sl] = pack_slots<E>(ds, sl);
                    }
                }
#pragma unroll
                for (int sl = 0; sl < 2; ++sl) {
#pragma unroll
                    for (int dt = 0; dt < 2 * NP; ++dt) {
                        lds_char* gi = g_tr + (dt >> 1) * kImage;
                        lds_char* qi_img = q_tr + (dt >> 1) * kImage;
                        const bf16x8_t gt = sl == 0 ? read_transposed<32 * qt>(gi, ro, dt & 1) : read_transposed<32 * qt + 16>(gi, ro, dt & 1);
                        const bf16x8_t qtr = sl == 0 ? read_transposed<32 * qt>(qi_img, ro, dt & 1) : read_transposed<32 * qt + 16>(qi_img, ro, dt & 1);
#pragma unroll
                        for (int kg = 0; kg < KG; ++kg) {
                            dv[kg][dt] = mfma16<E>(gt, pb[kg][sl], dv[kg][dt]);
                            dk[kg][dt] = mfma16<E>(qtr, dsb[kg][sl], dk[kg][dt]);
                        }
                    }
                }
            };
            q_tile(std::integral_constant<int, 0>{});
            q_tile(std::integral_constant<int, 1>{});
        }
        if (t + 1 < n_tiles) store_stats(lds + (1 - STAGE) * kDkdvStage);
        dma_wait<0>();
        __syncthreads();
    };
    {
        int t = first_tile;
        for (; t + 1 < n_tiles; t += 2) {
            tile_step(t, std::integral_constant<int, 0>{});
            tile_step(t + 1, std::integral_constant<int, 1>{});
        }
        if (t < n_tiles) tile_step(t, std::integral_constant<int, 0>{});
    }
#pragma unroll
    for (int kg = 0; kg < KG; ++kg) {
        const int kvi = kw0 + 32 * kg + l32;
        if (kvi < S) {
            uint16_t* dkrow = a.dk + b * a.gb + (int64_t)kvi * a.gs + h * a.gh;
            uint16_t* dvrow = a.dv + b * a.gb + (int64_t)kvi * a.gs + h * a.gh;
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                store_row_pieces<E>(dkrow + 64 * p, dk[kg] + 2 * p, a.scale, half);
                store_row_pieces<E>(dvrow + 64 * p, dv[kg] + 2 * p, 1.0f, half);
            }
        }
    }
}

// The three launches of the backward for element type E.
template <typename E>
int launch_bwd(const BwdArgs& a, int64_t B, int64_t H, int64_t S, int64_t D, int64_t nblk, hipStream_t s) {
    if (D == 64) hipLaunchKernelGGL((attn_dq_kernel<1, E>), dim3((unsigned)(nblk * B * H)), dim3(kThreads), 0, s, a);
    else hipLaunchKernelGGL((attn_dq_kernel<2, E>), dim3((unsigned)(nblk * B * H)), dim3(kThreads), 0, s, a);
    if (const int rc = check_launch("attn_dq_kernel"); rc != CW_OK) return rc;
    // both head sizes: 4 wavefronts (128 keys) per workgroup
    const int64_t nkv = (S + kDkdvWaves * kRowsPerWave - 1) / (kDkdvWaves * kRowsPerWave);
    if (nkv * B * H > INT32_MAX) return fail(CW_ERR_INVALID, "cw_attn_bwd: S or B*H too large");
    if (D == 64) {
        constexpr int lds_bytes = 2 * dkdv_stage_bytes<1>();
        auto kern = attn_dkdv_kernel<1, kDkdvWaves, 1, E>;
        if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)(lds_bytes), "attn_dkdv_kernel"); lrc != CW_OK) return lrc;
        hipLaunchKernelGGL(kern, dim3((unsigned)(nkv * B * H)), dim3(kDkdvWaves * 64), lds_bytes, s, a);
    } else {
        constexpr int lds_bytes = 2 * dkdv_stage_bytes<2>();
        auto kern = attn_dkdv_kernel<2, kDkdvWaves, 1, E>;
        if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)(lds_bytes), "attn_dkdv_kernel"); lrc != CW_OK) return lrc;
        hipLaunchKernelGGL(kern, dim3((unsigned)(nkv * B * H)), dim3(kDkdvWaves * 64), lds_bytes, s, a);
    }
    return check_launch("attn_dkdv_kernel");
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
    if (io_dtype != CW_BF16 && io_dtype != CW_F16) return fail(CW_ERR_UNSUPPORTED, "cw_attn_bwd: only bf16 and fp16 are provided");
    if (D != 64 && D != 128) return fail(CW_ERR_UNSUPPORTED, "cw_attn_bwd: head size %lld is not provided (64 and 128)", (long long)D);
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
    if (stride_s <= 0 || stride_s >= (1 << 23) || out_stride_s <= 0 || out_stride_s >= (1 << 23))
        return fail(CW_ERR_INVALID, "cw_attn_bwd: token strides %lld / %lld outside (0, 2^23) elements", (long long)stride_s,
                    (long long)out_stride_s);
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
    a.D = (int)D;
    if (const int drc = require_gfx950("cw_attn_bwd"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return io_dtype == CW_F16 ? launch_bwd<f16_t>(a, B, H, S, D, nblk, s) : launch_bwd<bf16_t>(a, B, H, S, D, nblk, s);
}
