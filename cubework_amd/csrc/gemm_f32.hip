// fp32 variant of the SUMMA block GEMM for gfx950 (v_mfma_f32_32x32x2_f32:
// exact fp32 products, fp32 accumulation) for the layers' fp32 path, where
// results have to agree with torch's fp32 matmul to ~1e-6.
// 128x128 or 256x128 tile per 256-thread block, 2x2 wavefronts of 64x64 or
// 128x64, k tiles of 16 (flattened over the k-steps), operands in LDS as
// [k][row] so a fragment read is 32 consecutive floats, register-staged
// prefetch with two LDS stages. The taller tile is taken when it still leaves
// two tiles per compute unit: both are then resident at once and no partial
// last round of tiles remains (config-1 forward: 1024 tiles of 128x128 are
// 1 1/3 rounds of the 768 that fit).
//
// Large aligned problems (at least 128 tiles of 256x256) take gemm_f32_ring_kernel instead: the ring of LDS
// stages filled by the load unit that the 16-bit kernel uses (gemm_bf16_dma.h), with a k extent of 16 per
// stage. There is no register staging, no LDS write instruction and no fragment read right behind the
// barrier, so a wavefront arrives at the one barrier per stage with the next products' operands already
// in registers.
#include <cstdlib>
#include <cstring>

#include "cw_common.h"
#include "gemm.h"
#include "gemm_bf16_kernel.h"

namespace cw {

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kFBN = 128, kFBK = 16;
constexpr int kFThreads = 256;
constexpr int f32_pitch(int rows) { return rows + 4; }  // floats per LDS k-row

__device__ __forceinline__ float4 load4_guarded(const float* __restrict__ base, int64_t ld, int r, int c, int rmax,
                                                int cmax, bool vec_ok) {
    float4 out = make_float4(0.f, 0.f, 0.f, 0.f);
    if (r >= rmax || c >= cmax) return out;
    const float* p = base + (int64_t)r * ld + c;
    if (vec_ok && c + 4 <= cmax) return *reinterpret_cast<const float4*>(p);
    out.x = p[0];
    if (c + 1 < cmax) out.y = p[1];
    if (c + 2 < cmax) out.z = p[2];
    if (c + 3 < cmax) out.w = p[3];
    return out;
}

// KCONTIG: memory [rows][k]; otherwise memory [k][rows].
template <bool KCONTIG, bool GUARD, int ROWS>
__device__ __forceinline__ void f32_g2r(float4 (&reg)[ROWS / 64], const float* __restrict__ base, int64_t ld, int row0,
                                        int k0, int rmax, int kmax, int tid, bool vec_ok) {
#pragma unroll
    for (int it = 0; it < ROWS / 64; ++it) {
        const int c = it * kFThreads + tid;
        if constexpr (KCONTIG) {
            const int row = row0 + (c >> 2), k = k0 + (c & 3) * 4;
            reg[it] = GUARD ? load4_guarded(base, ld, row, k, rmax, kmax, vec_ok)
                            : *reinterpret_cast<const float4*>(base + (int64_t)row * ld + k);
        } else {
            const int k = k0 + c / (ROWS / 4), row = row0 + (c % (ROWS / 4)) * 4;
            reg[it] = GUARD ? load4_guarded(base, ld, k, row, kmax, rmax, vec_ok)
                            : *reinterpret_cast<const float4*>(base + (int64_t)k * ld + row);
        }
    }
}

// LDS image of one operand's k tile. An operand that is k-contiguous in memory stays [row][k] (pitch
// kRowPitch floats: one ds_write_b128 per 16-byte load, fragments read four k values at a time); the
// other kind is [k][row] (pitch rows + 4, fragments read one float per k).
constexpr int kRowPitch = kFBK + 4;
template <bool KCONTIG>
constexpr int f32_image_floats(int rows) { return KCONTIG ? rows * kRowPitch : kFBK * f32_pitch(rows); }

template <bool KCONTIG, int ROWS>
__device__ __forceinline__ void f32_r2s(const float4 (&reg)[ROWS / 64], float* __restrict__ lds, int tid) {
    constexpr int P = f32_pitch(ROWS);
#pragma unroll
    for (int it = 0; it < ROWS / 64; ++it) {
        const int c = it * kFThreads + tid;
        if constexpr (KCONTIG) {
            const int r = c >> 2, kc = (c & 3) * 4;
            *reinterpret_cast<float4*>(lds + r * kRowPitch + kc) = reg[it];
        } else {
            const int k = c / (ROWS / 4), r = (c % (ROWS / 4)) * 4;
            *reinterpret_cast<float4*>(lds + k * P + r) = reg[it];
        }
    }
}

// The k tile of 16 is consumed in the order k(t, j, h) = 8 t + 4 h + j (t < 2, j < 4; h = lane / 32 is the
// k slot of the MFMA), the same for both operands: the four k values a lane reads with one ds_read_b128
// of a [row][k] image are then four consecutive steps. Fragments of read t for NB blocks of 32 rows.
template <bool KCONTIG, int ROWS, int NB>
__device__ __forceinline__ void f32_read_frags(const float* __restrict__ img, int row0, int lane, int t, float (&f)[NB][4]) {
    const int r = lane & 31, h = lane >> 5;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        if constexpr (KCONTIG) {
            const float4 v = *reinterpret_cast<const float4*>(img + (row0 + 32 * b + r) * kRowPitch + 8 * t + 4 * h);
            f[b][0] = v.x; f[b][1] = v.y; f[b][2] = v.z; f[b][3] = v.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) f[b][j] = img[(8 * t + 4 * h + j) * f32_pitch(ROWS) + row0 + 32 * b + r];
        }
    }
}

// Epilogue of one wavefront's IM x 2 blocks of 32 x 32, one block at a time through a wavefront-private
// LDS patch: the accumulator layout (lane = column, 16 rows per lane) goes in, rows of four consecutive
// columns per lane come out, so bias, addends, pre-activation copy, activation and the store are 16-byte
// accesses along rows. `patch` = 32 x kPatchPitch floats of LDS owned by this wavefront.
constexpr int kPatchPitch = 36;

template <int EPI>
__device__ __forceinline__ float f32_activate(float x) {
    if (EPI == CW_EPI_BIAS_GELU_TANH) return gelu_tanh(x);
    if (EPI == CW_EPI_BIAS_GELU_ERF) return gelu_erf(x);
    if (EPI == CW_EPI_BIAS_RELU) return x < 0.0f ? 0.0f : x;  // NaN stays NaN, as torch.relu leaves it
    return x;
}

template <int EPI, bool GUARD>
__device__ __forceinline__ void f32_store_block(const f32x16_t& blk, float* patch, const GemmArgs& args, int row0, int col0,
                                                int lane) {
    // in: lane holds column lane % 32, rows 8 (v / 4) + 4 (lane / 32) + v % 4
#pragma unroll
    for (int v = 0; v < 16; ++v) patch[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * kPatchPitch + (lane & 31)] = blk[v];
    // out: lane holds columns 4 (lane % 8) .. +3 of rows lane / 8 + 8 pass
    const int c4 = 4 * (lane & 7);
    const int col = col0 + c4;
    const float* bias = reinterpret_cast<const float*>(args.bias);
    float* C = reinterpret_cast<float*>(args.C);
    float* P = reinterpret_cast<float*>(args.preact);
    const bool vec = !GUARD;  // exact tiles of aligned operands: 16-byte accesses
    float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (EPI != CW_EPI_NONE && bias != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e) bv[e] = (!GUARD || col + e < args.N) ? bias[col + e] : 0.0f;
    }
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int r = (lane >> 3) + 8 * pass;
        const int row = row0 + r;
        const float4 t = *reinterpret_cast<const float4*>(patch + r * kPatchPitch + c4);
        float x[4] = {t.x + bv[0], t.y + bv[1], t.z + bv[2], t.w + bv[3]};
        if (GUARD && row >= args.M) continue;
        for (int a = 0; a < args.n_addends; ++a) {
            const float* ad = reinterpret_cast<const float*>(args.addend[a]) + (int64_t)row * args.ldadd + col;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (!GUARD || col + e < args.N) x[e] += ad[e];
        }
        if (P != nullptr) {
            float* pp = P + (int64_t)row * args.ldp + col;
            if (vec && (args.ldp & 3) == 0 && (reinterpret_cast<uintptr_t>(P) & 15u) == 0) {
                *reinterpret_cast<float4*>(pp) = make_float4(x[0], x[1], x[2], x[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (!GUARD || col + e < args.N) pp[e] = x[e];
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = f32_activate<EPI>(x[e]);
        float* cp = C + (int64_t)row * args.ldc + col;
        if (vec && (args.ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0) {
            *reinterpret_cast<float4*>(cp) = make_float4(x[0], x[1], x[2], x[3]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (!GUARD || col + e < args.N) cp[e] = x[e];
        }
    }
}

template <int EPI, int IM, bool GUARD>
__device__ __forceinline__ void f32_store_tile(const f32x16_t (&acc)[IM][2], float* patch, const GemmArgs& args,
                                               int row_base, int col_base, int lane) {
#pragma unroll
    for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) f32_store_block<EPI, GUARD>(acc[i][j], patch, args, row_base + i * 32, col_base + j * 32, lane);
}

template <int BM, bool A_KCONTIG, bool B_KCONTIG, bool GUARD>
__global__ __launch_bounds__(kFThreads, BM == 256 ? 2 : 3) void gemm_f32_kernel(const GemmArgs args, int epilogue) {
    constexpr int OPER_A = f32_image_floats<A_KCONTIG>(BM), OPER_B = f32_image_floats<B_KCONTIG>(kFBN);
    constexpr int STAGE = OPER_A + OPER_B;
    constexpr int IM = BM / 64;  // 32-row MFMA blocks per wavefront
    __shared__ __attribute__((aligned(16))) float lds[2 * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int M = args.M, N = args.N, K = args.K;
    const int tiles_m = (M + BM - 1) / BM;
    const int tiles_n = (N + kFBN - 1) / kFBN;
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= total) return;
    constexpr int GROUP_M = 8;
    const int group = tile / (GROUP_M * tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int in_group = tile - group * GROUP_M * tiles_n;
    const int m0 = (first_m + in_group % gsz) * BM;
    const int n0 = (in_group / gsz) * kFBN;

    const int kt_per_step = (K + kFBK - 1) / kFBK;
    const int KT = kt_per_step * args.n_steps;
    const bool vec_a = args.vec_a != 0, vec_b = args.vec_b != 0;

    f32x16_t acc[IM][2];
#pragma unroll
    for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    float4 ra[BM / 64], rb[kFBN / 64];
    auto issue_loads = [&](int kt) {
        const int step = kt / kt_per_step;
        const int k0 = (kt - step * kt_per_step) * kFBK;
        f32_g2r<A_KCONTIG, GUARD, BM>(ra, reinterpret_cast<const float*>(args.A[step]), args.lda, m0, k0, M, K, tid, vec_a);
        f32_g2r<B_KCONTIG, GUARD, kFBN>(rb, reinterpret_cast<const float*>(args.B[step]), args.ldb, n0, k0, N, K, tid, vec_b);
    };
    auto commit_loads = [&](int stage) {
        float* s = lds + stage * STAGE;
        f32_r2s<A_KCONTIG, BM>(ra, s, tid);
        f32_r2s<B_KCONTIG, kFBN>(rb, s + OPER_A, tid);
    };

    if (KT > 0) {
        issue_loads(0);
        commit_loads(0);
    }
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) issue_loads(kt + 1);
        const float* s = lds + cur * STAGE;
        // fragments of the second half of the k tile are read while the products of the first run
        float af[2][IM][4], bf[2][2][4];
        f32_read_frags<A_KCONTIG, BM, IM>(s, wm * (BM / 2), lane, 0, af[0]);
        f32_read_frags<B_KCONTIG, kFBN, 2>(s + OPER_A, wn * 64, lane, 0, bf[0]);
        f32_read_frags<A_KCONTIG, BM, IM>(s, wm * (BM / 2), lane, 1, af[1]);
        f32_read_frags<B_KCONTIG, kFBN, 2>(s + OPER_A, wn * 64, lane, 1, bf[1]);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4)
#pragma unroll
                for (int i = 0; i < IM; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[t][i][j4], bf[t][j][j4], acc[i][j], 0, 0, 0);
        if (kt + 1 < KT) commit_loads(cur ^ 1);
        __syncthreads();
    }

    // acc[i][j][v]: row m = m0 + wm*(BM/2) + i*32 + 8*(v/4) + 4*(lane>>5) + v%4
    //               col n = n0 + wn*64 + j*32 + (lane & 31)
    // the loop ended with a barrier: the stages are free, each wavefront takes a patch of its own
    float* patch = lds + wave * 32 * kPatchPitch;
    const int row_base = m0 + wm * (BM / 2);
    const int col_base = n0 + wn * 64;
    switch (epilogue) {
        case CW_EPI_BIAS_GELU_TANH: f32_store_tile<CW_EPI_BIAS_GELU_TANH, IM, GUARD>(acc, patch, args, row_base, col_base, lane); break;
        case CW_EPI_BIAS_GELU_ERF: f32_store_tile<CW_EPI_BIAS_GELU_ERF, IM, GUARD>(acc, patch, args, row_base, col_base, lane); break;
        case CW_EPI_BIAS_RELU: f32_store_tile<CW_EPI_BIAS_RELU, IM, GUARD>(acc, patch, args, row_base, col_base, lane); break;
        case CW_EPI_BIAS: f32_store_tile<CW_EPI_BIAS, IM, GUARD>(acc, patch, args, row_base, col_base, lane); break;
        default: f32_store_tile<CW_EPI_NONE, IM, GUARD>(acc, patch, args, row_base, col_base, lane); break;
    }
}

// ---------------------------------------------------------------------------------------------------
// Ring kernel: 256x256 tile per 256-thread block (2x2 wavefronts of 128x128 = 4x4 MFMA blocks, 256
// accumulators per lane; 128x128 and 128x64 tiles, two workgroups per compute unit, for outputs with fewer
// tiles), NS stages of k = 16 in LDS (64 bytes per row, operand and stage), filled by
// global_load_lds_dwordx4 (lane l writes LDS bytes [16 l, 16 l + 16) of the instruction's 1 KB, so an
// image's swizzle is applied on the global side).
//   k-contiguous operand ([rows][k] in memory): image [256 rows][16 k], 64 B per row, 16-byte chunk c of
//     row r at position c ^ ((r >> 2) & 3); a lane reads its row's k = 4h .. 4h+3 and 8+4h .. 8+4h+3
//     (h = lane / 32) with two ds_read_b128;
//   k-slow operand ([k][rows] in memory): image [16 k][256 rows], 1 KB per k row, the 128-byte group g of
//     k row k at position g ^ ((k >> 2) & 1), which puts the two half-wavefronts of a read (k rows 4 apart)
//     on different banks; one ds_read_b32 per product.
// Both kinds consume k in the order k(s, h) = 4h + s (s < 4), 8 + 4h + (s - 4): steps 0..3 ("lo") and 4..7
// ("hi") of a stage. Per stage: products of lo, barrier, products of hi; the hi operands are read during
// the lo products and the next stage's lo operands during the hi products, the eight load instructions of
// the tile NS-1 ahead are spread over both. The loads are inline asm and counted by hand (dma_wait), as in
// the 16-bit kernel.
namespace ring {

typedef __attribute__((address_space(3))) char lds_char;
typedef float f32x4_t __attribute__((ext_vector_type(4)));
constexpr int kBK = 16, kThreads = 256, kStages = 4;
// A tile is 64 TI x 64 TJ (TI, TJ in {1, 2, 4}): 2x2 wavefronts of TI x TJ blocks of 32 x 32. An operand of
// ROWS = 64 T rows takes ROWS * 64 bytes per stage and T load instructions per wavefront.
constexpr int oper_bytes(int t) { return 64 * t * kBK * 4; }


// Byte offset, inside the span of one load instruction, of the 16 bytes this lane fetches.
template <bool KSLOW, int T>
__device__ __forceinline__ uint32_t lane_voff(int lane, int wave, int64_t ld, int row0) {
    if constexpr (!KSLOW) {
        const int r = lane >> 2, c = (lane & 3) ^ (lane >> 4);  // 16 rows x 64 B; swizzle (row >> 2) & 3 = lane >> 4
        return (uint32_t)((((int64_t)(row0 + r)) * ld + c * 4) * 4);
    } else {
        // an instruction's 1 KB holds 4 / T k rows of 16 T chunks; the wavefront's T instructions cover
        // k rows 4 wave .. 4 wave + 3, so (k >> 2) & 1 = wave & 1
        constexpr int kChunks = 16 * T;
        const int kr = lane / kChunks, c = (lane % kChunks) ^ ((wave & 1) << 3);
        return (uint32_t)((((int64_t)kr) * ld + row0 + 4 * c) * 4);
    }
}
// Load instruction I (of T) of this wavefront for one operand (64 T rows) of the tile at k0.
template <bool KSLOW, int T, int I>
__device__ __forceinline__ void dma_one(const char* gbase, int64_t ld_bytes, int k0, uint32_t voff, uint32_t lds_oper, int wave) {
    if constexpr (!KSLOW) {
        const int row = (wave * T + I) * 16;
        dma16(gbase + ((int64_t)row * ld_bytes + (int64_t)k0 * 4), voff, lds_oper + row * 64);
    } else {
        const int k = wave * 4 + I * (4 / T);
        dma16(gbase + (int64_t)(k0 + k) * ld_bytes, voff, lds_oper + k * (256 * T));
    }
}

// Operand values of one half stage: v[block of 32 rows][step].
struct Frag {
    float v[4][4];
};

template <bool KSLOW, int T>
struct Reader {
    uint32_t off[4];  // k-contiguous: [0] lo, [1] hi; k-slow: [block]
    __device__ __forceinline__ void init(int lane, int wrow) {
        const int r = lane & 31, h = lane >> 5;
        if constexpr (!KSLOW) {
            const int swz = (r >> 2) & 3;
            off[0] = (uint32_t)((wrow + r) * 64 + ((h ^ swz) << 4));
            off[1] = (uint32_t)((wrow + r) * 64 + (((2 + h) ^ swz) << 4));
            off[2] = off[3] = 0;
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t) off[t] = (uint32_t)(4 * h * (256 * T) + ((((wrow >> 5) + t) ^ h) << 7) + r * 4);
        }
    }
    // Read number Q of a half stage (HI: steps 4..7) into f: T reads (one per block) for a k-contiguous
    // operand, 4 T (block Q / 4, step Q % 4) for a k-slow one.
    template <int Q, bool HI>
    __device__ __forceinline__ void read(lds_char* oper, Frag& f) const {
        if constexpr (!KSLOW) {
            const f32x4_t x = *(__attribute__((address_space(3))) const f32x4_t*)(oper + off[HI ? 1 : 0] + Q * 2048);
            f.v[Q][0] = x[0]; f.v[Q][1] = x[1]; f.v[Q][2] = x[2]; f.v[Q][3] = x[3];
        } else {
            constexpr int B = Q >> 2, S = Q & 3;
            f.v[B][S] = *(__attribute__((address_space(3))) const float*)(oper + off[B] + ((HI ? 8 : 0) + S) * (256 * T));
        }
    }
    static constexpr int kReads = KSLOW ? 4 * T : T;
};

#define CW_F32_PIN() __builtin_amdgcn_sched_barrier(0)

// One 32 x 32 block of the result through a wavefront-private LDS patch (as f32_store_block), activation
// chosen at run time; whole tile in bounds, 16-byte aligned rows.
__device__ __forceinline__ void store_block(const f32x16_t& blk, float* patch, const RingArgs& args, int epilogue, int row0,
                                            int col0, int lane) {
#pragma unroll
    for (int v = 0; v < 16; ++v) patch[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * kPatchPitch + (lane & 31)] = blk[v];
    const int c4 = 4 * (lane & 7);
    const int col = col0 + c4;
    float4 bv = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (epilogue != CW_EPI_NONE && args.bias != nullptr) bv = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(args.bias) + col);
    float* C = reinterpret_cast<float*>(args.C);
    float* P = reinterpret_cast<float*>(args.preact);
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int r = (lane >> 3) + 8 * pass;
        const int64_t row = row0 + r;
        const float4 t = *reinterpret_cast<const float4*>(patch + r * kPatchPitch + c4);
        float x[4] = {t.x + bv.x, t.y + bv.y, t.z + bv.z, t.w + bv.w};
#pragma unroll 1
        for (int a = 0; a < args.n_addends; ++a) {
            const float4 ad = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(gemm_bf16::pick_ptr(args.addend, a)) + row * args.ldadd + col);
            x[0] += ad.x; x[1] += ad.y; x[2] += ad.z; x[3] += ad.w;
        }
        if (P != nullptr) *reinterpret_cast<float4*>(P + row * args.ldp + col) = make_float4(x[0], x[1], x[2], x[3]);
        if (epilogue == CW_EPI_BIAS_GELU_TANH) {
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = gelu_tanh(x[e]);
        } else if (epilogue == CW_EPI_BIAS_GELU_ERF) {
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = gelu_erf(x[e]);
        } else if (epilogue == CW_EPI_BIAS_RELU) {
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = x[e] < 0.0f ? 0.0f : x[e];  // NaN stays NaN, as torch.relu leaves it
        }
        *reinterpret_cast<float4*>(C + row * args.ldc + col) = make_float4(x[0], x[1], x[2], x[3]);
    }
}

template <int TI, int TJ, bool A_KSLOW, bool B_KSLOW>
__global__ __launch_bounds__(kThreads, (TI * TJ <= 4) ? 2 : 1) void gemm_f32_ring_kernel(const RingArgs args, int epilogue) {
    constexpr int NS = kStages;
    constexpr int BM = 64 * TI, BN = 64 * TJ;
    constexpr int kOperA = oper_bytes(TI), kStageBytes = oper_bytes(TI) + oper_bytes(TJ);
    constexpr int kDmaPerTile = TI + TJ;  // load instructions per wavefront and tile
    extern __shared__ __attribute__((aligned(16))) float lds_f[];
    lds_char* lds_base = (lds_char*)lds_f;
    const uint32_t lds_addr0 = (uint32_t)(uintptr_t)lds_base;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int M = args.M, N = args.N, K = args.K;
    // the last tile of a row or column of tiles is moved back to end at the edge (it overlaps its neighbour;
    // both compute the shared elements from the same operands in the same order)
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
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
    int m0 = (first_m + in_group % gsz) * BM;
    int n0 = (in_group / gsz) * BN;
    m0 = m0 + BM > M ? M - BM : m0;
    n0 = n0 + BN > N ? N - BN : n0;

    const int kt_per_step = K / kBK;
    const int KT = kt_per_step * args.n_steps;
    const uint32_t a_voff = lane_voff<A_KSLOW, TI>(lane, wave, args.lda, m0);
    const uint32_t b_voff = lane_voff<B_KSLOW, TJ>(lane, wave, args.ldb, n0);
    const int64_t lda_bytes = args.lda * 4, ldb_bytes = args.ldb * 4;

    Reader<A_KSLOW, TI> ra;
    Reader<B_KSLOW, TJ> rb;
    ra.init(lane, wm * (BM / 2));
    rb.init(lane, wn * (BN / 2));

    f32x16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // the tile whose loads are issued next; past the last tile the position stays on it (harmless duplicate
    // loads into a free stage keep the load counting the same in every iteration)
    int is_kt = 0, is_step = 0, is_k0 = 0, is_stage = 0;
    const char* is_a = reinterpret_cast<const char*>(args.A[0]);
    const char* is_b = reinterpret_cast<const char*>(args.B[0]);
    auto issue_advance = [&]() {
        if (is_kt + 1 < KT) {
            ++is_kt;
            is_k0 += kBK;
            if (is_k0 >= K) {
                is_k0 = 0;
                ++is_step;
                is_a = reinterpret_cast<const char*>(gemm_bf16::pick_ptr(args.A, is_step));
                is_b = reinterpret_cast<const char*>(gemm_bf16::pick_ptr(args.B, is_step));
            }
        }
        is_stage = (is_stage + 1 == NS) ? 0 : is_stage + 1;
    };

    // prologue: tiles 0 .. NS-3 in flight, plus the A part of tile NS-2
    for (int p = 0; p < NS - 2; ++p) {
        const uint32_t st = lds_addr0 + is_stage * kStageBytes;
        gemm_bf16::static_for<TI>([&](auto I) { dma_one<A_KSLOW, TI, I.value>(is_a, lda_bytes, is_k0, a_voff, st, wave); });
        gemm_bf16::static_for<TJ>([&](auto I) { dma_one<B_KSLOW, TJ, I.value>(is_b, ldb_bytes, is_k0, b_voff, st + kOperA, wave); });
        issue_advance();
    }
    {
        const uint32_t st = lds_addr0 + is_stage * kStageBytes;
        gemm_bf16::static_for<TI>([&](auto I) { dma_one<A_KSLOW, TI, I.value>(is_a, lda_bytes, is_k0, a_voff, st, wave); });
    }
    dma_wait<kDmaPerTile*(NS - 3) + TI>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    constexpr int NRA = Reader<A_KSLOW, TI>::kReads, NRB = Reader<B_KSLOW, TJ>::kReads;
    Frag a_lo, a_hi, b_lo, b_hi;
    gemm_bf16::static_for<NRA>([&](auto q) { ra.template read<q.value, false>(lds_base, a_lo); });
    gemm_bf16::static_for<NRB>([&](auto q) { rb.template read<q.value, false>(lds_base + kOperA, b_lo); });

    constexpr int NM = 4 * TI * TJ;            // products of a half stage
    constexpr int NOPS = NRA + NRB + TI + TJ;  // memory instructions of a stage, spread evenly behind them
    constexpr int NOP1 = NRA + NRB + TJ, NOP2 = TI + NRA + NRB;
    static_assert(NOP1 + NOP2 == 2 * NOPS - TI - TJ, "operation count");
    int cur = 0;
    for (int kt = 0; kt < KT; ++kt) {
        lds_char* sa = lds_base + cur * kStageBytes;
        lds_char* sb = sa + kOperA;
        const int nxt = (cur + 1 == NS) ? 0 : cur + 1;
        lds_char* na = lds_base + nxt * kStageBytes;
        lds_char* nb = na + kOperA;

        // ---- products of steps 0..3; behind them the reads of steps 4..7 and the B part of the tile whose
        //      A part went out in the previous iteration
        CW_F32_PIN();
        {
            const uint32_t st = lds_addr0 + is_stage * kStageBytes;
            gemm_bf16::static_for<NM>([&](auto qq) {
                constexpr int Q = qq.value, S = Q / (TI * TJ), I = (Q / TJ) % TI, J = Q % TJ;
                acc[I][J] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_lo.v[I][S], b_lo.v[J][S], acc[I][J], 0, 0, 0);
                constexpr int first = Q * NOP1 / NM, last = (Q + 1) * NOP1 / NM;
                gemm_bf16::static_for<last - first>([&](auto oo) {
                    constexpr int O = first + oo.value;
                    if constexpr (O < NRA) ra.template read<O, true>(sa, a_hi);
                    else if constexpr (O < NRA + NRB) rb.template read<O - NRA, true>(sb, b_hi);
                    else dma_one<B_KSLOW, TJ, O - NRA - NRB>(is_b, ldb_bytes, is_k0, b_voff, st + kOperA, wave);
                });
                CW_F32_PIN();
            });
            issue_advance();
        }
        // ---- tile kt+1 complete for everybody, stage of tile kt-1 free
        dma_wait<kDmaPerTile*(NS - 3)>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        CW_F32_PIN();
        // ---- products of steps 4..7; behind them the A part of tile kt+NS-1 and the reads of (kt+1, steps 0..3)
        {
            const uint32_t st = lds_addr0 + is_stage * kStageBytes;
            gemm_bf16::static_for<NM>([&](auto qq) {
                constexpr int Q = qq.value, S = Q / (TI * TJ), I = (Q / TJ) % TI, J = Q % TJ;
                acc[I][J] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_hi.v[I][S], b_hi.v[J][S], acc[I][J], 0, 0, 0);
                constexpr int first = Q * NOP2 / NM, last = (Q + 1) * NOP2 / NM;
                gemm_bf16::static_for<last - first>([&](auto oo) {
                    constexpr int O = first + oo.value;
                    if constexpr (O < TI) dma_one<A_KSLOW, TI, O>(is_a, lda_bytes, is_k0, a_voff, st, wave);
                    else if constexpr (O < TI + NRA) ra.template read<O - TI, false>(na, a_lo);
                    else rb.template read<O - TI - NRA, false>(nb, b_lo);
                });
                CW_F32_PIN();
            });
        }
        cur = nxt;
    }
    dma_wait<0>();
    __syncthreads();
    // acc[i][j][v]: row m0 + wm*(BM/2) + i*32 + 8 (v/4) + 4 (lane/32) + v%4, column n0 + wn*(BN/2) + j*32 + lane%32
    float* patch = lds_f + wave * 32 * kPatchPitch;
    gemm_bf16::static_for<TI * TJ>([&](auto b) {
        constexpr int I = b.value / TJ, J = b.value % TJ;
        store_block(acc[I][J], patch, args, epilogue, m0 + wm * (BM / 2) + I * 32, n0 + wn * (BN / 2) + J * 32, lane);
    });
}

template <int TI, int TJ, bool AS, bool BS>
int launch(const GemmArgs& g, int epilogue, hipStream_t s) {
    RingArgs r = {};
    for (int i = 0; i < g.n_steps && i < kRingMaxSteps; ++i) { r.A[i] = g.A[i]; r.B[i] = g.B[i]; }
    for (int i = 0; i < g.n_addends && i < kRingMaxAddends; ++i) r.addend[i] = g.addend[i];
    r.bias = g.bias; r.C = g.C; r.preact = g.preact;
    r.lda = g.lda; r.ldb = g.ldb; r.ldc = g.ldc; r.ldp = g.ldp; r.ldadd = g.ldadd;
    r.M = g.M; r.N = g.N; r.K = g.K; r.n_steps = g.n_steps; r.n_addends = g.n_addends;
    r.vec_bias = 1; r.vec_add = 1; r.k_tail = 0; r.partial = nullptr;
    auto kern = gemm_f32_ring_kernel<TI, TJ, AS, BS>;
    constexpr int stages = kStages * (oper_bytes(TI) + oper_bytes(TJ));
    constexpr int patches = 4 * 32 * kPatchPitch * 4;
    constexpr int lds = stages > patches ? stages : patches;
    static_assert(lds <= 160 * 1024, "LDS image does not fit the CU");
    if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)(lds), "gemm_f32_ring"); lrc != CW_OK) return lrc;
    const int tiles = ((g.M + 64 * TI - 1) / (64 * TI)) * ((g.N + 64 * TJ - 1) / (64 * TJ));
    hipLaunchKernelGGL(kern, dim3(((tiles + 7) / 8) * 8), dim3(kThreads), lds, s, r, epilogue);
    return check_launch("gemm_f32_ring_kernel");
}

template <int TI, int TJ>
int launch_layout(const GemmArgs& g, int layout, int epilogue, hipStream_t s) {
    switch (layout) {
        case CW_NN: return launch<TI, TJ, false, true>(g, epilogue, s);
        case CW_NT: return launch<TI, TJ, false, false>(g, epilogue, s);
        case CW_TN: return launch<TI, TJ, true, true>(g, epilogue, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

}  // namespace ring

template <int BM, bool AK, bool BK_, bool GUARD>
int launch_f32(const GemmArgs& args, int epilogue, hipStream_t s) {
    const int tiles = ((args.M + BM - 1) / BM) * ((args.N + kFBN - 1) / kFBN);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL((gemm_f32_kernel<BM, AK, BK_, GUARD>), dim3(grid), dim3(kFThreads), 0, s, args, epilogue);
    return check_launch("gemm_f32_kernel");
}

template <int BM, bool GUARD>
int launch_f32_layout(const GemmArgs& args, int layout, int epilogue, hipStream_t s) {
    switch (layout) {
        case CW_NN: return launch_f32<BM, true, false, GUARD>(args, epilogue, s);
        case CW_NT: return launch_f32<BM, true, true, GUARD>(args, epilogue, s);
        case CW_TN: return launch_f32<BM, false, false, GUARD>(args, epilogue, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

}  // namespace

int gemm_f32_launch(const GemmArgs& args, int layout, int epilogue, hipStream_t s) {
    if (epilogue < CW_EPI_NONE || epilogue > CW_EPI_BIAS_RELU)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    // ring kernel: many 256x256 tiles, every pointer and leading dimension good for 16-byte accesses, the
    // reduction a multiple of the stage's k extent, byte offsets within 32 bits
    {
        const int64_t tiles256 = ((int64_t)(args.M + 255) / 256) * ((args.N + 255) / 256);
        const int64_t max_dim = args.M > args.N ? (args.M > args.K ? args.M : args.K) : (args.N > args.K ? args.N : args.K);
        const bool fits32 = (max_dim + 64) * (args.lda > args.ldb ? args.lda : args.ldb) * 4 < ((int64_t)1 << 32);
        const bool all_vec = args.vec_a && args.vec_b && args.vec_c && (args.preact == nullptr || args.vec_p) &&
                             (args.n_addends == 0 || args.vec_add) &&
                             (args.bias == nullptr || (reinterpret_cast<uintptr_t>(args.bias) & 15u) == 0);
        static const bool ring_enabled = [] {
            const char* v = std::getenv("CW_GEMM_IMPL");
            return !(v != nullptr && std::strcmp(v, "staged") == 0);
        }();
        const bool ring_ok = ring_enabled && all_vec && fits32 && (args.N % 4) == 0 && (layout != CW_TN || (args.M % 4) == 0) &&
                             args.K >= ring::kBK && (args.K % ring::kBK) == 0 && args.n_steps >= 1 &&
                             args.n_steps <= kRingMaxSteps && args.n_addends <= kRingMaxAddends;
        // 256 x 256 tiles (one workgroup per compute unit) for long reductions over many tiles; 128 x 128 or
        // 128 x 64 (two per unit, one's prologue and epilogue under the other's products) for fewer tiles and for
        // short reductions (config-1 forward, K = 1024: 241 us against 256 us with the large tiles)
        const int64_t tiles128 = ((int64_t)(args.M + 127) / 128) * ((args.N + 127) / 128);
        const int64_t tiles128x64 = ((int64_t)(args.M + 127) / 128) * ((args.N + 63) / 64);
        if (ring_ok && tiles256 >= 128 && args.M >= 256 && args.N >= 256 && (int64_t)args.K * args.n_steps > 2048)
            return ring::launch_layout<4, 4>(args, layout, epilogue, s);
        if (ring_ok && tiles128 >= 384 && args.M >= 128 && args.N >= 128) return ring::launch_layout<2, 2>(args, layout, epilogue, s);
        if (ring_ok && tiles128x64 >= 256 && args.M >= 128 && args.N >= 64) return ring::launch_layout<2, 1>(args, layout, epilogue, s);
    }
    const bool vec = args.vec_a && args.vec_b && (args.N % kFBN) == 0 && (args.K % kFBK) == 0;
    // 256-row tiles when they still give every compute unit two tiles
    const int64_t tall_tiles = ((int64_t)(args.M + 255) / 256) * ((args.N + kFBN - 1) / kFBN);
    if (tall_tiles >= 512) {
        return (vec && (args.M % 256) == 0) ? launch_f32_layout<256, false>(args, layout, epilogue, s)
                                            : launch_f32_layout<256, true>(args, layout, epilogue, s);
    }
    return (vec && (args.M % 128) == 0) ? launch_f32_layout<128, false>(args, layout, epilogue, s)
                                        : launch_f32_layout<128, true>(args, layout, epilogue, s);
}

}  // namespace cw
