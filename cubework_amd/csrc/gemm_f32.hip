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
#include "cw_common.h"
#include "gemm.h"

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
