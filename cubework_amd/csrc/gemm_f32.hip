// fp32 variant of the SUMMA block GEMM for gfx950 (v_mfma_f32_32x32x2_f32:
// exact fp32 products, fp32 accumulation) for the layers' fp32 path, where
// results have to agree with torch's fp32 matmul to ~1e-6.
// 128x128 tile per 256-thread block, 2x2 wavefronts of 64x64, k tiles of 16
// (flattened over the k-steps), operands in LDS as [k][row] so a fragment read
// is 32 consecutive floats, register-staged prefetch with two LDS stages.
#include "cw_common.h"
#include "gemm.h"

namespace cw {

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kFBM = 128, kFBN = 128, kFBK = 16;
constexpr int kFP = 132;  // floats per LDS k-row (128 + 4)
constexpr int kFThreads = 256;

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
template <bool KCONTIG, bool GUARD>
__device__ __forceinline__ void f32_g2r(float4 (&reg)[2], const float* __restrict__ base, int64_t ld, int row0,
                                        int k0, int rmax, int kmax, int tid, bool vec_ok) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int c = it * kFThreads + tid;
        if constexpr (KCONTIG) {
            const int row = row0 + (c >> 2), k = k0 + (c & 3) * 4;
            reg[it] = GUARD ? load4_guarded(base, ld, row, k, rmax, kmax, vec_ok)
                            : *reinterpret_cast<const float4*>(base + (int64_t)row * ld + k);
        } else {
            const int k = k0 + (c >> 5), row = row0 + (c & 31) * 4;
            reg[it] = GUARD ? load4_guarded(base, ld, k, row, kmax, rmax, vec_ok)
                            : *reinterpret_cast<const float4*>(base + (int64_t)k * ld + row);
        }
    }
}

template <bool KCONTIG>
__device__ __forceinline__ void f32_r2s(const float4 (&reg)[2], float* __restrict__ lds, int tid) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int c = it * kFThreads + tid;
        if constexpr (KCONTIG) {
            const int r = c >> 2, kc = (c & 3) * 4;
            lds[(kc + 0) * kFP + r] = reg[it].x;
            lds[(kc + 1) * kFP + r] = reg[it].y;
            lds[(kc + 2) * kFP + r] = reg[it].z;
            lds[(kc + 3) * kFP + r] = reg[it].w;
        } else {
            const int k = c >> 5, r = (c & 31) * 4;
            *reinterpret_cast<float4*>(lds + k * kFP + r) = reg[it];
        }
    }
}

template <bool A_KCONTIG, bool B_KCONTIG, bool GUARD>
__global__ __launch_bounds__(kFThreads) void gemm_f32_kernel(const GemmArgs args, int epilogue) {
    constexpr int OPER = kFBK * kFP;
    __shared__ __attribute__((aligned(16))) float lds[2 * 2 * OPER];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int M = args.M, N = args.N, K = args.K;
    const int tiles_m = (M + kFBM - 1) / kFBM;
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
    const int m0 = (first_m + in_group % gsz) * kFBM;
    const int n0 = (in_group / gsz) * kFBN;

    const int kt_per_step = (K + kFBK - 1) / kFBK;
    const int KT = kt_per_step * args.n_steps;
    const bool vec_a = args.vec_a != 0, vec_b = args.vec_b != 0;

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    float4 ra[2], rb[2];
    auto issue_loads = [&](int kt) {
        const int step = kt / kt_per_step;
        const int k0 = (kt - step * kt_per_step) * kFBK;
        f32_g2r<A_KCONTIG, GUARD>(ra, reinterpret_cast<const float*>(args.A[step]), args.lda, m0, k0, M, K, tid, vec_a);
        f32_g2r<B_KCONTIG, GUARD>(rb, reinterpret_cast<const float*>(args.B[step]), args.ldb, n0, k0, N, K, tid, vec_b);
    };
    auto commit_loads = [&](int stage) {
        float* s = lds + stage * 2 * OPER;
        f32_r2s<A_KCONTIG>(ra, s, tid);
        f32_r2s<B_KCONTIG>(rb, s + OPER, tid);
    };

    if (KT > 0) {
        issue_loads(0);
        commit_loads(0);
    }
    __syncthreads();

    const int a_off = (lane >> 5) * kFP + wm * 64 + (lane & 31);
    const int b_off = OPER + (lane >> 5) * kFP + wn * 64 + (lane & 31);
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) issue_loads(kt + 1);
        const float* s = lds + cur * 2 * OPER;
#pragma unroll
        for (int kk = 0; kk < kFBK / 2; ++kk) {
            float af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) af[i] = s[a_off + 2 * kk * kFP + i * 32];
#pragma unroll
            for (int j = 0; j < 2; ++j) bf[j] = s[b_off + 2 * kk * kFP + j * 32];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < KT) commit_loads(cur ^ 1);
        __syncthreads();
    }

    // acc[i][j][v]: row m = m0 + wm*64 + i*32 + 8*(v/4) + 4*(lane>>5) + v%4
    //               col n = n0 + wn*64 + j*32 + (lane & 31)
    const float* bias = reinterpret_cast<const float*>(args.bias);
    float* C = reinterpret_cast<float*>(args.C);
    float* P = reinterpret_cast<float*>(args.preact);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        if (col >= N) continue;
        const float bv = (epilogue != CW_EPI_NONE && bias != nullptr) ? bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row >= M) continue;
                float x = acc[i][j][v] + bv;
                for (int a = 0; a < args.n_addends; ++a)
                    x += reinterpret_cast<const float*>(args.addend[a])[(int64_t)row * args.ldadd + col];
                if (P != nullptr) P[(int64_t)row * args.ldp + col] = x;
                switch (epilogue) {
                    case CW_EPI_BIAS_GELU_TANH: x = gelu_tanh(x); break;
                    case CW_EPI_BIAS_GELU_ERF: x = gelu_erf(x); break;
                    case CW_EPI_BIAS_RELU: x = x > 0.0f ? x : 0.0f; break;
                    default: break;
                }
                C[(int64_t)row * args.ldc + col] = x;
            }
    }
}

template <bool AK, bool BK_, bool GUARD>
int launch_f32(const GemmArgs& args, int epilogue, hipStream_t s) {
    const int tiles = ((args.M + kFBM - 1) / kFBM) * ((args.N + kFBN - 1) / kFBN);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL((gemm_f32_kernel<AK, BK_, GUARD>), dim3(grid), dim3(kFThreads), 0, s, args, epilogue);
    return check_launch("gemm_f32_kernel");
}

template <bool GUARD>
int launch_f32_layout(const GemmArgs& args, int layout, int epilogue, hipStream_t s) {
    switch (layout) {
        case CW_NN: return launch_f32<true, false, GUARD>(args, epilogue, s);
        case CW_NT: return launch_f32<true, true, GUARD>(args, epilogue, s);
        case CW_TN: return launch_f32<false, false, GUARD>(args, epilogue, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

}  // namespace

int gemm_f32_launch(const GemmArgs& args, int layout, int epilogue, hipStream_t s) {
    if (epilogue < CW_EPI_NONE || epilogue > CW_EPI_BIAS_RELU)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    const bool exact = args.vec_a && args.vec_b && (args.M % kFBM) == 0 && (args.N % kFBN) == 0 && (args.K % kFBK) == 0;
    return exact ? launch_f32_layout<false>(args, layout, epilogue, s) : launch_f32_layout<true>(args, layout, epilogue, s);
}

}  // namespace cw
