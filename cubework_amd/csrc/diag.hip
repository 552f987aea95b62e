// Measurement aid (libcubework_diag.so, loaded by bench.py only): the rate at which this GPU sustains the block GEMM's matrix instruction when nothing else
// is in the way. Every wavefront keeps 4 x 4 accumulator tiles (the register blocking of the ring kernel) and
// eight operand fragments of seeded random bf16 values in registers and issues v_mfma_f32_32x32x16_bf16 back to
// back: no global loads, no LDS, no barriers. With mode 1 the fragments are all zero (no switching activity in
// the multipliers). With mode 2 the eight fragments of every trip are read from LDS (64 KB of the same random
// values, 16-byte reads, the next trip's fragments requested before the current trip's MFMAs), which is the
// LDS traffic of the ring kernel's k loop: 8 KB per wavefront and 16 MFMAs. The result says what the power
// management of the board leaves of the 2516.6 TFLOP/s that the data sheet quotes at 2.4 GHz, for operands that
// toggle like the workload's, and what it leaves a kernel that also has to fetch them from LDS; bench.py reports
// both beside the GEMM kernel's own rate. Mode 3 is the register-only loop with the 16 x 16 x 32 instruction.
// Further down: two probes of what a SIMD / a compute unit can do at once (matrix and vector instructions of two
// wavefronts; LDS read rates of the two kinds of fragment read), the bounds of the attention kernels.
#include "cw_common.h"
#include "gemm_bf16_kernel.h"

namespace cw {
namespace {

using gemm_bf16::bf16x8_t;
using gemm_bf16::f32x16_t;

__device__ __forceinline__ uint32_t mix(uint32_t x) {
    x ^= x >> 15;
    x *= 2246822519u;
    x ^= x >> 13;
    x *= 3266489917u;
    x ^= x >> 16;
    return x;
}

// a bf16 pair with the magnitudes of N(0, scale): sum of four uniform 16-bit numbers per value
__device__ __forceinline__ uint32_t random_bf16_pair(uint32_t seed, float scale) {
    uint32_t out = 0;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t x = mix(seed * 2u + h), y = mix(x + 0x9e3779b9u);
        const float f = (float)((int)(x & 0xffff) + (int)(x >> 16) + (int)(y & 0xffff) + (int)(y >> 16) - 131070) * (scale / 37837.0f);
        out |= (__float_as_uint(f) >> 16) << (16 * h);
    }
    return out;
}

template <bool LDS>
__global__ __launch_bounds__(256) void mfma_rate_kernel(int iters, int zeros, float* __restrict__ sink) {
    __shared__ __attribute__((aligned(16))) uint32_t frag_lds[LDS ? 16384 : 4];  // 64 fragments of 1 KB
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    bf16x8_t a[4], b[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        uint32_t wa[4], wb[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            wa[d] = zeros ? 0u : random_bf16_pair(gid * 64u + t * 8u + d, 1.0f);
            wb[d] = zeros ? 0u : random_bf16_pair(gid * 64u + 32u + t * 8u + d, 0.02f);
        }
        a[t] = __builtin_bit_cast(bf16x8_t, (u32x4){wa[0], wa[1], wa[2], wa[3]});
        b[t] = __builtin_bit_cast(bf16x8_t, (u32x4){wb[0], wb[1], wb[2], wb[3]});
    }
    if constexpr (LDS) {
        // fragment f of the block's 64: lanes' 16-byte pieces side by side, A fragments (magnitude 1) in the even
        // slots, B fragments (0.02) in the odd ones
        for (int i = threadIdx.x; i < 16384; i += 256) {
            const int f = i >> 8;
            frag_lds[i] = random_bf16_pair(blockIdx.x * 16384u + (uint32_t)i, (f & 1) ? 0.02f : 1.0f);
        }
        __syncthreads();
    }
    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    auto frag = [&](int slot) {  // slot < 64
        return *reinterpret_cast<const bf16x8_t*>(reinterpret_cast<const char*>(frag_lds) + slot * 1024 + lane * 16);
    };
    for (int it = 0; it < iters; ++it) {
        bf16x8_t an[4], bn[4];
        if constexpr (LDS) {
            // the next trip's fragments: the wavefront walks its 16 slots (8 A, 8 B) two trips round
            const int base = wave * 16 + ((it & 1) << 3);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                an[t] = frag(base + 2 * t);
                bn[t] = frag(base + 2 * t + 1);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int js = (i & 1) ? 3 - j : j;
                acc[i][js] = gemm_bf16::mfma_32x32x16<bf16_t>(b[js], a[i], acc[i][js]);
            }
        if constexpr (LDS) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                a[t] = an[t];
                b[t] = bn[t];
            }
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[i][j][e];
    if (sink != nullptr) sink[gid] = s;  // keeps the products alive
}

// The same FLOP per trip from the other bf16 matrix instruction, v_mfma_f32_16x16x32_bf16: 8 x 4 accumulator
// tiles of 16 x 16 and 32 instructions per trip, random operands in registers. Says whether the choice of
// instruction shape changes what the board sustains (time and energy per FLOP).
__global__ __launch_bounds__(256) void mfma16_rate_kernel(int iters, float* __restrict__ sink) {
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    bf16x8_t a[8], b[4];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        uint32_t w[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) w[d] = random_bf16_pair(gid * 64u + t * 4u + d, 1.0f);
        a[t] = __builtin_bit_cast(bf16x8_t, (u32x4){w[0], w[1], w[2], w[3]});
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        uint32_t w[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) w[d] = random_bf16_pair(gid * 64u + 32u + t * 4u + d, 0.02f);
        b[t] = __builtin_bit_cast(bf16x8_t, (u32x4){w[0], w[1], w[2], w[3]});
    }
    f32x4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int js = (i & 1) ? 3 - j : j;
                acc[i][js] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[js], a[i], acc[i][js], 0, 0, 0);
            }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) s += acc[i][j][e];
    if (sink != nullptr) sink[gid] = s;
}

// ---- two facts about a gfx950 SIMD / CU that bound the attention kernels -------------------------------------------
// (1) How far matrix and vector instructions of DIFFERENT wavefronts on one SIMD overlap. Workgroups of 8 wavefronts,
// two per SIMD: wavefronts 0-3 issue four independent 32x32x16 MFMAs per trip (128 cycles of the matrix pipe),
// wavefronts 4-7 issue 32 vector instructions per trip in 8 independent chains (v_fma_f32, or v_exp_f32). roles bit 0:
// the MFMA wavefronts work, bit 1: the vector wavefronts work; the others leave at once.
template <int VOP>
__global__ __launch_bounds__(512) void overlap_kernel(int iters, int roles, float* __restrict__ sink) {
    const int wave = threadIdx.x >> 6;
    float r = 0.0f;
    if (wave < 4) {
        if (!(roles & 1)) return;
        bf16x8_t a, b;
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        a = __builtin_bit_cast(bf16x8_t, (u32x4){random_bf16_pair(threadIdx.x, 1.0f), random_bf16_pair(threadIdx.x + 512, 1.0f),
                                                 random_bf16_pair(threadIdx.x + 1024, 1.0f), random_bf16_pair(threadIdx.x + 1536, 1.0f)});
        b = __builtin_bit_cast(bf16x8_t, (u32x4){random_bf16_pair(threadIdx.x + 2048, 0.02f), random_bf16_pair(threadIdx.x + 2560, 0.02f),
                                                 random_bf16_pair(threadIdx.x + 3072, 0.02f), random_bf16_pair(threadIdx.x + 3584, 0.02f)});
        f32x16_t c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        for (int it = 0; it < iters; ++it) {
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %4, %5, %0\n v_mfma_f32_32x32x16_bf16 %1, %4, %5, %1\n"
                         "v_mfma_f32_32x32x16_bf16 %2, %4, %5, %2\n v_mfma_f32_32x32x16_bf16 %3, %4, %5, %3\n"
                         : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(a), "v"(b));
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) r += c0[e] + c1[e] + c2[e] + c3[e];
    } else {
        if (!(roles & 2)) return;
        float x0 = threadIdx.x * 1e-3f, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3, x4 = x0 + 4, x5 = x0 + 5, x6 = x0 + 6, x7 = x0 + 7;
        const float m = 0.999f, ad = 1e-3f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if constexpr (VOP == 0) {
                    asm volatile("v_fma_f32 %0, %0, %8, %9\n v_fma_f32 %1, %1, %8, %9\n v_fma_f32 %2, %2, %8, %9\n v_fma_f32 %3, %3, %8, %9\n"
                                 "v_fma_f32 %4, %4, %8, %9\n v_fma_f32 %5, %5, %8, %9\n v_fma_f32 %6, %6, %8, %9\n v_fma_f32 %7, %7, %8, %9\n"
                                 : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3), "+v"(x4), "+v"(x5), "+v"(x6), "+v"(x7) : "v"(m), "v"(ad));
                } else {
                    asm volatile("v_exp_f32 %0, %0\n v_exp_f32 %1, %1\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n"
                                 "v_exp_f32 %4, %4\n v_exp_f32 %5, %5\n v_exp_f32 %6, %6\n v_exp_f32 %7, %7\n"
                                 : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3), "+v"(x4), "+v"(x5), "+v"(x6), "+v"(x7));
                }
            }
        }
        r = x0 + x1 + x2 + x3 + x4 + x5 + x6 + x7;
    }
    if (sink != nullptr) sink[blockIdx.x * 512 + threadIdx.x] = r;
}

// (2) What a compute unit reads from LDS per second with 8 wavefronts streaming 8 KB per trip each: 16-byte reads of
// consecutive lanes (ds_read_b128, the k-contiguous fragments) or the transposing 8-byte read (ds_read_b64_tr_b16, the
// fragments of an operand stored with k as the slow index), both free of bank conflicts.
template <int TR>
__global__ __launch_bounds__(512) void lds_rate_kernel(int iters, int* __restrict__ sink) {
    __shared__ __attribute__((aligned(16))) char buf[65536];
    for (int i = threadIdx.x; i < 65536 / 4; i += 512) reinterpret_cast<uint32_t*>(buf)[i] = mix((uint32_t)i);
    __syncthreads();
    typedef __attribute__((address_space(3))) char lds_c;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    lds_c* base = (lds_c*)buf + wave * 8192;
    int acc = 0;
    if constexpr (TR == 0) {
        lds_c* p = base + lane * 16;
        for (int it = 0; it < iters; ++it) {
            asm volatile("" : "+v"(p));  // keeps the reads inside the loop
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const i32x4 v = *(__attribute__((address_space(3))) i32x4*)(p + u * 1024);
                acc ^= v.x ^ v.y ^ v.z ^ v.w;
            }
        }
    } else {
        // 16 lanes cover 128 consecutive bytes; the four groups of 16 lanes sit 384 bytes apart (banks 0-31 / 32-63 in turn)
        lds_c* p = base + (lane >> 4) * 384 + (lane & 15) * 8;
        for (int it = 0; it < iters; ++it) {
            asm volatile("" : "+v"(p));
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p + (u & 7) * 512 + (u >> 3) * 2048));
                acc ^= (int)v.x ^ ((int)v.y << 4) ^ ((int)v.z << 8) ^ ((int)v.w << 12);
            }
        }
    }
    if (sink != nullptr) sink[blockIdx.x * 512 + threadIdx.x] = acc;
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int64_t cw_diag_mfma_rate_flop(int iters) {
    // 1024 wavefronts x 16 instructions per trip x 32 x 32 x 16 x 2 (mode 3: 32 instructions x 16 x 16 x 32 x 2)
    return iters <= 0 ? 0 : (int64_t)iters * 1024 * 16 * 32768;
}

extern "C" int cw_diag_mfma_rate(int iters, int mode, float* sink, void* stream) {
    if (mode < 0 || mode > 3) return fail(CW_ERR_INVALID, "cw_diag_mfma_rate: mode %d outside [0, 3]", mode);
    if (iters <= 0 || iters > (1 << 24)) return fail(CW_ERR_INVALID, "cw_diag_mfma_rate: iters=%d outside [1, 2^24]", iters);
    if (const int drc = require_gfx950("cw_diag_mfma_rate"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    // one workgroup of four wavefronts per compute unit, one wavefront per SIMD: 256 x 256 threads
    if (mode == 3) hipLaunchKernelGGL(mfma16_rate_kernel, dim3(256), dim3(256), 0, s, iters, sink);
    else if (mode == 2) hipLaunchKernelGGL(mfma_rate_kernel<true>, dim3(256), dim3(256), 0, s, iters, 0, sink);
    else hipLaunchKernelGGL(mfma_rate_kernel<false>, dim3(256), dim3(256), 0, s, iters, mode, sink);
    return check_launch("mfma_rate_kernel");
}

// sink: at least 256 x 512 floats. roles: 1 = MFMA wavefronts only, 2 = vector wavefronts only, 3 = both. vop: 0 = v_fma_f32,
// 1 = v_exp_f32. Every trip is 4 matrix instructions and / or 32 vector instructions per SIMD.
extern "C" int cw_diag_overlap(int iters, int roles, int vop, float* sink, void* stream) {
    if (roles < 1 || roles > 3 || vop < 0 || vop > 1) return fail(CW_ERR_INVALID, "cw_diag_overlap: roles %d / vop %d", roles, vop);
    if (iters <= 0 || iters > (1 << 24)) return fail(CW_ERR_INVALID, "cw_diag_overlap: iters=%d outside [1, 2^24]", iters);
    if (sink == nullptr) return fail(CW_ERR_INVALID, "cw_diag_overlap: sink is NULL");
    if (const int drc = require_gfx950("cw_diag_overlap"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (vop == 0) hipLaunchKernelGGL(overlap_kernel<0>, dim3(256), dim3(512), 0, s, iters, roles, sink);
    else hipLaunchKernelGGL(overlap_kernel<1>, dim3(256), dim3(512), 0, s, iters, roles, sink);
    return check_launch("overlap_kernel");
}

// sink: at least 256 x 512 ints. transposing: 0 = ds_read_b128, 1 = ds_read_b64_tr_b16. Every trip reads 64 KB per
// compute unit (8 wavefronts x 8 KB); cw_diag_lds_rate_bytes gives the bytes one call reads per compute unit.
extern "C" int64_t cw_diag_lds_rate_bytes(int iters) { return iters <= 0 ? 0 : (int64_t)iters * 65536; }
extern "C" int cw_diag_lds_rate(int iters, int transposing, int* sink, void* stream) {
    if (transposing < 0 || transposing > 1) return fail(CW_ERR_INVALID, "cw_diag_lds_rate: transposing %d", transposing);
    if (iters <= 0 || iters > (1 << 24)) return fail(CW_ERR_INVALID, "cw_diag_lds_rate: iters=%d outside [1, 2^24]", iters);
    if (sink == nullptr) return fail(CW_ERR_INVALID, "cw_diag_lds_rate: sink is NULL");
    if (const int drc = require_gfx950("cw_diag_lds_rate"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (transposing == 0) hipLaunchKernelGGL(lds_rate_kernel<0>, dim3(256), dim3(512), 0, s, iters, sink);
    else hipLaunchKernelGGL(lds_rate_kernel<1>, dim3(256), dim3(512), 0, s, iters, sink);
    return check_launch("lds_rate_kernel");
}
