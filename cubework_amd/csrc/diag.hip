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
