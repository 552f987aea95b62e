// Shared device/host helpers for the gfx950 kernels of libcubework_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cubework_hip.h"

namespace cw {

// ---- host side: thread-local error text --------------------------------
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);
// CW_OK when the current device runs this library's gfx950 code objects; otherwise CW_ERR_DEVICE with the
// message set (no device, or another architecture). The answer is cached per device.
int require_gfx950(const char* who);
// Raises a kernel's dynamic-LDS limit to `bytes`. The attribute is sticky, so it is set once per kernel and
// device (and again only for a larger size): later launches make no runtime call for it, which also keeps
// a non-stream API call out of regions a caller captures into a graph after a first eager call.
int ensure_dynamic_lds(const void* kernel, int bytes, const char* what);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- element types -------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};

// IEEE half precision: what torch's autocast hands the GEMM-type operators by default.
struct f16_t {
    uint16_t bits;
};

template <typename T>
struct elem;

template <>
struct elem<bf16_t> {
    static constexpr int kVec = 8;  // elements per 16-byte vector
};
template <>
struct elem<f16_t> {
    static constexpr int kVec = 8;
};
template <>
struct elem<float> {
    static constexpr int kVec = 4;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Round-to-nearest-even, the rounding torch uses for float -> bfloat16
// (lowers to v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    __bf16 b = static_cast<__bf16>(f);
    return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, b));
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// fp16 <-> fp32: v_cvt_f32_f16 is exact, v_cvt_f16_f32 rounds to nearest even (the mode the kernels run in),
// overflow goes to infinity as torch's conversion does.
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<_Float16>(f)));
}
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    const half2_t h = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return __builtin_bit_cast(uint32_t, h);
}

// The two 16-bit element types share every kernel; what differs is the conversion.
template <typename T>
struct half_conv;
template <>
struct half_conv<bf16_t> {
    static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
    static __device__ __forceinline__ float one(uint32_t bits) { return bf16_bits_to_f32(bits); }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_bf16x2(a, b); }
};
template <>
struct half_conv<f16_t> {
    static __device__ __forceinline__ float lo(uint32_t w) { return f16_bits_to_f32(w & 0xffffu); }
    static __device__ __forceinline__ float hi(uint32_t w) { return f16_bits_to_f32(w >> 16); }
    static __device__ __forceinline__ float one(uint32_t bits) { return f16_bits_to_f32(bits); }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_f16x2(a, b); }
};

__device__ __forceinline__ float load_elem(const f16_t* p) { return f16_bits_to_f32(p->bits); }
__device__ __forceinline__ void store_elem(f16_t* p, float v) { p->bits = static_cast<uint16_t>(f32_to_f16_bits(v)); }
__device__ __forceinline__ float load_elem(const bf16_t* p) { return bf16_bits_to_f32(p->bits); }
__device__ __forceinline__ float load_elem(const float* p) { return *p; }
__device__ __forceinline__ void store_elem(bf16_t* p, float v) { p->bits = static_cast<uint16_t>(f32_to_bf16_bits(v)); }
__device__ __forceinline__ void store_elem(float* p, float v) { *p = v; }

// 16-byte vector load of kVec consecutive elements into floats. p must be
// 16-byte aligned.
__device__ __forceinline__ void load_vec(const bf16_t* p, float (&v)[8]) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(u.x << 16);
    v[1] = __uint_as_float(u.x & 0xffff0000u);
    v[2] = __uint_as_float(u.y << 16);
    v[3] = __uint_as_float(u.y & 0xffff0000u);
    v[4] = __uint_as_float(u.z << 16);
    v[5] = __uint_as_float(u.z & 0xffff0000u);
    v[6] = __uint_as_float(u.w << 16);
    v[7] = __uint_as_float(u.w & 0xffff0000u);
}
__device__ __forceinline__ void load_vec(const f16_t* p, float (&v)[8]) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        v[2 * d] = half_conv<f16_t>::lo(w[d]);
        v[2 * d + 1] = half_conv<f16_t>::hi(w[d]);
    }
}
__device__ __forceinline__ void store_vec(f16_t* p, const float (&v)[8]) {
    uint4 u;
    u.x = pack_f16x2(v[0], v[1]);
    u.y = pack_f16x2(v[2], v[3]);
    u.z = pack_f16x2(v[4], v[5]);
    u.w = pack_f16x2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = u;
}
__device__ __forceinline__ void load_vec(const float* p, float (&v)[4]) {
    const float4 u = *reinterpret_cast<const float4*>(p);
    v[0] = u.x;
    v[1] = u.y;
    v[2] = u.z;
    v[3] = u.w;
}
__device__ __forceinline__ void store_vec(bf16_t* p, const float (&v)[8]) {
    uint4 u;
    u.x = pack_bf16x2(v[0], v[1]);
    u.y = pack_bf16x2(v[2], v[3]);
    u.z = pack_bf16x2(v[4], v[5]);
    u.w = pack_bf16x2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = u;
}
__device__ __forceinline__ void store_vec(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

// ---- raw 16-byte moves for streaming kernels -----------------------------
// Data that a kernel touches exactly once goes through non-temporal loads and
// stores, which do not displace reusable lines from the caches.
typedef uint32_t raw16_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ raw16_t load_raw(const void* p) { return *reinterpret_cast<const raw16_t*>(p); }
__device__ __forceinline__ raw16_t load_raw_stream(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const raw16_t*>(p));
}
__device__ __forceinline__ void store_raw_stream(void* p, raw16_t u) {
    __builtin_nontemporal_store(u, reinterpret_cast<raw16_t*>(p));
}
__device__ __forceinline__ void unpack_raw(raw16_t u, float (&v)[8], const bf16_t*) {
    v[0] = __uint_as_float(u.x << 16);
    v[1] = __uint_as_float(u.x & 0xffff0000u);
    v[2] = __uint_as_float(u.y << 16);
    v[3] = __uint_as_float(u.y & 0xffff0000u);
    v[4] = __uint_as_float(u.z << 16);
    v[5] = __uint_as_float(u.z & 0xffff0000u);
    v[6] = __uint_as_float(u.w << 16);
    v[7] = __uint_as_float(u.w & 0xffff0000u);
}
__device__ __forceinline__ void unpack_raw(raw16_t u, float (&v)[8], const f16_t*) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        v[2 * d] = half_conv<f16_t>::lo(u[d]);
        v[2 * d + 1] = half_conv<f16_t>::hi(u[d]);
    }
}
__device__ __forceinline__ raw16_t pack_raw(const float (&v)[8], const f16_t*) {
    raw16_t u;
    u.x = pack_f16x2(v[0], v[1]);
    u.y = pack_f16x2(v[2], v[3]);
    u.z = pack_f16x2(v[4], v[5]);
    u.w = pack_f16x2(v[6], v[7]);
    return u;
}
__device__ __forceinline__ void unpack_raw(raw16_t u, float (&v)[4], const float*) {
    v[0] = __uint_as_float(u.x);
    v[1] = __uint_as_float(u.y);
    v[2] = __uint_as_float(u.z);
    v[3] = __uint_as_float(u.w);
}
__device__ __forceinline__ raw16_t pack_raw(const float (&v)[8], const bf16_t*) {
    raw16_t u;
    u.x = pack_bf16x2(v[0], v[1]);
    u.y = pack_bf16x2(v[2], v[3]);
    u.z = pack_bf16x2(v[4], v[5]);
    u.w = pack_bf16x2(v[6], v[7]);
    return u;
}
__device__ __forceinline__ raw16_t pack_raw(const float (&v)[4], const float*) {
    raw16_t u;
    u.x = __float_as_uint(v[0]);
    u.y = __float_as_uint(v[1]);
    u.z = __float_as_uint(v[2]);
    u.w = __float_as_uint(v[3]);
    return u;
}

// ---- loads straight into LDS ----------------------------------------------
// global_load_lds_dwordx4: lane l of the issuing wavefront fetches 16 bytes at gbase + voff and the load
// unit writes them at LDS address lds_addr + 16 l (M0 holds lds_addr): no staging registers, no LDS write
// instructions. The compiler does not see these loads (inline asm); a kernel that uses them counts them and
// waits with dma_wait<N> (at most N of this thread's loads still in flight; loads complete in issue order)
// before the barrier that publishes the data.
__device__ __forceinline__ void dma16(const char* gbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(gbase) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// ---- wavefront (64 lanes) reductions ------------------------------------
// Within a row of 16 lanes the partner values come through DPP operand
// modifiers of the adds themselves (no LDS traffic); the four row results are
// combined through lane reads. Every lane returns the same bits.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7-i of each 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15-i of each 16

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    v += dpp_move<kDppMirror>(v);
    const int iv = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(iv, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(iv, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(iv, 48));
    return (r0 + r1) + (r2 + r3);
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<kDppXor1>(v));
    v = fmaxf(v, dpp_move<kDppXor2>(v));
    v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_move<kDppMirror>(v));
    const int iv = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(iv, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(iv, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(iv, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// exp(x) through the hardware exp2; x <= 0 in every use here.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

// ---- activations ---------------------------------------------------------
__device__ __forceinline__ float tanh_fast(float x) {
    // tanh(x) = 1 - 2 / (exp(2x) + 1); saturates cleanly for |x| large.
    const float e = __builtin_amdgcn_exp2f(x * (2.0f * kLog2e));
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}
__device__ __forceinline__ float gelu_tanh(float x) {
    // 0.5 x (1 + tanh(u)) = x / (1 + exp(-2u)), u = sqrt(2/pi) (x + 0.044715 x^3):
    // two multiplies, one fma, one exp2, one add, one reciprocal, one multiply.
    const float a = -2.0f * 0.7978845608028654f * kLog2e;
    const float b = a * 0.044715f;
    const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(x * x, b, a));
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float gelu_tanh_grad(float x) {
    // gelu = x s with s = sigmoid(2u), u = k0 (x + k1 x^3):
    // gelu' = s + x s (1 - s) 2u',  2u' = 2 k0 (1 + 3 k1 x^2).
    // s (1 - s) is formed as s - s*s so that s = 0 (exp2 overflowed) gives 0.
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    const float a = -2.0f * k0 * kLog2e;
    const float b = a * k1;
    const float x2 = x * x;
    const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(x2, b, a));
    const float s = __builtin_amdgcn_rcpf(1.0f + e);
    const float ds = __builtin_fmaf(-s, s, s);
    const float up = __builtin_fmaf(x2, 6.0f * k0 * k1, 2.0f * k0);
    return __builtin_fmaf(x * ds, up, s);
}
__device__ __forceinline__ float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f)); }
__device__ __forceinline__ float gelu_erf_grad(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.7071067811865476f));
    const float pdf = 0.3989422804014327f * __expf(-0.5f * x * x);
    return cdf + x * pdf;
}

template <int ACT>
__device__ __forceinline__ float apply_act(float x) {
    if constexpr (ACT == CW_ACT_GELU_TANH) return gelu_tanh(x);
    if constexpr (ACT == CW_ACT_GELU_ERF) return gelu_erf(x);
    if constexpr (ACT == CW_ACT_RELU) return x < 0.0f ? 0.0f : x;  // NaN stays NaN, as torch.relu leaves it
    return x;
}
template <int ACT>
__device__ __forceinline__ float act_grad_of(float x) {
    if constexpr (ACT == CW_ACT_GELU_TANH) return gelu_tanh_grad(x);
    if constexpr (ACT == CW_ACT_GELU_ERF) return gelu_erf_grad(x);
    if constexpr (ACT == CW_ACT_RELU) return x > 0.0f ? 1.0f : 0.0f;
    return 1.0f;
}
__device__ __forceinline__ float act_grad(int act, float x) {
    switch (act) {
        case CW_ACT_GELU_TANH: return gelu_tanh_grad(x);
        case CW_ACT_GELU_ERF: return gelu_erf_grad(x);
        case CW_ACT_RELU: return x > 0.0f ? 1.0f : 0.0f;
        default: return 1.0f;
    }
}

// Calls f with a null pointer to the element type io_dtype names (CW_BF16, CW_F16, otherwise float):
// `with_elem_type(dt, [&](auto* tag) { using T = std::remove_pointer_t<decltype(tag)>; ... })`.
template <typename F>
int with_elem_type(int io_dtype, F&& f) {
    if (io_dtype == CW_BF16) return f((bf16_t*)nullptr);
    if (io_dtype == CW_F16) return f((f16_t*)nullptr);
    return f((float*)nullptr);
}

}  // namespace cw
