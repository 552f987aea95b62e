// Bias-gradient column sums and the backward of the fused activation
// epilogue, for gfx950. Streaming kernels: a block owns a slab of rows and a
// tile of 64 vectors of columns, lanes keep their columns' sums in registers,
// wavefronts are combined in a fixed-order LDS tree, slabs by a finalize
// kernel (no atomics: bit-reproducible).
#include <atomic>
#include <mutex>
#include <type_traits>

#include "cw_common.h"
#include "gemm_plan.h"
#include "reduce_cols.h"

namespace cw {

namespace {

constexpr int64_t kGenericSlabRows = kColGenericSlabRows;  // rows per slab of the element-wise kernel (gemm_plan.h)

// MODE 0: column sums of dY. MODE 1: dPre = dY * ACT'(pre), column sums of dPre.
template <typename T, int MODE, int ACT>
__global__ __launch_bounds__(kColWaves * 64) void colsum_vec_kernel(
    int64_t M, int64_t N, const T* __restrict__ dY, int64_t ld_dy, const T* __restrict__ pre, int64_t ld_pre,
    T* __restrict__ dPre, int64_t ld_dpre, float* __restrict__ ws, int64_t rows_per_slab, int want_sum) {
    constexpr int V = elem<T>::kVec;
    extern __shared__ float lds_red[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t c0 = ((int64_t)blockIdx.x * 64 + lane) * V;
    const bool valid = c0 < N;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_slab;
    const int64_t r1 = (r0 + rows_per_slab < M) ? r0 + rows_per_slab : M;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.0f;
    if (valid) {
        // kColUnroll rows per wavefront are in flight at a time. The loads are
        // unconditional (a row past the slab reads the slab's last row and is
        // then dropped): loads under a branch would wait for one another.
        for (int64_t row = r0 + wave; row < r1; row += kColWaves * kColUnroll) {
            raw16_t d_raw[kColUnroll], p_raw[kColUnroll];
#pragma unroll
            for (int u = 0; u < kColUnroll; ++u) {
                const int64_t rr = row + u * kColWaves;
                const int64_t rc = rr < r1 ? rr : r1 - 1;
                d_raw[u] = load_raw_stream(dY + rc * ld_dy + c0);
                if constexpr (MODE == 1) p_raw[u] = load_raw_stream(pre + rc * ld_pre + c0);
            }
#pragma unroll
            for (int u = 0; u < kColUnroll; ++u) {
                const int64_t rr = row + u * kColWaves;
                const bool live = rr < r1;
                float dy[V];
                unpack_raw(d_raw[u], dy, (const T*)nullptr);
                if constexpr (MODE == 1) {
                    float p[V];
                    unpack_raw(p_raw[u], p, (const T*)nullptr);
#pragma unroll
                    for (int e = 0; e < V; ++e) dy[e] *= act_grad_of<ACT>(p[e]);
                    if (live) store_raw_stream(dPre + rr * ld_dpre + c0, pack_raw(dy, (const T*)nullptr));
                }
#pragma unroll
                for (int e = 0; e < V; ++e) acc[e] += live ? dy[e] : 0.0f;
            }
        }
    }
    if (!want_sum) return;
    block_tree_reduce<V, kColWaves>(acc, lds_red, wave, lane);
    if (wave == 0 && valid) {
        float* out = ws + (int64_t)blockIdx.y * N + c0;
#pragma unroll
        for (int e = 0; e < V; e += 4)
            *reinterpret_cast<float4*>(out + e) = make_float4(acc[e], acc[e + 1], acc[e + 2], acc[e + 3]);
    }
}

template <typename T, int MODE>
__global__ __launch_bounds__(256) void colsum_generic_kernel(int64_t M, int64_t N, const T* __restrict__ dY,
                                                             int64_t ld_dy, const T* __restrict__ pre,
                                                             int64_t ld_pre, T* __restrict__ dPre, int64_t ld_dpre,
                                                             int act, float* __restrict__ ws,
                                                             int64_t rows_per_slab, int want_sum) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= N) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_slab;
    const int64_t r1 = (r0 + rows_per_slab < M) ? r0 + rows_per_slab : M;
    float acc = 0.0f;
    for (int64_t row = r0; row < r1; ++row) {
        float d = load_elem(dY + row * ld_dy + c);
        if constexpr (MODE == 1) {
            d *= act_grad(act, load_elem(pre + row * ld_pre + c));
            store_elem(dPre + row * ld_dpre + c, d);
        }
        acc += d;
    }
    if (want_sum) ws[(int64_t)blockIdx.y * N + c] = acc;
}

// grid (ceil(C/64), nsets); 16 groups of 64 threads split the partials, each
// with 16 independent loads in flight, and are combined in a fixed order.
constexpr int kFinGroups = 16;
__global__ __launch_bounds__(kFinGroups * 64) void finalize_cols_kernel(const float* __restrict__ ws, int64_t nparts,
                                                                        int64_t part_stride, int64_t C,
                                                                        void* __restrict__ out0,
                                                                        void* __restrict__ out1, int out_dtype) {
    __shared__ float red[kFinGroups][64];
    const int lane = threadIdx.x & 63;
    const int grp = threadIdx.x >> 6;
    const int64_t c = (int64_t)blockIdx.x * 64 + lane;
    const int k = blockIdx.y;
    float acc = 0.0f;
    if (c < C) {
        const float* base = ws + (int64_t)k * C + c;
        // 16 loads in flight per batch; indices past the end re-read the last
        // partial and are dropped, so no load waits behind a branch.
        for (int64_t p = grp; p < nparts; p += 16 * kFinGroups) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int64_t q = p + u * kFinGroups;
                v[u] = base[(q < nparts ? q : nparts - 1) * part_stride];
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) acc += (p + u * kFinGroups < nparts) ? v[u] : 0.0f;
        }
    }
    red[grp][lane] = acc;
    __syncthreads();
    if (grp == 0 && c < C) {
        float total = red[0][lane];
#pragma unroll
        for (int g = 1; g < kFinGroups; ++g) total += red[g][lane];
        void* out = (k == 0) ? out0 : out1;
        if (out != nullptr) store_col_total(out, c, total, out_dtype);
    }
}

template <typename T, int MODE>
int colsum_impl(int64_t M, int64_t N, const void* dY, int64_t ld_dy, const void* pre, int64_t ld_pre, void* dPre,
                int64_t ld_dpre, int act, void* out, int out_dtype, void* workspace, int64_t workspace_bytes,
                hipStream_t s) {
    constexpr int V = elem<T>::kVec;
    const int want_sum = out != nullptr ? 1 : 0;
    bool vec = aligned16(dY) && (ld_dy % V) == 0 && (N % V) == 0;
    if (MODE == 1) vec = vec && aligned16(pre) && (ld_pre % V) == 0 && aligned16(dPre) && (ld_dpre % V) == 0;
    int64_t slabs, rows_per_slab;
    if (vec) {
        const int64_t coltiles = (N + 64 * V - 1) / (64 * V);
        colsum_plan(M, N, V, true, slabs, rows_per_slab);
        if (want_sum && workspace_bytes < slabs * N * (int64_t)sizeof(float))
            return fail(CW_ERR_INVALID, "column sum: workspace too small (%lld bytes)", (long long)workspace_bytes);
        const size_t lds = tree_reduce_lds_bytes(V, kColWaves);
        const dim3 grid((unsigned)coltiles, (unsigned)slabs), block(kColWaves * 64);
        auto launch = [&](auto act_c) {
            constexpr int ACT = decltype(act_c)::value;
            hipLaunchKernelGGL((colsum_vec_kernel<T, MODE, ACT>), grid, block, lds, s, M, N, (const T*)dY, ld_dy,
                               (const T*)pre, ld_pre, (T*)dPre, ld_dpre, (float*)workspace, rows_per_slab, want_sum);
        };
        if (MODE == 0 || act == CW_ACT_NONE) launch(std::integral_constant<int, CW_ACT_NONE>{});
        else if (act == CW_ACT_GELU_TANH) launch(std::integral_constant<int, CW_ACT_GELU_TANH>{});
        else if (act == CW_ACT_GELU_ERF) launch(std::integral_constant<int, CW_ACT_GELU_ERF>{});
        else launch(std::integral_constant<int, CW_ACT_RELU>{});
    } else {
        colsum_plan(M, N, V, false, slabs, rows_per_slab);
        if (want_sum && workspace_bytes < slabs * N * (int64_t)sizeof(float))
            return fail(CW_ERR_INVALID, "column sum: workspace too small (%lld bytes)", (long long)workspace_bytes);
        hipLaunchKernelGGL((colsum_generic_kernel<T, MODE>), dim3((unsigned)((N + 255) / 256), (unsigned)slabs),
                           dim3(256), 0, s, M, N, (const T*)dY, ld_dy, (const T*)pre, ld_pre, (T*)dPre, ld_dpre, act,
                           (float*)workspace, rows_per_slab, want_sum);
    }
    int rc = check_launch("colsum kernel");
    if (rc != CW_OK || !want_sum) return rc;
    return finalize_col_partials((const float*)workspace, slabs, N, 1, N, out, nullptr, out_dtype, s);
}

}  // namespace

int finalize_col_partials(const float* ws, int64_t nparts, int64_t part_stride, int nsets, int64_t C, void* out0,
                          void* out1, int out_dtype, hipStream_t s) {
    hipLaunchKernelGGL(finalize_cols_kernel, dim3((unsigned)((C + 63) / 64), (unsigned)nsets), dim3(kFinGroups * 64), 0, s, ws,
                       nparts, part_stride, C, out0, out1, out_dtype);
    return check_launch("finalize_cols_kernel");
}

// ---- library-owned scratch for the entry point that allocates nothing ------------------------------
// One zero-initialised array per GPU, part of the code object: it exists from the moment the library is
// loaded on a device until the process ends. `scratch` names it in device code only; host code uses the
// device address hipGetSymbolAddress reports, looked up once per device with that device current.
constexpr int64_t kStaticScratchBytes = 4ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;
}  // namespace

// Device address of this GPU's copy of `scratch` (nullptr + error text, *rc set, on failure). The first call on a
// device looks the address up; a stream that is being captured is not the place for that (the lookup may load the
// code object), so such a first call is refused and records nothing.
static void* static_scratch_ptr(hipStream_t s, int* rc) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        *rc = fail(CW_ERR_DEVICE, "cw_colsum_static: no current HIP device (or device index above %d)", kMaxDevices - 1);
        return nullptr;
    }
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p != nullptr) return p;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing != hipStreamCaptureStatusNone) {
        *rc = fail(CW_ERR_UNSUPPORTED,
                   "cw_colsum_static: the first call on a device looks up the scratch array's address and must be made "
                   "outside a stream capture; call it once before capturing");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p != nullptr) return p;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
        (void)hipGetLastError();
        *rc = fail(CW_ERR_DEVICE, "cw_colsum_static: hipGetSymbolAddress(scratch) failed on device %d: %s", dev,
                   hipGetErrorString(e));
        return nullptr;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);
    return p;
}

// Bytes of partial sums cw_colsum's kernels write for an [M,N] operand.
template <typename T>
static int64_t colsum_partial_bytes(int64_t M, int64_t N, const void* dY, int64_t ld) {
    constexpr int V = elem<T>::kVec;
    int64_t slabs, rows_per_slab;
    colsum_plan(M, N, V, aligned16(dY) && (ld % V) == 0 && (N % V) == 0, slabs, rows_per_slab);
    return slabs * N * (int64_t)sizeof(float);
}

int64_t colsum_workspace_bytes(int64_t M, int64_t N) {
    int64_t parts = (M + kGenericSlabRows - 1) / kGenericSlabRows;
    if (parts < 512) parts = 512;
    return parts * N * (int64_t)sizeof(float);
}

}  // namespace cw

using namespace cw;

extern "C" int64_t cw_colsum_workspace_bytes(int64_t M, int64_t N) {
    if (M < 0 || N < 0) return 0;
    const int64_t a = colsum_workspace_bytes(M, N);
    const int64_t b = ln_bwd_workspace_bytes(M, N);
    return a > b ? a : b;
}

extern "C" int cw_colsum(int64_t M, int64_t N, const void* dY, int64_t ld, void* out, int out_dtype, void* workspace,
                         int64_t workspace_bytes, int io_dtype, void* stream) {
    if (M < 0 || N <= 0) return fail(CW_ERR_INVALID, "cw_colsum: bad shape M=%lld N=%lld", (long long)M, (long long)N);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_colsum: bad io_dtype %d", io_dtype);
    if (out == nullptr) return fail(CW_ERR_INVALID, "cw_colsum: out is NULL");
    if (!col_out_dtype_ok(out_dtype)) return fail(CW_ERR_INVALID, "cw_colsum: bad out_dtype %d", out_dtype);
    if (const int drc = require_gfx950("cw_colsum"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (M == 0) return finalize_col_partials(nullptr, 0, N, 1, N, out, nullptr, out_dtype, s);  // zero fill
    if (dY == nullptr || workspace == nullptr || ld < N)
        return fail(CW_ERR_INVALID, "cw_colsum: null pointer or ld < N");
    if (io_dtype == CW_F16)
        return colsum_impl<f16_t, 0>(M, N, dY, ld, nullptr, 0, nullptr, 0, 0, out, out_dtype, workspace, workspace_bytes, s);
    return io_dtype == CW_BF16
               ? colsum_impl<bf16_t, 0>(M, N, dY, ld, nullptr, 0, nullptr, 0, 0, out, out_dtype, workspace, workspace_bytes, s)
               : colsum_impl<float, 0>(M, N, dY, ld, nullptr, 0, nullptr, 0, 0, out, out_dtype, workspace, workspace_bytes, s);
}

extern "C" int64_t cw_colsum_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int cw_colsum_static(int64_t M, int64_t N, const void* dY, int64_t ld, void* out, int out_dtype,
                                int io_dtype, void* stream) {
    if (M < 0 || N <= 0)
        return fail(CW_ERR_INVALID, "cw_colsum_static: bad shape M=%lld N=%lld", (long long)M, (long long)N);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_colsum_static: bad io_dtype %d", io_dtype);
    if (out == nullptr) return fail(CW_ERR_INVALID, "cw_colsum_static: out is NULL");
    if (!col_out_dtype_ok(out_dtype)) return fail(CW_ERR_INVALID, "cw_colsum_static: bad out_dtype %d", out_dtype);
    if (const int drc = require_gfx950("cw_colsum_static"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (M == 0) return finalize_col_partials(nullptr, 0, N, 1, N, out, nullptr, out_dtype, s);  // zero fill
    if (dY == nullptr || ld < N) return fail(CW_ERR_INVALID, "cw_colsum_static: null pointer or ld < N");
    const int64_t need = with_elem_type(io_dtype, [&](auto* tag) -> int {
        using T = std::remove_pointer_t<decltype(tag)>;
        const int64_t b = colsum_partial_bytes<T>(M, N, dY, ld);
        return b > kStaticScratchBytes ? -1 : 0;
    });
    if (need != 0)
        return fail(CW_ERR_UNSUPPORTED,
                    "cw_colsum_static: [%lld, %lld] needs more than the %lld bytes of the library's static scratch "
                    "(16-byte aligned operands: N <= 1048576; others: ceil(M/64) * N <= 1048576); use cw_colsum",
                    (long long)M, (long long)N, (long long)kStaticScratchBytes);
    int prc = CW_ERR_DEVICE;
    void* ws = static_scratch_ptr(s, &prc);  // the device address, never the array's name
    if (ws == nullptr) return prc;
    return cw_colsum(M, N, dY, ld, out, out_dtype, ws, kStaticScratchBytes, io_dtype, stream);
}

extern "C" int cw_act_bwd_colsum(int activation, int64_t M, int64_t N, const void* dY, int64_t ld_dy,
                                 const void* preact, int64_t ld_pre, void* dPre, int64_t ld_dpre, void* dbias,
                                 int dbias_dtype, void* workspace, int64_t workspace_bytes, int io_dtype,
                                 void* stream) {
    if (M < 0 || N <= 0)
        return fail(CW_ERR_INVALID, "cw_act_bwd_colsum: bad shape M=%lld N=%lld", (long long)M, (long long)N);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_act_bwd_colsum: bad io_dtype %d", io_dtype);
    if (activation != CW_ACT_NONE && activation != CW_ACT_GELU_TANH && activation != CW_ACT_GELU_ERF &&
        activation != CW_ACT_RELU)
        return fail(CW_ERR_INVALID, "cw_act_bwd_colsum: bad activation %d", activation);
    if (dbias != nullptr && !col_out_dtype_ok(dbias_dtype))
        return fail(CW_ERR_INVALID, "cw_act_bwd_colsum: bad dbias_dtype %d", dbias_dtype);
    if (const int drc = require_gfx950("cw_act_bwd_colsum"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (M == 0) {
        if (dbias == nullptr) return CW_OK;
        return finalize_col_partials(nullptr, 0, N, 1, N, dbias, nullptr, dbias_dtype, s);  // zero fill
    }
    if (dY == nullptr || preact == nullptr || dPre == nullptr || ld_dy < N || ld_pre < N || ld_dpre < N)
        return fail(CW_ERR_INVALID, "cw_act_bwd_colsum: null pointer or leading dimension < N");
    if (dbias != nullptr && workspace == nullptr)
        return fail(CW_ERR_INVALID, "cw_act_bwd_colsum: workspace is NULL");
    if (io_dtype == CW_F16)
        return colsum_impl<f16_t, 1>(M, N, dY, ld_dy, preact, ld_pre, dPre, ld_dpre, activation, dbias, dbias_dtype,
                                     workspace, workspace_bytes, s);
    return io_dtype == CW_BF16 ? colsum_impl<bf16_t, 1>(M, N, dY, ld_dy, preact, ld_pre, dPre, ld_dpre, activation, dbias,
                                                        dbias_dtype, workspace, workspace_bytes, s)
                               : colsum_impl<float, 1>(M, N, dY, ld_dy, preact, ld_pre, dPre, ld_dpre, activation, dbias,
                                                       dbias_dtype, workspace, workspace_bytes, s);
}
