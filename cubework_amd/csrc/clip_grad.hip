// Gradient-norm clipping over many tensors at once, for gfx950.
//   cw_multi_norm_partials : (sum over "standard" tensors of |g|^p, sum over tensor-parallel tensors of
//                            factor * |g|^p), or the maximum |g| for the infinity norm, of up to
//                            thousands of gradient tensors in a handful of launches
//                            (cubework/utils/clip_grad.py:33-50 of the reference runs torch.norm per
//                            tensor and stacks the results);
//   cw_multi_scale         : g *= coef for all of them, coef read from device memory so that no
//                            host synchronisation is needed (clip_grad.py:64-68).
// Tensors are handled in batches of kMaxTensors whose pointers travel by value in the kernel
// arguments; a block owns one chunk of one tensor. Block partials go to a workspace and are
// added in index order by a second kernel: no atomics, bit-reproducible.
#include "cw_common.h"

namespace cw {

namespace {

constexpr int kMaxTensors = 48;
constexpr int kChunk = 64 * 1024;  // elements per block
constexpr int kClipThreads = 256;

struct TensorBatch {
    const void* ptr[kMaxTensors];
    int64_t numel[kMaxTensors];
    float factor[kMaxTensors];   // weight of the tensor's sum (num_partitions), 1 for standard tensors
    int first_block[kMaxTensors + 1];
    unsigned char group[kMaxTensors];  // 0 standard, 1 tensor-parallel
    int n;
};

__device__ __forceinline__ int find_tensor(const TensorBatch& b, int block) {
    int t = 0;
#pragma unroll 1
    while (t + 1 < b.n && b.first_block[t + 1] <= block) ++t;
    return t;
}

// Maximum of absolute values through their bit patterns: for non-negative floats the unsigned order is the
// float order, +inf sorts above every number and every NaN above +inf, so a NaN gradient makes the maximum
// NaN, as torch's abs().max() does (fmaxf would drop it).
__device__ __forceinline__ float abs_max(float a, float b) {
    const uint32_t ua = __float_as_uint(a) & 0x7fffffffu, ub = __float_as_uint(b) & 0x7fffffffu;
    return __uint_as_float(ua > ub ? ua : ub);
}
__device__ __forceinline__ float wave_abs_max(float v) {
    v = abs_max(v, dpp_move<kDppXor1>(v));
    v = abs_max(v, dpp_move<kDppXor2>(v));
    v = abs_max(v, dpp_move<kDppHalfMirror>(v));
    v = abs_max(v, dpp_move<kDppMirror>(v));
    const int iv = __float_as_int(v);
    float r = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
    r = abs_max(r, __int_as_float(__builtin_amdgcn_readlane(iv, 16)));
    r = abs_max(r, __int_as_float(__builtin_amdgcn_readlane(iv, 32)));
    return abs_max(r, __int_as_float(__builtin_amdgcn_readlane(iv, 48)));
}

// KIND 0: max |g|;  KIND 2: sum g^2;  KIND 1: sum |g|^p (general p)
template <typename T, int KIND>
__global__ __launch_bounds__(kClipThreads) void multi_norm_kernel(const TensorBatch b, float p, float* __restrict__ ws,
                                                                 int ws_offset) {
    constexpr int V = elem<T>::kVec;
    __shared__ float red[kClipThreads / 64];
    const int t = find_tensor(b, blockIdx.x);
    const int64_t start = (int64_t)(blockIdx.x - b.first_block[t]) * kChunk;
    int64_t len = b.numel[t] - start;
    len = len < kChunk ? len : kChunk;
    const T* g = reinterpret_cast<const T*>(b.ptr[t]) + start;
    float acc = 0.0f;
    auto add = [&](float x) {
        const float a = fabsf(x);
        if (KIND == 0) acc = abs_max(acc, x);
        else if (KIND == 2) acc = __builtin_fmaf(x, x, acc);
        else acc += __powf(a, p);
    };
    if ((reinterpret_cast<uintptr_t>(g) & 15u) == 0) {
        const int64_t nvec = len / V;
#pragma unroll 4
        for (int64_t i = threadIdx.x; i < nvec; i += kClipThreads) {
            float v[V];
            unpack_raw(load_raw_stream(g + i * V), v, (const T*)nullptr);
#pragma unroll
            for (int e = 0; e < V; ++e) add(v[e]);
        }
        for (int64_t i = nvec * V + threadIdx.x; i < len; i += kClipThreads) add(load_elem(g + i));
    } else {
        for (int64_t i = threadIdx.x; i < len; i += kClipThreads) add(load_elem(g + i));
    }
    acc = (KIND == 0) ? wave_abs_max(acc) : wave_sum(acc);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = red[0];
#pragma unroll
        for (int w = 1; w < kClipThreads / 64; ++w) r = (KIND == 0) ? abs_max(r, red[w]) : r + red[w];
        // the partial and, beside it, the group it belongs to
        ws[2 * (ws_offset + blockIdx.x)] = (KIND == 0) ? r : r * b.factor[t];
        ws[2 * (ws_offset + blockIdx.x) + 1] = (float)b.group[t];
    }
}

// out[0] = combination of the standard tensors' partials, out[1] = of the tensor-parallel ones.
template <int KIND>
__global__ __launch_bounds__(256) void norm_finalize_kernel(const float* __restrict__ ws, int n_partials,
                                                            float* __restrict__ out) {
    __shared__ float red[2][256];
    float a0 = 0.0f, a1 = 0.0f;
    for (int i = threadIdx.x; i < n_partials; i += 256) {
        const float v = ws[2 * i];
        const bool tp = ws[2 * i + 1] != 0.0f;
        if (KIND == 0) {
            a0 = tp ? a0 : abs_max(a0, v);
            a1 = tp ? abs_max(a1, v) : a1;
        } else {
            a0 += tp ? 0.0f : v;
            a1 += tp ? v : 0.0f;
        }
    }
    red[0][threadIdx.x] = a0;
    red[1][threadIdx.x] = a1;
    __syncthreads();
    if (threadIdx.x < 2) {
        float r = red[threadIdx.x][0];
        for (int i = 1; i < 256; ++i) r = (KIND == 0) ? abs_max(r, red[threadIdx.x][i]) : r + red[threadIdx.x][i];
        out[threadIdx.x] = r;
    }
}

template <typename T>
__global__ __launch_bounds__(kClipThreads) void multi_scale_kernel(const TensorBatch b, const float* __restrict__ coef) {
    constexpr int V = elem<T>::kVec;
    const int t = find_tensor(b, blockIdx.x);
    const int64_t start = (int64_t)(blockIdx.x - b.first_block[t]) * kChunk;
    int64_t len = b.numel[t] - start;
    len = len < kChunk ? len : kChunk;
    T* g = reinterpret_cast<T*>(const_cast<void*>(b.ptr[t])) + start;
    const float c = coef[0];
    if ((reinterpret_cast<uintptr_t>(g) & 15u) == 0) {
        const int64_t nvec = len / V;
#pragma unroll 4
        for (int64_t i = threadIdx.x; i < nvec; i += kClipThreads) {
            float v[V];
            unpack_raw(load_raw_stream(g + i * V), v, (const T*)nullptr);
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] *= c;
            store_raw_stream(g + i * V, pack_raw(v, (const T*)nullptr));
        }
        for (int64_t i = nvec * V + threadIdx.x; i < len; i += kClipThreads) store_elem(g + i, load_elem(g + i) * c);
    } else {
        for (int64_t i = threadIdx.x; i < len; i += kClipThreads) store_elem(g + i, load_elem(g + i) * c);
    }
}

// One thread: combines the (standard, tensor-parallel) results of n_sets calls of the norm stage into
// the total norm and the clamped scaling coefficient.
__global__ void clip_coef_kernel(const float* __restrict__ sets, int n_sets, float tp_scale, float norm_type,
                                 float max_norm, float* __restrict__ out2) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    float norm;
    if (__builtin_isinf(norm_type)) {
        norm = 0.0f;
        for (int i = 0; i < 2 * n_sets; ++i) norm = abs_max(norm, sets[i]);  // NaN-propagating, as torch.max is
    } else {
        float std_sum = 0.0f, tp_sum = 0.0f;
        for (int i = 0; i < n_sets; ++i) {
            std_sum += sets[2 * i];
            tp_sum += sets[2 * i + 1];
        }
        const float total = std_sum + tp_sum * tp_scale;
        norm = norm_type == 2.0f ? sqrtf(total) : (norm_type == 1.0f ? total : powf(total, 1.0f / norm_type));
    }
    const float coef = max_norm / (norm + 1e-6f);
    out2[0] = norm;
    out2[1] = coef > 1.0f ? 1.0f : coef;  // NaN stays NaN, as torch.clamp(max=1) leaves it
}

int64_t blocks_of(int64_t numel) { return (numel + kChunk - 1) / kChunk; }

// Fills `b` with tensors [first, ...) until it is full; returns the index of the next tensor.
int fill_batch(TensorBatch& b, int first, int n_tensors, const void* const* ptrs, const int64_t* numels,
               const float* factors, const unsigned char* groups) {
    b.n = 0;
    int blocks = 0;
    int i = first;
    for (; i < n_tensors && b.n < kMaxTensors; ++i) {
        if (numels[i] == 0) continue;
        b.ptr[b.n] = ptrs[i];
        b.numel[b.n] = numels[i];
        b.factor[b.n] = factors != nullptr ? factors[i] : 1.0f;
        b.group[b.n] = groups != nullptr ? groups[i] : 0;
        b.first_block[b.n] = blocks;
        blocks += (int)blocks_of(numels[i]);
        ++b.n;
    }
    b.first_block[b.n] = blocks;
    return i;
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int64_t cw_multi_norm_workspace_bytes(int n_tensors, const int64_t* numels) {
    if (n_tensors <= 0 || numels == nullptr) return 16;
    int64_t blocks = 0;
    for (int i = 0; i < n_tensors; ++i) blocks += numels[i] > 0 ? blocks_of(numels[i]) : 0;
    return (blocks > 0 ? blocks : 1) * 2 * (int64_t)sizeof(float);
}

extern "C" int cw_multi_norm_partials(int n_tensors, const void* const* grads, const int64_t* numels,
                                      const float* factors, const unsigned char* groups, float norm_type,
                                      float* out2, void* workspace, int64_t workspace_bytes, int io_dtype,
                                      void* stream) {
    if (n_tensors < 0) return fail(CW_ERR_INVALID, "cw_multi_norm_partials: negative tensor count");
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_multi_norm_partials: bad io_dtype %d", io_dtype);
    if (out2 == nullptr || workspace == nullptr) return fail(CW_ERR_INVALID, "cw_multi_norm_partials: null output or workspace");
    if (!(norm_type > 0.0f)) return fail(CW_ERR_INVALID, "cw_multi_norm_partials: norm_type must be positive (inf for the maximum norm)");
    if (n_tensors > 0 && (grads == nullptr || numels == nullptr)) return fail(CW_ERR_INVALID, "cw_multi_norm_partials: null tables");
    for (int i = 0; i < n_tensors; ++i)
        if (numels[i] < 0 || (numels[i] > 0 && grads[i] == nullptr) || blocks_of(numels[i]) > (1 << 24))
            return fail(CW_ERR_INVALID, "cw_multi_norm_partials: tensor %d is NULL or has a bad size", i);
    if (workspace_bytes < cw_multi_norm_workspace_bytes(n_tensors, numels))
        return fail(CW_ERR_INVALID, "cw_multi_norm_partials: workspace too small (%lld bytes)", (long long)workspace_bytes);
    if (const int drc = require_gfx950("cw_multi_norm_partials"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    const int kind = __builtin_isinf(norm_type) ? 0 : (norm_type == 2.0f ? 2 : 1);
    float* ws = (float*)workspace;
    int done = 0, offset = 0;
    while (done < n_tensors) {
        TensorBatch b;
        done = fill_batch(b, done, n_tensors, grads, numels, factors, groups);
        const int blocks = b.first_block[b.n];
        if (blocks == 0) continue;
#define CW_LAUNCH_NORM(T, KIND) hipLaunchKernelGGL((multi_norm_kernel<T, KIND>), dim3(blocks), dim3(kClipThreads), 0, s, b, norm_type, ws, offset)
        if (io_dtype == CW_BF16) {
            if (kind == 0) CW_LAUNCH_NORM(bf16_t, 0); else if (kind == 2) CW_LAUNCH_NORM(bf16_t, 2); else CW_LAUNCH_NORM(bf16_t, 1);
        } else if (io_dtype == CW_F16) {
            if (kind == 0) CW_LAUNCH_NORM(f16_t, 0); else if (kind == 2) CW_LAUNCH_NORM(f16_t, 2); else CW_LAUNCH_NORM(f16_t, 1);
        } else {
            if (kind == 0) CW_LAUNCH_NORM(float, 0); else if (kind == 2) CW_LAUNCH_NORM(float, 2); else CW_LAUNCH_NORM(float, 1);
        }
#undef CW_LAUNCH_NORM
        const int rc = check_launch("multi_norm_kernel");
        if (rc != CW_OK) return rc;
        offset += blocks;
    }
    if (kind == 0) hipLaunchKernelGGL(norm_finalize_kernel<0>, dim3(1), dim3(256), 0, s, ws, offset, out2);
    else hipLaunchKernelGGL(norm_finalize_kernel<2>, dim3(1), dim3(256), 0, s, ws, offset, out2);
    return check_launch("norm_finalize_kernel");
}

extern "C" int cw_clip_coef(int n_sets, const float* sets, float tp_scale, float norm_type, float max_norm,
                            float* out2, void* stream) {
    if (n_sets < 1 || n_sets > 64) return fail(CW_ERR_INVALID, "cw_clip_coef: n_sets %d outside [1, 64]", n_sets);
    if (sets == nullptr || out2 == nullptr) return fail(CW_ERR_INVALID, "cw_clip_coef: null argument");
    if (!(norm_type > 0.0f)) return fail(CW_ERR_INVALID, "cw_clip_coef: norm_type must be positive (inf for the maximum norm)");
    if (const int drc = require_gfx950("cw_clip_coef"); drc != CW_OK) return drc;
    hipLaunchKernelGGL(clip_coef_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, sets, n_sets, tp_scale, norm_type,
                       max_norm, out2);
    return check_launch("clip_coef_kernel");
}

extern "C" int cw_multi_scale(int n_tensors, void* const* grads, const int64_t* numels, const float* coef,
                              int io_dtype, void* stream) {
    if (n_tensors < 0) return fail(CW_ERR_INVALID, "cw_multi_scale: negative tensor count");
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_multi_scale: bad io_dtype %d", io_dtype);
    if (coef == nullptr) return fail(CW_ERR_INVALID, "cw_multi_scale: coef is NULL");
    if (n_tensors > 0 && (grads == nullptr || numels == nullptr)) return fail(CW_ERR_INVALID, "cw_multi_scale: null tables");
    for (int i = 0; i < n_tensors; ++i)
        if (numels[i] < 0 || (numels[i] > 0 && grads[i] == nullptr) || blocks_of(numels[i]) > (1 << 24))
            return fail(CW_ERR_INVALID, "cw_multi_scale: tensor %d is NULL or has a bad size", i);
    if (const int drc = require_gfx950("cw_multi_scale"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    int done = 0;
    while (done < n_tensors) {
        TensorBatch b;
        done = fill_batch(b, done, n_tensors, (const void* const*)grads, numels, nullptr, nullptr);
        const int blocks = b.first_block[b.n];
        if (blocks == 0) continue;
        if (io_dtype == CW_BF16) hipLaunchKernelGGL(multi_scale_kernel<bf16_t>, dim3(blocks), dim3(kClipThreads), 0, s, b, coef);
        else if (io_dtype == CW_F16) hipLaunchKernelGGL(multi_scale_kernel<f16_t>, dim3(blocks), dim3(kClipThreads), 0, s, b, coef);
        else hipLaunchKernelGGL(multi_scale_kernel<float>, dim3(blocks), dim3(kClipThreads), 0, s, b, coef);
        const int rc = check_launch("multi_scale_kernel");
        if (rc != CW_OK) return rc;
    }
    return CW_OK;
}
