// Gradient-norm clipping over many tensors at once, for gfx950.
//   cw_multi_norm_partials : (sum over "standard" tensors of |g|^p, sum over tensor-parallel tensors of
//                            factor * |g|^p), or the maximum |g| for the infinity norm, of up to
//                            thousands of gradient tensors in a handful of launches
//                            (cubework/utils/clip_grad.py:33-50 of the reference runs torch.norm per
//                            tensor and stacks the results);
//   cw_multi_scale         : g *= coef for all of them, coef read from device memory so that no
//                            host synchronisation is needed (clip_grad.py:64-68);
//   cw_clip_scale          : the same launch, which first works the coefficient out of the norm stage's
//                            results itself (every workgroup adds the few thousand block partials in the
//                            same fixed order while its first loads are in flight), so that a clipping
//                            call without a tensor-parallel exchange is two launches per dtype.
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

// (standard, tensor-parallel) combination of n (value, group) pairs and of n_sets finished (standard,
// tensor-parallel) pairs: sums, or maxima of absolute values when is_max. Fixed order (thread-strided, lanes
// through wave_sum, the four wavefronts in index order), so every workgroup that runs it gets the same bits.
// Must be reached by all 256 threads; red holds 8 floats.
__device__ __forceinline__ void reduce_pairs(const float* __restrict__ pairs, int n, const float* __restrict__ sets,
                                             int n_sets, bool is_max, float* red, float& std_out, float& tp_out) {
    float a0 = 0.0f, a1 = 0.0f;
    for (int i = threadIdx.x; i < n; i += kClipThreads) {
        const float v = pairs[2 * i];
        const bool tp = pairs[2 * i + 1] != 0.0f;
        if (is_max) {
            a0 = tp ? a0 : abs_max(a0, v);
            a1 = tp ? abs_max(a1, v) : a1;
        } else {
            a0 += tp ? 0.0f : v;
            a1 += tp ? v : 0.0f;
        }
    }
    for (int i = threadIdx.x; i < n_sets; i += kClipThreads) {
        a0 = is_max ? abs_max(a0, sets[2 * i]) : a0 + sets[2 * i];
        a1 = is_max ? abs_max(a1, sets[2 * i + 1]) : a1 + sets[2 * i + 1];
    }
    a0 = is_max ? wave_abs_max(a0) : wave_sum(a0);
    a1 = is_max ? wave_abs_max(a1) : wave_sum(a1);
    if ((threadIdx.x & 63) == 0) {
        red[2 * (threadIdx.x >> 6)] = a0;
        red[2 * (threadIdx.x >> 6) + 1] = a1;
    }
    __syncthreads();
    float r0 = red[0], r1 = red[1];
#pragma unroll
    for (int w = 1; w < kClipThreads / 64; ++w) {
        r0 = is_max ? abs_max(r0, red[2 * w]) : r0 + red[2 * w];
        r1 = is_max ? abs_max(r1, red[2 * w + 1]) : r1 + red[2 * w + 1];
    }
    std_out = r0;
    tp_out = r1;
}

// out[0] = combination of the standard tensors' partials, out[1] = of the tensor-parallel ones.
template <int KIND>
__global__ __launch_bounds__(kClipThreads) void norm_finalize_kernel(const float* __restrict__ ws, int n_partials,
                                                                    float* __restrict__ out) {
    __shared__ float red[2 * kClipThreads / 64];
    float r0, r1;
    reduce_pairs(ws, n_partials, nullptr, 0, KIND == 0, red, r0, r1);
    if (threadIdx.x == 0) {
        out[0] = r0;
        out[1] = r1;
    }
}

// Total norm and clamped coefficient from the (standard, tensor-parallel) combination.
__device__ __forceinline__ void norm_and_coef(float std_part, float tp_part, float tp_scale, float norm_type,
                                              float max_norm, float& norm, float& coef) {
    if (__builtin_isinf(norm_type)) {
        norm = abs_max(std_part, tp_part);  // NaN-propagating, as torch.max is
    } else {
        const float total = std_part + tp_part * tp_scale;
        norm = norm_type == 2.0f ? sqrtf(total) : (norm_type == 1.0f ? total : powf(total, 1.0f / norm_type));
    }
    const float c = max_norm / (norm + 1e-6f);
    coef = c > 1.0f ? 1.0f : c;  // NaN stays NaN, as torch.clamp(max=1) leaves it
}

// What cw_clip_scale hands its launch: the norm stage's results, finished (sets) or as block partials.
struct ClipArgs {
    const float* sets;
    const float* partials;
    float* out2;
    int n_sets, n_partials;
    float tp_scale, norm_type, max_norm;
};

// The coefficient stage of cw_clip_scale alone, for a call without elements to scale.
__global__ __launch_bounds__(kClipThreads) void clip_only_kernel(const ClipArgs clip) {
    __shared__ float red[2 * kClipThreads / 64];
    float std_part, tp_part, norm, c;
    reduce_pairs(clip.partials, clip.n_partials, clip.sets, clip.n_sets, __builtin_isinf(clip.norm_type), red, std_part, tp_part);
    norm_and_coef(std_part, tp_part, clip.tp_scale, clip.norm_type, clip.max_norm, norm, c);
    if (threadIdx.x == 0) {
        clip.out2[0] = norm;
        clip.out2[1] = c;
    }
}

// FUSED: the coefficient comes from `clip` (every workgroup works it out, workgroup 0 also stores the norm and
// the coefficient to clip.out2) instead of from coef[0]. A thread's first kScaleBatch vectors are requested
// before the coefficient is looked at, so its computation runs under their latency. A workgroup owns 32 KB of
// one tensor, one batch per thread (measured on 100 MB of bf16 gradients: 35.0 us against 40.9 us with 128 KB
// per workgroup in four batches).
constexpr int kScaleBatch = 8;
constexpr int kFusedPairsMax = 2048;  // pairs that every workgroup of the fused scaling launch may read
constexpr int kScaleChunkBytes = kScaleBatch * kClipThreads * 16;  // one batch per thread: 32 KB per workgroup

template <typename T, bool FUSED>
__global__ __launch_bounds__(kClipThreads) void multi_scale_kernel(const TensorBatch b, const float* __restrict__ coef,
                                                                  const ClipArgs clip) {
    constexpr int V = elem<T>::kVec;
    constexpr int U = kScaleBatch;
    constexpr int kScaleChunk = kScaleChunkBytes / (int)sizeof(T);
    __shared__ float red[2 * kClipThreads / 64];
    const int t = find_tensor(b, blockIdx.x);
    const int64_t start = (int64_t)(blockIdx.x - b.first_block[t]) * kScaleChunk;
    int64_t len = b.numel[t] - start;
    len = len < kScaleChunk ? len : kScaleChunk;
    T* g = reinterpret_cast<T*>(const_cast<void*>(b.ptr[t])) + start;
    const bool aligned = (reinterpret_cast<uintptr_t>(g) & 15u) == 0;
    const int64_t nvec = aligned ? len / V : 0;
    raw16_t r[U];
    const bool head = (int64_t)threadIdx.x + (U - 1) * kClipThreads < nvec;
    if (head) {
#pragma unroll
        for (int u = 0; u < U; ++u) r[u] = load_raw_stream(g + ((int64_t)threadIdx.x + u * kClipThreads) * V);
    }
    float c;
    if constexpr (FUSED) {
        float std_part, tp_part, norm;
        reduce_pairs(clip.partials, clip.n_partials, clip.sets, clip.n_sets, __builtin_isinf(clip.norm_type), red, std_part,
                     tp_part);
        norm_and_coef(std_part, tp_part, clip.tp_scale, clip.norm_type, clip.max_norm, norm, c);
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            clip.out2[0] = norm;
            clip.out2[1] = c;
        }
    } else {
        c = coef[0];
    }
    auto scaled = [&](raw16_t u) {
        float v[V];
        unpack_raw(u, v, (const T*)nullptr);
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] *= c;
        return pack_raw(v, (const T*)nullptr);
    };
    int64_t i = threadIdx.x;
    if (head) {
#pragma unroll
        for (int u = 0; u < U; ++u) store_raw_stream(g + (i + u * kClipThreads) * V, scaled(r[u]));
        i += U * kClipThreads;
    }
    for (; i + (U - 1) * kClipThreads < nvec; i += U * kClipThreads) {
#pragma unroll
        for (int u = 0; u < U; ++u) r[u] = load_raw_stream(g + (i + u * kClipThreads) * V);
#pragma unroll
        for (int u = 0; u < U; ++u) store_raw_stream(g + (i + u * kClipThreads) * V, scaled(r[u]));
    }
    for (; i < nvec; i += kClipThreads) store_raw_stream(g + i * V, scaled(load_raw_stream(g + i * V)));
    for (int64_t j = nvec * V + threadIdx.x; j < len; j += kClipThreads) store_elem(g + j, load_elem(g + j) * c);
}

// One thread: combines the (standard, tensor-parallel) results of n_sets calls of the norm stage into
// the total norm and the clamped scaling coefficient.
__global__ void clip_coef_kernel(const float* __restrict__ sets, int n_sets, float tp_scale, float norm_type,
                                 float max_norm, float* __restrict__ out2) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const bool is_max = __builtin_isinf(norm_type);
    float std_sum = 0.0f, tp_sum = 0.0f;
    for (int i = 0; i < n_sets; ++i) {
        std_sum = is_max ? abs_max(std_sum, sets[2 * i]) : std_sum + sets[2 * i];
        tp_sum = is_max ? abs_max(tp_sum, sets[2 * i + 1]) : tp_sum + sets[2 * i + 1];
    }
    float norm, coef;
    norm_and_coef(std_sum, tp_sum, tp_scale, norm_type, max_norm, norm, coef);
    out2[0] = norm;
    out2[1] = coef;
}

int64_t blocks_of(int64_t numel) { return (numel + kChunk - 1) / kChunk; }

// Fills `b` with tensors [first, ...) until it is full; returns the index of the next tensor.
int fill_batch(TensorBatch& b, int first, int n_tensors, const void* const* ptrs, const int64_t* numels,
               const float* factors, const unsigned char* groups, int chunk = kChunk) {
    b.n = 0;
    int64_t blocks = 0;
    int i = first;
    for (; i < n_tensors && b.n < kMaxTensors; ++i) {
        if (numels[i] == 0) continue;
        const int64_t nb = (numels[i] + chunk - 1) / chunk;  // at most 2^27 (2^24 chunks of kChunk elements)
        if (b.n > 0 && blocks + nb > (1 << 30)) break;       // the grid of one launch
        b.ptr[b.n] = ptrs[i];
        b.numel[b.n] = numels[i];
        b.factor[b.n] = factors != nullptr ? factors[i] : 1.0f;
        b.group[b.n] = groups != nullptr ? groups[i] : 0;
        b.first_block[b.n] = (int)blocks;
        blocks += nb;
        ++b.n;
    }
    b.first_block[b.n] = (int)blocks;
    return i;
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int64_t cw_multi_norm_partial_count(int n_tensors, const int64_t* numels) {
    if (n_tensors <= 0 || numels == nullptr) return 0;
    int64_t blocks = 0;
    for (int i = 0; i < n_tensors; ++i) blocks += numels[i] > 0 ? blocks_of(numels[i]) : 0;
    return blocks;
}

extern "C" int64_t cw_multi_norm_workspace_bytes(int n_tensors, const int64_t* numels) {
    const int64_t blocks = cw_multi_norm_partial_count(n_tensors, numels);
    return (blocks > 0 ? blocks : 1) * 2 * (int64_t)sizeof(float);
}

extern "C" int cw_multi_norm_partials(int n_tensors, const void* const* grads, const int64_t* numels,
                                      const float* factors, const unsigned char* groups, float norm_type,
                                      float* out2, void* workspace, int64_t workspace_bytes, int io_dtype,
                                      void* stream) {
    if (n_tensors < 0) return fail(CW_ERR_INVALID, "cw_multi_norm_partials: negative tensor count");
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_multi_norm_partials: bad io_dtype %d", io_dtype);
    if (workspace == nullptr) return fail(CW_ERR_INVALID, "cw_multi_norm_partials: null workspace");
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
    if (out2 == nullptr) return CW_OK;  // the block partials stay in the workspace for cw_clip_scale
    if (kind == 0) hipLaunchKernelGGL(norm_finalize_kernel<0>, dim3(1), dim3(kClipThreads), 0, s, ws, offset, out2);
    else hipLaunchKernelGGL(norm_finalize_kernel<2>, dim3(1), dim3(kClipThreads), 0, s, ws, offset, out2);
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

namespace {

int scale_impl(const char* who, int n_tensors, void* const* grads, const int64_t* numels, const float* coef,
               const ClipArgs* clip, int io_dtype, void* stream) {
    if (n_tensors < 0) return fail(CW_ERR_INVALID, "%s: negative tensor count", who);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16) return fail(CW_ERR_INVALID, "%s: bad io_dtype %d", who, io_dtype);
    if (n_tensors > 0 && (grads == nullptr || numels == nullptr)) return fail(CW_ERR_INVALID, "%s: null tables", who);
    for (int i = 0; i < n_tensors; ++i)
        if (numels[i] < 0 || (numels[i] > 0 && grads[i] == nullptr) || blocks_of(numels[i]) > (1 << 24))
            return fail(CW_ERR_INVALID, "%s: tensor %d is NULL or has a bad size", who, i);
    if (const int drc = require_gfx950(who); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    const ClipArgs none = {};
    // Every workgroup of the fused scaling launch reads all pairs: fine for a few thousand (16 KB from L2 beside the
    // 64 KB it moves), quadratic beyond. More pairs than that (the gradients of a billion parameters leave 16384) are
    // combined by one launch of their own first, and the scaling launch reads the coefficient it leaves in out2.
    if (clip != nullptr && clip->n_partials > kFusedPairsMax) {
        hipLaunchKernelGGL(clip_only_kernel, dim3(1), dim3(kClipThreads), 0, s, *clip);
        if (const int rc = check_launch("clip_only_kernel"); rc != CW_OK) return rc;
        coef = clip->out2 + 1;
        clip = nullptr;
    }
    int done = 0, launches = 0;
    while (done < n_tensors) {
        TensorBatch b;
        done = fill_batch(b, done, n_tensors, (const void* const*)grads, numels, nullptr, nullptr,
                          kScaleChunkBytes / (io_dtype == CW_F32 ? 4 : 2));
        const int blocks = b.first_block[b.n];
        if (blocks == 0) continue;
#define CW_LAUNCH_SCALE(T)                                                                                              \
    do {                                                                                                                \
        if (clip != nullptr) hipLaunchKernelGGL((multi_scale_kernel<T, true>), dim3(blocks), dim3(kClipThreads), 0, s, b, coef, *clip); \
        else hipLaunchKernelGGL((multi_scale_kernel<T, false>), dim3(blocks), dim3(kClipThreads), 0, s, b, coef, none);  \
    } while (0)
        if (io_dtype == CW_BF16) CW_LAUNCH_SCALE(bf16_t);
        else if (io_dtype == CW_F16) CW_LAUNCH_SCALE(f16_t);
        else CW_LAUNCH_SCALE(float);
#undef CW_LAUNCH_SCALE
        const int rc = check_launch("multi_scale_kernel");
        if (rc != CW_OK) return rc;
        ++launches;
    }
    if (clip != nullptr && launches == 0) {
        // nothing to scale: the norm and the coefficient are still owed to the caller
        hipLaunchKernelGGL(clip_only_kernel, dim3(1), dim3(kClipThreads), 0, s, *clip);
        return check_launch("clip_only_kernel");
    }
    return CW_OK;
}

}  // namespace

extern "C" int cw_multi_scale(int n_tensors, void* const* grads, const int64_t* numels, const float* coef,
                              int io_dtype, void* stream) {
    if (coef == nullptr) return fail(CW_ERR_INVALID, "cw_multi_scale: coef is NULL");
    return scale_impl("cw_multi_scale", n_tensors, grads, numels, coef, nullptr, io_dtype, stream);
}

extern "C" int cw_clip_scale(int n_tensors, void* const* grads, const int64_t* numels, int io_dtype, int n_sets,
                             const float* sets, int64_t n_partials, const float* partials, float tp_scale,
                             float norm_type, float max_norm, float* out2, void* stream) {
    if (n_sets < 0 || n_sets > 64) return fail(CW_ERR_INVALID, "cw_clip_scale: n_sets %d outside [0, 64]", n_sets);
    if (n_partials < 0 || n_partials > (1 << 24)) return fail(CW_ERR_INVALID, "cw_clip_scale: n_partials %lld outside [0, 2^24]", (long long)n_partials);
    if ((n_sets > 0 && sets == nullptr) || (n_partials > 0 && partials == nullptr) || out2 == nullptr)
        return fail(CW_ERR_INVALID, "cw_clip_scale: null argument");
    if (!(norm_type > 0.0f)) return fail(CW_ERR_INVALID, "cw_clip_scale: norm_type must be positive (inf for the maximum norm)");
    ClipArgs clip;
    clip.sets = sets;
    clip.partials = partials;
    clip.out2 = out2;
    clip.n_sets = n_sets;
    clip.n_partials = (int)n_partials;
    clip.tp_scale = tp_scale;
    clip.norm_type = norm_type;
    clip.max_norm = max_norm;
    return scale_impl("cw_clip_scale", n_tensors, grads, numels, nullptr, &clip, io_dtype, stream);
}
