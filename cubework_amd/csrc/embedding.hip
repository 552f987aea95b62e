// Vocab-parallel embedding, one rank's vocabulary slice, for gfx950.
// forward : out[t, :] = (start <= id[t] < start + V_loc) ? weight[id[t] - start, :] : 0
//           (cubework/module/parallel_1d/module.py:441-455, parallel_2d/module.py:345-355 of the
//           reference: mask, shifted index, F.embedding, zeroed masked rows) in one pass: a masked
//           row is never read, only written as zeros.
// backward: d_weight[r, :] = sum over tokens with id - start == r of d_out[t, :]
//           (autograd of F.embedding), deterministic: the caller supplies the token order sorted
//           by id; a run of equal ids is summed by the blocks at its first positions (column
//           slices), whose wavefronts stride the run's tokens and are combined in a fixed order.
//           No atomics.
// Both are HBM-streaming kernels: 16-byte accesses, one wavefront per row.
#include <type_traits>

#include "cw_common.h"

namespace cw {

namespace {

constexpr int kEmbWaves = 4;

template <typename T>
__global__ __launch_bounds__(kEmbWaves * 64) void embed_fwd_kernel(int64_t T_rows, int64_t E, const int64_t* __restrict__ ids,
                                                                   int64_t vocab_start, int64_t V_loc,
                                                                   const T* __restrict__ weight, int64_t ldw,
                                                                   T* __restrict__ out, int64_t ldo, int vec_ok) {
    constexpr int V = elem<T>::kVec;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kEmbWaves + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * kEmbWaves;
    for (int64_t t = wave; t < T_rows; t += nwaves) {
        const int64_t local = ids[t] - vocab_start;
        const bool masked = local < 0 || local >= V_loc;  // same for the whole wavefront
        const T* src = weight + (masked ? 0 : local) * ldw;
        T* dst = out + t * ldo;
        if (vec_ok) {
            const int64_t nvec = E / V;
            for (int64_t c = lane; c < nvec; c += 64) {
                raw16_t v = (raw16_t){0u, 0u, 0u, 0u};
                if (!masked) v = load_raw(src + c * V);
                store_raw_stream(dst + c * V, v);
            }
            for (int64_t c = nvec * V + lane; c < E; c += 64) store_elem(dst + c, masked ? 0.0f : load_elem(src + c));
        } else {
            for (int64_t c = lane; c < E; c += 64) store_elem(dst + c, masked ? 0.0f : load_elem(src + c));
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void zero_rows_kernel(int64_t R, int64_t E, T* __restrict__ p, int64_t ld, int vec_ok) {
    constexpr int V = elem<T>::kVec;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    for (int64_t r = wave; r < R; r += nwaves) {
        T* dst = p + r * ld;
        if (vec_ok) {
            const int64_t nvec = E / V;
            for (int64_t c = lane; c < nvec; c += 64) store_raw_stream(dst + c * V, (raw16_t){0u, 0u, 0u, 0u});
            for (int64_t c = nvec * V + lane; c < E; c += 64) store_elem(dst + c, 0.0f);
        } else {
            for (int64_t c = lane; c < E; c += 64) store_elem(dst + c, 0.0f);
        }
    }
}

// One block per position i of the sorted order. A run of fewer than kRunBlocks equal ids is summed by
// its first block, a column slice per wavefront. The first kRunBlocks positions of a longer run share its
// work by column slices of 64 vectors (block k takes slices k, k + kRunBlocks, ...); the other positions
// exit after a few index loads. Inside such a block, wavefront w sums tokens w, w + 8, ... of the run,
// eight row loads in flight, and finds the run's end as it goes (no scan for the length ahead of the
// work); the eight sums are added in wavefront order. Everything is a fixed order: bit-reproducible, no atomics. A run of
// L tokens costs L / 8 row slices per wavefront: token frequencies of real text (one id hundreds of times
// in a batch) stay in the microseconds.
constexpr int kRunBlocks = 4;
constexpr int kRunWaves = 8;

template <typename T>
__global__ __launch_bounds__(kRunWaves * 64) void embed_bwd_kernel(int64_t T_rows, int64_t E,
                                                                   const int64_t* __restrict__ sorted_ids,
                                                                   const int64_t* __restrict__ order, int64_t vocab_start,
                                                                   int64_t V_loc, int64_t skip_row,
                                                                   const T* __restrict__ d_out, int64_t ldo,
                                                                   T* __restrict__ d_weight, int64_t ldw) {
    constexpr int V = elem<T>::kVec;
    constexpr int kSlices = 16 / V;      // column slices held in registers at a time: 1024 columns
    constexpr int kTokens = 8 / kSlices;  // tokens of the run a wavefront loads together
    __shared__ float red[kRunWaves - 1][kSlices * V][64];
    const int64_t i = blockIdx.x;
    const int64_t id = sorted_ids[i];
    // equal predecessors (k) and successors, as far as kRunBlocks - 1 each way: all loads are independent
    int k = 0, after = 0;
    bool open = true, open_after = true;
#pragma unroll
    for (int j = 1; j < kRunBlocks; ++j) {
        const bool same = i - j >= 0 && sorted_ids[i - j >= 0 ? i - j : 0] == id;
        open = open && same;
        k += open ? 1 : 0;
        const bool same_after = i + j < T_rows && sorted_ids[i + j < T_rows ? i + j : T_rows - 1] == id;
        open_after = open_after && same_after;
        after += open_after ? 1 : 0;
    }
    if (k == kRunBlocks - 1 && i - kRunBlocks >= 0 && sorted_ids[i - kRunBlocks] == id) return;  // not among the first
    const int64_t local = id - vocab_start;
    if (local < 0 || local >= V_loc || local == skip_row) return;
    const int sharers = (k + 1 + after) < kRunBlocks ? (k + 1 + after) : kRunBlocks;  // min(run length, kRunBlocks)
    const int64_t first = i - k;  // first position of the run

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    T* dst = d_weight + local * ldw;
    const int64_t slice_cols = (int64_t)64 * V;
    if (sharers < kRunBlocks) {
        // A run of one to three tokens (its length is known exactly: sharers), the common case: its first
        // block does it alone, the wavefronts take a column slice each, no exchange between them.
        if (k != 0) return;
        int64_t tok[kRunBlocks - 1];
#pragma unroll
        for (int u = 0; u < kRunBlocks - 1; ++u) tok[u] = order[first + u < T_rows ? first + u : T_rows - 1];
        for (int64_t c = wave * slice_cols + (int64_t)lane * V; c < E; c += kRunWaves * slice_cols) {
            raw16_t raw[kRunBlocks - 1];
#pragma unroll
            for (int u = 0; u < kRunBlocks - 1; ++u) {
                raw[u] = raw16_t{0u, 0u, 0u, 0u};
                if (u < sharers) raw[u] = load_raw_stream(d_out + tok[u] * ldo + c);
            }
            float acc[V];
#pragma unroll
            for (int e = 0; e < V; ++e) acc[e] = 0.0f;
#pragma unroll
            for (int u = 0; u < kRunBlocks - 1; ++u) {
                float v[V];
                unpack_raw(raw[u], v, (const T*)nullptr);
#pragma unroll
                for (int e = 0; e < V; ++e) acc[e] += v[e];
            }
            store_raw_stream(dst + c, pack_raw(acc, (const T*)nullptr));
        }
        return;
    }
    // this block's slices k, k + sharers, ...: kSlices of them per pass (a run of one token does the whole
    // row of 4 slices in one pass, as many loads in flight as a longer run has with its tokens)
    for (int64_t s0 = k; s0 * slice_cols < E; s0 += (int64_t)kSlices * sharers) {
        int64_t c[kSlices];
        bool live[kSlices];
#pragma unroll
        for (int n = 0; n < kSlices; ++n) {
            c[n] = (s0 + (int64_t)n * sharers) * slice_cols + (int64_t)lane * V;
            live[n] = c[n] < E;  // E is a multiple of V on this path
        }
        float acc[kSlices][V];
#pragma unroll
        for (int n = 0; n < kSlices; ++n)
#pragma unroll
            for (int e = 0; e < V; ++e) acc[n][e] = 0.0f;
        bool more = true;
        for (int64_t r = first + wave; more; r += kTokens * kRunWaves) {
            int64_t tok[kTokens];
            bool in_run[kTokens];
#pragma unroll
            for (int u = 0; u < kTokens; ++u) {
                const int64_t pos = r + u * kRunWaves;
                const int64_t pc = pos < T_rows ? pos : T_rows - 1;
                in_run[u] = pos < T_rows && sorted_ids[pc] == id;
                tok[u] = order[pc];
            }
            // positions are the same in all lanes of a wavefront: the branch is a scalar one, and a
            // wavefront with no token of the run (all but one when the id occurs once) loads nothing
            raw16_t raw[kTokens][kSlices];
#pragma unroll
            for (int u = 0; u < kTokens; ++u) {
#pragma unroll
                for (int n = 0; n < kSlices; ++n) raw[u][n] = raw16_t{0u, 0u, 0u, 0u};
                if (in_run[u]) {
#pragma unroll
                    for (int n = 0; n < kSlices; ++n) raw[u][n] = load_raw_stream(d_out + tok[u] * ldo + (live[n] ? c[n] : 0));
                }
            }
#pragma unroll
            for (int u = 0; u < kTokens; ++u)
#pragma unroll
                for (int n = 0; n < kSlices; ++n) {
                    float v[V];
                    unpack_raw(raw[u][n], v, (const T*)nullptr);
#pragma unroll
                    for (int e = 0; e < V; ++e) acc[n][e] += v[e];
                }
            more = in_run[kTokens - 1];  // the run is contiguous: once a position is outside it, all later ones are
        }
        if (wave > 0) {
#pragma unroll
            for (int n = 0; n < kSlices; ++n)
#pragma unroll
                for (int e = 0; e < V; ++e) red[wave - 1][n * V + e][lane] = acc[n][e];
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int n = 0; n < kSlices; ++n) {
                if (!live[n]) continue;
#pragma unroll
                for (int w = 0; w < kRunWaves - 1; ++w)
#pragma unroll
                    for (int e = 0; e < V; ++e) acc[n][e] += red[w][n * V + e][lane];
                store_raw_stream(dst + c[n], pack_raw(acc[n], (const T*)nullptr));
            }
        }
        __syncthreads();
    }
}

// Element-wise variant for rows that are not 16-byte aligned / E not a multiple of the vector.
template <typename T>
__global__ __launch_bounds__(256) void embed_bwd_generic_kernel(int64_t T_rows, int64_t E,
                                                                const int64_t* __restrict__ sorted_ids,
                                                                const int64_t* __restrict__ order, int64_t vocab_start,
                                                                int64_t V_loc, int64_t skip_row,
                                                                const T* __restrict__ d_out, int64_t ldo,
                                                                T* __restrict__ d_weight, int64_t ldw) {
    const int64_t i = blockIdx.x;
    const int64_t id = sorted_ids[i];
    if (i > 0 && sorted_ids[i - 1] == id) return;
    const int64_t local = id - vocab_start;
    if (local < 0 || local >= V_loc || local == skip_row) return;
    int64_t run = 1;
    while (i + run < T_rows && sorted_ids[i + run] == id) ++run;
    for (int64_t c = threadIdx.x; c < E; c += 256) {
        float acc = 0.0f;
        for (int64_t r = 0; r < run; ++r) acc += load_elem(d_out + order[i + r] * ldo + c);
        store_elem(d_weight + local * ldw + c, acc);
    }
}

int rows_grid(int64_t rows, int waves_per_block) {
    int64_t blocks = (rows + waves_per_block - 1) / waves_per_block;
    const int64_t cap = 256 * 8;
    blocks = blocks < cap ? blocks : cap;
    return (int)(blocks > 0 ? blocks : 1);
}

template <typename T>
int fwd_impl(int64_t T_rows, int64_t E, const int64_t* ids, int64_t vocab_start, int64_t V_loc, const void* weight,
             int64_t ldw, void* out, int64_t ldo, hipStream_t s) {
    const int vec_ok = aligned16(weight) && aligned16(out) && ldw % elem<T>::kVec == 0 && ldo % elem<T>::kVec == 0;
    hipLaunchKernelGGL(embed_fwd_kernel<T>, dim3(rows_grid(T_rows, kEmbWaves)), dim3(kEmbWaves * 64), 0, s, T_rows, E, ids,
                       vocab_start, V_loc, (const T*)weight, ldw, (T*)out, ldo, vec_ok);
    return check_launch("embed_fwd_kernel");
}

template <typename T>
int bwd_impl(int64_t T_rows, int64_t E, const int64_t* sorted_ids, const int64_t* order, int64_t vocab_start,
             int64_t V_loc, int64_t skip_row, const void* d_out, int64_t ldo, void* d_weight, int64_t ldw, hipStream_t s) {
    constexpr int V = elem<T>::kVec;
    const int w_vec = aligned16(d_weight) && ldw % V == 0;
    hipLaunchKernelGGL(zero_rows_kernel<T>, dim3(rows_grid(V_loc, 4)), dim3(256), 0, s, V_loc, E, (T*)d_weight, ldw, w_vec);
    int rc = check_launch("zero_rows_kernel");
    if (rc != CW_OK || T_rows == 0) return rc;
    const bool vec = w_vec && aligned16(d_out) && ldo % V == 0 && E % V == 0;
    if (vec) {
        hipLaunchKernelGGL(embed_bwd_kernel<T>, dim3((unsigned)T_rows), dim3(kRunWaves * 64), 0, s, T_rows, E, sorted_ids, order,
                           vocab_start, V_loc, skip_row, (const T*)d_out, ldo, (T*)d_weight, ldw);
    } else {
        hipLaunchKernelGGL(embed_bwd_generic_kernel<T>, dim3((unsigned)T_rows), dim3(256), 0, s, T_rows, E, sorted_ids, order,
                           vocab_start, V_loc, skip_row, (const T*)d_out, ldo, (T*)d_weight, ldw);
    }
    return check_launch("embed_bwd_kernel");
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int cw_embed_fwd(int64_t T, int64_t E, const int64_t* ids, int64_t vocab_start, int64_t V_loc,
                            const void* weight, int64_t ldw, void* out, int64_t ldo, int io_dtype, void* stream) {
    if (T < 0 || E <= 0 || V_loc <= 0) return fail(CW_ERR_INVALID, "cw_embed_fwd: bad shape T=%lld E=%lld V_loc=%lld", (long long)T, (long long)E, (long long)V_loc);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_embed_fwd: bad io_dtype %d", io_dtype);
    if (T == 0) return CW_OK;
    if (ids == nullptr || weight == nullptr || out == nullptr || ldw < E || ldo < E)
        return fail(CW_ERR_INVALID, "cw_embed_fwd: null pointer or leading dimension < E");
    if (const int drc = require_gfx950("cw_embed_fwd"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return fwd_impl<std::remove_pointer_t<decltype(tag)>>(T, E, ids, vocab_start, V_loc, weight, ldw, out, ldo, s);
    });
}

extern "C" int cw_embed_bwd(int64_t T, int64_t E, const int64_t* sorted_ids, const int64_t* order, int64_t vocab_start,
                            int64_t V_loc, int64_t skip_row, const void* d_out, int64_t ldo, void* d_weight,
                            int64_t ldw, int io_dtype, void* stream) {
    if (T < 0 || E <= 0 || V_loc <= 0) return fail(CW_ERR_INVALID, "cw_embed_bwd: bad shape T=%lld E=%lld V_loc=%lld", (long long)T, (long long)E, (long long)V_loc);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_embed_bwd: bad io_dtype %d", io_dtype);
    if (T > INT32_MAX) return fail(CW_ERR_INVALID, "cw_embed_bwd: too many tokens");
    if (d_weight == nullptr || ldw < E) return fail(CW_ERR_INVALID, "cw_embed_bwd: d_weight is NULL or ldw < E");
    if (T > 0 && (sorted_ids == nullptr || order == nullptr || d_out == nullptr || ldo < E))
        return fail(CW_ERR_INVALID, "cw_embed_bwd: null pointer or leading dimension < E");
    if (const int drc = require_gfx950("cw_embed_bwd"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return bwd_impl<std::remove_pointer_t<decltype(tag)>>(T, E, sorted_ids, order, vocab_start, V_loc, skip_row, d_out,
                                                              ldo, d_weight, ldw, s);
    });
}
