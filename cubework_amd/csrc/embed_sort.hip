// Token order for the embedding backward, for gfx950: the ids of one batch sorted by the row of this rank's
// vocabulary slice they select, ties in token order (what a stable sort by id gives for the ids in
// range). Ids outside [vocab_start, vocab_start + V_loc) select no row of the slice; they are all mapped
// to the value vocab_start + V_loc, so they sort behind every row and the backward kernel skips them.
//
// Up to kRankTokens tokens (a training batch per rank): one launch that computes every token's final
// position directly, rank(t) = #{t' : row' < row} + #{t' < t : row' == row}, by comparing it with all
// the others. That is T^2 compares instead of T log^2 T, but they are independent 2-instruction
// compares spread over the whole chip (3.4 us of VALU time for 8192 tokens), where a sorting network
// of that size lives in one workgroup's LDS and is bound by its 91 dependent barrier-separated steps.
// Longer inputs: a bitonic network over 64-bit keys (row << 32 | token position), chunks of kChunkKeys
// sorted in LDS, the steps whose partner distance reaches across chunks as separate launches over a
// caller workspace.
#include "cw_common.h"

namespace cw {

namespace {

constexpr int kSortThreads = 1024;
constexpr int kChunkKeys = 4096;   // keys one workgroup sorts in LDS in the network path
constexpr uint64_t kPadKey = ~0ull;
constexpr int kRankTokens = 16384;  // longest input of the direct-rank path (rows of all tokens in 64 KB of LDS)
constexpr int kRankWaves = 16;
constexpr int kRankUnit = 64 * 2 * kRankWaves;  // granularity of the padded token count
constexpr uint32_t kPadRow = 0xffffffffu;

__device__ __forceinline__ uint32_t row_of(int64_t id, int64_t vocab_start, int64_t V_loc) {
    // unsigned difference: below V_loc exactly when vocab_start <= id < vocab_start + V_loc
    const uint64_t u = (uint64_t)id - (uint64_t)vocab_start;
    return (uint32_t)(u < (uint64_t)V_loc ? u : (uint64_t)V_loc);
}

// One workgroup per 32 tokens. A wavefront's lanes 0-31 and 32-63 hold the same 32 tokens and count over
// different halves of the wavefront's sixteenth of all tokens (an LDS read with two distinct addresses
// per wavefront is still a broadcast); the 32 counts per token are added through LDS and the first
// wavefront writes the token to its position. t_pad = T rounded up to a multiple of kRankUnit; rows of
// the padding never count.
__global__ __launch_bounds__(kRankWaves * 64) void rank_scatter_kernel(const int64_t* __restrict__ ids, int T, int t_pad,
                                                                       int64_t vocab_start, int64_t V_loc,
                                                                       int64_t* __restrict__ sorted_ids,
                                                                       int64_t* __restrict__ order) {
    extern __shared__ uint32_t rank_lds[];
    uint32_t* rows = rank_lds;                 // [t_pad]
    uint32_t* counts = rank_lds + t_pad;       // [kRankWaves][64]
    for (int i = threadIdx.x; i < t_pad; i += kRankWaves * 64) {
        const int64_t id = ids[i < T ? i : 0];
        rows[i] = i < T ? row_of(id, vocab_start, V_loc) : kPadRow;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int tok = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile0 = blockIdx.x * 32;         // first token of this workgroup
    const int own = tile0 & ~63;               // the 64-aligned chunk that holds the workgroup's tokens
    const int t = tile0 + tok;
    const uint32_t r = rows[t];                // t < t_pad: the grid covers ceil(T / 32) tiles
    const int span = t_pad / (2 * kRankWaves); // tokens one half-wavefront counts over, a multiple of 64
    const int first = (2 * wave + half) * span;
    uint32_t cnt = 0;
    // tokens before this one count when their row is <= r, tokens after it when it is < r; the chunk
    // with the workgroup's own tokens is left out here (bound 0: nothing is below it)
    for (int c = 0; c < span; c += 64) {
        const int c0 = first + c;
        const uint4* src = reinterpret_cast<const uint4*>(rows + c0);
        const uint32_t bound = c0 == own ? 0u : r + (c0 < own ? 1u : 0u);
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const uint4 v = src[q];
            cnt += v.x < bound ? 1u : 0u;
            cnt += v.y < bound ? 1u : 0u;
            cnt += v.z < bound ? 1u : 0u;
            cnt += v.w < bound ? 1u : 0u;
        }
    }
    if (own / (2 * span) == wave) {
        for (int e = 0; e < 32; ++e) {
            const int other_t = own + 32 * half + e;
            cnt += rows[other_t] < r + (other_t < t ? 1u : 0u) ? 1u : 0u;
        }
    }
    counts[wave * 64 + lane] = cnt;
    __syncthreads();
    if (wave == 0 && half == 0 && t < T) {
        uint32_t pos = 0;
#pragma unroll
        for (int w = 0; w < kRankWaves; ++w) pos += counts[w * 64 + tok] + counts[w * 64 + 32 + tok];
        sorted_ids[pos] = vocab_start + (int64_t)r;
        order[pos] = t;
    }
}

__device__ __forceinline__ uint64_t make_key(int64_t id, int64_t vocab_start, int64_t V_loc, uint32_t pos) {
    return ((uint64_t)row_of(id, vocab_start, V_loc) << 32) | pos;
}

// One compare-exchange step of stage k with partner distance j (< n_local) on a chunk held in LDS.
__device__ __forceinline__ void local_step(uint64_t* lds, int n_local, int base, int k, int j) {
    for (int p = threadIdx.x; p < (n_local >> 1); p += kSortThreads) {
        const int i = ((p & ~(j - 1)) << 1) | (p & (j - 1));
        const int l = i | j;
        const bool ascending = ((base + i) & k) == 0;
        const uint64_t a = lds[i], b = lds[l];
        if ((a > b) == ascending) {
            lds[i] = b;
            lds[l] = a;
        }
    }
}

// BUILD: make the keys from the ids and run the stages k = 2 .. n_local completely.
// otherwise: take the keys from `keys`, run the steps j = n_local/2 .. 1 of stage k_stage.
// last: write sorted_ids / order (the first T entries) instead of the keys.
template <bool BUILD>
__global__ __launch_bounds__(kSortThreads) void sort_local_kernel(const int64_t* __restrict__ ids, int T, int64_t vocab_start,
                                                                  int64_t V_loc, uint64_t* __restrict__ keys, int n_local,
                                                                  int k_stage, int last, int64_t* __restrict__ sorted_ids,
                                                                  int64_t* __restrict__ order) {
    extern __shared__ uint64_t lds[];
    const int base = blockIdx.x * n_local;
    for (int i = threadIdx.x; i < n_local; i += kSortThreads) {
        const int g = base + i;
        uint64_t key;
        if (BUILD) {
            const int64_t id = ids[g < T ? g : 0];
            key = g < T ? make_key(id, vocab_start, V_loc, (uint32_t)g) : kPadKey;
        } else {
            key = keys[g];
        }
        lds[i] = key;
    }
    __syncthreads();
    if (BUILD) {
        for (int k = 2; k <= n_local; k <<= 1)
            for (int j = k >> 1; j > 0; j >>= 1) {
                local_step(lds, n_local, base, k, j);
                __syncthreads();
            }
    } else {
        for (int j = n_local >> 1; j > 0; j >>= 1) {
            local_step(lds, n_local, base, k_stage, j);
            __syncthreads();
        }
    }
    for (int i = threadIdx.x; i < n_local; i += kSortThreads) {
        const int g = base + i;
        const uint64_t key = lds[i];
        if (last) {
            if (g < T) {
                sorted_ids[g] = vocab_start + (int64_t)(key >> 32);
                order[g] = (int64_t)(key & 0xffffffffull);
            }
        } else {
            keys[g] = key;
        }
    }
}

// One compare-exchange step of stage k with partner distance j across chunks, one pair per thread.
__global__ __launch_bounds__(256) void sort_global_step_kernel(uint64_t* __restrict__ keys, int n_pairs, int k, int j) {
    const int p = blockIdx.x * 256 + threadIdx.x;
    if (p >= n_pairs) return;
    const int i = ((p & ~(j - 1)) << 1) | (p & (j - 1));
    const int l = i | j;
    const bool ascending = (i & k) == 0;
    const uint64_t a = keys[i], b = keys[l];
    if ((a > b) == ascending) {
        keys[i] = b;
        keys[l] = a;
    }
}

int64_t padded_keys(int64_t T) {
    int64_t n = 2;
    while (n < T) n <<= 1;
    return n;
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int64_t cw_embed_sort_workspace_bytes(int64_t T) {
    if (T <= kRankTokens) return 0;
    return padded_keys(T) * (int64_t)sizeof(uint64_t);
}

extern "C" int cw_embed_sort_ids(int64_t T, const int64_t* ids, int64_t vocab_start, int64_t V_loc, int64_t* sorted_ids,
                                 int64_t* order, void* workspace, int64_t workspace_bytes, void* stream) {
    if (T < 0 || T > (1ll << 30)) return fail(CW_ERR_INVALID, "cw_embed_sort_ids: T=%lld outside [0, 2^30]", (long long)T);
    if (V_loc <= 0 || V_loc >= 0xffffffffll) return fail(CW_ERR_INVALID, "cw_embed_sort_ids: V_loc=%lld outside (0, 2^32-1)", (long long)V_loc);
    if (vocab_start < 0 || vocab_start > INT64_MAX - V_loc) return fail(CW_ERR_INVALID, "cw_embed_sort_ids: bad vocab_start %lld", (long long)vocab_start);
    if (T == 0) return CW_OK;
    if (ids == nullptr || sorted_ids == nullptr || order == nullptr) return fail(CW_ERR_INVALID, "cw_embed_sort_ids: null pointer");
    const int64_t need = cw_embed_sort_workspace_bytes(T);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 7u) != 0))
        return fail(CW_ERR_INVALID, "cw_embed_sort_ids: workspace of %lld bytes (8-byte aligned) required", (long long)need);
    if (const int drc = require_gfx950("cw_embed_sort_ids"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (T <= kRankTokens) {
        const int t_pad = (int)((T + kRankUnit - 1) / kRankUnit) * kRankUnit;
        const int lds_bytes = (t_pad + kRankWaves * 64) * (int)sizeof(uint32_t);
        if (const int lrc = ensure_dynamic_lds((const void*)rank_scatter_kernel, (int)((kRankTokens + kRankWaves * 64) * (int)sizeof(uint32_t)), "rank_scatter_kernel"); lrc != CW_OK) return lrc;
        hipLaunchKernelGGL(rank_scatter_kernel, dim3((unsigned)((T + 31) / 32)), dim3(kRankWaves * 64), lds_bytes, s, ids, (int)T,
                           t_pad, vocab_start, V_loc, sorted_ids, order);
        return check_launch("rank_scatter_kernel");
    }
    const int n = (int)padded_keys(T);
    const int n_local = n < kChunkKeys ? n : kChunkKeys;
    const int chunks = n / n_local;
    const int lds_bytes = n_local * (int)sizeof(uint64_t);
    if (const int lrc = ensure_dynamic_lds((const void*)sort_local_kernel<true>, kChunkKeys * 8, "sort_local_kernel"); lrc != CW_OK)
        return lrc;
    if (const int lrc = ensure_dynamic_lds((const void*)sort_local_kernel<false>, kChunkKeys * 8, "sort_local_kernel"); lrc != CW_OK)
        return lrc;
    uint64_t* keys = (uint64_t*)workspace;
    hipLaunchKernelGGL(sort_local_kernel<true>, dim3(chunks), dim3(kSortThreads), lds_bytes, s, ids, (int)T, vocab_start, V_loc,
                       keys, n_local, 0, chunks == 1 ? 1 : 0, sorted_ids, order);
    int rc = check_launch("sort_local_kernel<build>");
    if (rc != CW_OK) return rc;
    for (int64_t k = 2ll * n_local; k <= n; k <<= 1) {
        for (int64_t j = k >> 1; j >= n_local; j >>= 1) {
            hipLaunchKernelGGL(sort_global_step_kernel, dim3((n / 2 + 255) / 256), dim3(256), 0, s, keys, n / 2, (int)k, (int)j);
            rc = check_launch("sort_global_step_kernel");
            if (rc != CW_OK) return rc;
        }
        hipLaunchKernelGGL(sort_local_kernel<false>, dim3(chunks), dim3(kSortThreads), lds_bytes, s, ids, (int)T, vocab_start, V_loc,
                           keys, n_local, (int)k, k == n ? 1 : 0, sorted_ids, order);
        rc = check_launch("sort_local_kernel<merge>");
        if (rc != CW_OK) return rc;
    }
    return CW_OK;
}
