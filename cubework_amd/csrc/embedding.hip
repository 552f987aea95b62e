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

// Rows of the gradient that no token selects are written as zeros by the same launch that sums the others:
// the first `zero_blocks` workgroups of the backward grid. A wavefront takes kZeroRows consecutive rows, sixteen
// lanes per row; each group of sixteen finds its row's first position in the sorted ids with a 16-ary search
// (probes of one step side by side, 4 dependent loads for 8192 tokens, any run lengths), and the rows that are
// absent (or are skip_row, which the summing blocks leave alone) are then cleared by the whole wavefront.
// Summing blocks write every column of a present row, so each row of the slice is written exactly once.
constexpr int kZeroGroup = 16;
constexpr int kZeroRows = 64 / kZeroGroup;

template <typename T>
__device__ __forceinline__ void zero_absent_rows(int64_t wave_global, int lane, int T_rows, int64_t E,
                                                 const int64_t* __restrict__ sorted_ids, int64_t vocab_start,
                                                 int64_t V_loc, int64_t skip_row, T* __restrict__ d_weight, int64_t ldw,
                                                 int vec_ok) {
    constexpr int V = elem<T>::kVec;
    const int grp = lane / kZeroGroup, g = lane % kZeroGroup;
    const int64_t row0 = wave_global * kZeroRows;
    if (row0 >= V_loc) return;
    const int64_t row = row0 + grp;
    const int64_t target = vocab_start + row;
    int lo = 0, hi = row < V_loc ? T_rows : 0;  // the first position with sorted_ids >= target lies in [lo, hi]
    while (__ballot(hi > lo) != 0ull) {
        const int step = (hi - lo + kZeroGroup - 1) / kZeroGroup;
        const int pos = lo + (g + 1) * step - 1;
        const bool valid = hi > lo && pos < hi;
        const bool less = valid && sorted_ids[valid ? pos : 0] < target;
        const uint32_t mv = (uint32_t)(__ballot(valid) >> (grp * kZeroGroup)) & 0xffffu;
        const uint32_t ml = (uint32_t)(__ballot(less) >> (grp * kZeroGroup)) & 0xffffu;
        if (hi > lo) {
            const int nless = __popc(ml);
            lo += nless * step;                          // everything up to the last smaller probe is smaller
            if (nless < __popc(mv)) hi = lo + step - 1;  // the next probe is not: the answer is at or before it
        }
    }
    const bool present = row < V_loc && lo < T_rows && sorted_ids[lo < T_rows ? lo : 0] == target && row != skip_row;
    const uint64_t mp = __ballot(present);
#pragma unroll
    for (int j = 0; j < kZeroRows; ++j) {
        if (row0 + j >= V_loc || ((mp >> (j * kZeroGroup)) & 1ull)) continue;
        T* dst = d_weight + (row0 + j) * ldw;
        if (vec_ok) {
            const int64_t nvec = E / V;
            for (int64_t c = lane; c < nvec; c += 64) store_raw_stream(dst + c * V, (raw16_t){0u, 0u, 0u, 0u});
            for (int64_t c = nvec * V + lane; c < E; c += 64) store_elem(dst + c, 0.0f);
        } else {
            for (int64_t c = lane; c < E; c += 64) store_elem(dst + c, 0.0f);
        }
    }
}

int zero_blocks_for(int64_t V_loc, int waves_per_block) {
    const int64_t rows_per_block = (int64_t)kZeroRows * waves_per_block;
    return (int)((V_loc + rows_per_block - 1) / rows_per_block);
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
                                                                   T* __restrict__ d_weight, int64_t ldw,
                                                                   int zero_blocks) {
    constexpr int V = elem<T>::kVec;
    constexpr int kSlices = 16 / V;      // column slices held in registers at a time: 1024 columns
    constexpr int kTokens = 8 / kSlices;  // tokens of the run a wavefront loads together
    __shared__ float red[kRunWaves - 1][kSlices * V][64];
    if ((int)blockIdx.x < zero_blocks) {
        zero_absent_rows<T>((int64_t)blockIdx.x * kRunWaves + (threadIdx.x >> 6), threadIdx.x & 63, (int)T_rows, E, sorted_ids,
                            vocab_start, V_loc, skip_row, d_weight, ldw, 1);
        return;
    }
    const int64_t i = (int64_t)blockIdx.x - zero_blocks;
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
                                                                T* __restrict__ d_weight, int64_t ldw, int zero_blocks,
                                                                int w_vec) {
    if ((int)blockIdx.x < zero_blocks) {
        zero_absent_rows<T>((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & 63, (int)T_rows, E, sorted_ids,
                            vocab_start, V_loc, skip_row, d_weight, ldw, w_vec);
        return;
    }
    const int64_t i = (int64_t)blockIdx.x - zero_blocks;
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

// Backward straight from the unsorted ids, one launch, for batches of up to kDirMaxTokens tokens. A workgroup owns
// up to kDirRows rows of the slice, interleaved with the other workgroups' (row b, b + G, b + 2 G, ...). It reads all ids (they stay in L2: every workgroup reads the same
// 8 T bytes) and marks, per row, the tokens that select it in a bitmap in LDS. The rows that up to kDirHeavy
// tokens select are dealt round-robin to the wavefronts, which sum a row's tokens round by round, the lowest
// remaining token of every 32-token word of its bitmap, words ascending (ascending token position - what a stable
// sort by id would hand the sorted kernel - when no two of the row's tokens share a word), kDirBatch token rows in flight; the row of a row's
// first token (known from the marking pass, an LDS minimum) is requested before any wavefront of the group
// starts on the zeros, so the reads do not queue behind them in the compute unit's memory pipeline. The rows
// without tokens are then written as zeros, a fixed share per wavefront. A row that more than kDirHeavy tokens select is left to the end and summed by all
// wavefronts together, each over its contiguous range of token positions, partial sums added in wavefront
// order. Fixed orders throughout: bit-reproducible, no global atomics. Every row of the slice is written
// exactly once, so the zeros cost no pass of their own, and no token order has to be made first.
constexpr int kDirWaves = 8;
constexpr int kDirRows = 32;
constexpr int kDirRowsPerWave = kDirRows / kDirWaves;
constexpr int kDirMaxTokens = 16384;
constexpr int kDirHeavy = 8;
constexpr int kDirBatch = 2;       // token rows a wavefront has in flight (twice that on the shared rows)
constexpr int kDirIdsPerPass = 16;  // ids a thread has in flight
static_assert(kDirRows <= 64 && kDirRows % kDirWaves == 0, "one lane per row of the group; whole rows per wavefront");

template <typename T, int NV, int BATCH>
__device__ __forceinline__ void dir_load_rows(const T* __restrict__ d_out, int64_t ldo, const int (&tok)[BATCH], int n,
                                              const int64_t (&col)[NV], raw16_t (&raw)[BATCH][NV]) {
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
#pragma unroll
        for (int v = 0; v < NV; ++v) raw[b][v] = raw16_t{0u, 0u, 0u, 0u};
        if (b < n) {
#pragma unroll
            for (int v = 0; v < NV; ++v) raw[b][v] = load_raw_stream(d_out + (int64_t)tok[b] * ldo + col[v]);
        }
    }
}

template <typename T, int NV, int BATCH>
__device__ __forceinline__ void dir_accumulate(const raw16_t (&raw)[BATCH][NV], float (&acc)[NV][elem<T>::kVec]) {
    constexpr int V = elem<T>::kVec;
#pragma unroll
    for (int b = 0; b < BATCH; ++b)
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            float x[V];
            unpack_raw(raw[b][v], x, (const T*)nullptr);
#pragma unroll
            for (int e = 0; e < V; ++e) acc[v][e] += x[e];
        }
}

// One round over 64 words of a row's bitmap held one per lane in `word`: the lowest marked token of each word
// that has one, words in ascending order, goes to queue[0..n) (at most `want` of them) and is cleared in `word`.
// Returns n. LDS operations of one wavefront execute in order, so the queue can be read back right after.
__device__ __forceinline__ int dir_take_tokens(uint32_t& word, int wi, int want, uint16_t* queue) {
    const uint64_t mask = __ballot(word != 0u);
    const int rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
    if (word != 0u && rank < want) {
        queue[rank] = (uint16_t)(wi * 32 + __builtin_ctz(word));
        word &= word - 1u;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    const int n = __popcll(mask);
    return n < want ? n : want;
}

// acc += d_out rows of the tokens marked in words [w_lo, w_hi) of one row's bitmap, BATCH rows in flight.
// The order is fixed by the bitmap alone: round by round the lowest marked token of every word, words ascending.
template <typename T, int NV, int BATCH>
__device__ __forceinline__ void dir_sum_tokens(const uint32_t* bm_row, int w_lo, int w_hi, int lane, uint16_t* queue,
                                               const T* __restrict__ d_out, int64_t ldo, const int64_t (&col)[NV],
                                               float (&acc)[NV][elem<T>::kVec]) {
    for (int wb = w_lo; wb < w_hi; wb += 64) {
        const int wi = wb + lane;
        uint32_t word = wi < w_hi ? bm_row[wi] : 0u;
        for (;;) {
            const int n = dir_take_tokens(word, wi, 64, queue);
            if (n == 0) break;
            for (int i = 0; i < n; i += BATCH) {
                int tok[BATCH];
#pragma unroll
                for (int b = 0; b < BATCH; ++b) tok[b] = __builtin_amdgcn_readfirstlane((int)queue[i + b < n ? i + b : i]);
                raw16_t raw[BATCH][NV];
                dir_load_rows<T, NV, BATCH>(d_out, ldo, tok, n - i, col, raw);
                dir_accumulate<T, NV, BATCH>(raw, acc);
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");  // the queue is rewritten by the next round
        }
    }
}

template <typename T, int NV>
__device__ __forceinline__ void dir_columns(int64_t c0, int lane, int64_t E, int64_t (&col)[NV], float (&acc)[NV][elem<T>::kVec]) {
    constexpr int V = elem<T>::kVec;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t cv = c0 + ((int64_t)v * 64 + lane) * V;
        col[v] = cv < E ? cv : E - V;  // a position past the end re-reads the last vector and stores nothing
#pragma unroll
        for (int e = 0; e < V; ++e) acc[v][e] = 0.0f;
    }
}

template <typename T, int NV>
__device__ __forceinline__ void dir_store_columns(T* dst, int64_t c0, int lane, int64_t E, const int64_t (&col)[NV],
                                                  const float (&acc)[NV][elem<T>::kVec]) {
    constexpr int V = elem<T>::kVec;
#pragma unroll
    for (int v = 0; v < NV; ++v)
        if (c0 + ((int64_t)v * 64 + lane) * V < E) store_raw_stream(dst + col[v], pack_raw(acc[v], (const T*)nullptr));
}

template <typename T>
__global__ __launch_bounds__(kDirWaves * 64) void embed_bwd_direct_kernel(int T_rows, int64_t E, const int64_t* __restrict__ ids,
                                                                          int64_t vocab_start, int64_t V_loc, int64_t skip_row,
                                                                          const T* __restrict__ d_out, int64_t ldo,
                                                                          T* __restrict__ d_weight, int64_t ldw, int log2_groups) {
    constexpr int V = elem<T>::kVec;
    constexpr int NV = 4;   // column vectors per lane and pass of a row a wavefront sums alone
    constexpr int NVH = 2;  // the same for a row all wavefronts share
    constexpr int kThreads = kDirWaves * 64;
    extern __shared__ uint32_t dir_bitmap[];  // [kDirRows][words]
    __shared__ int cnt[kDirRows];
    __shared__ int first_tok[kDirRows];  // lowest token position of each row
    __shared__ float red[kDirWaves - 1][NVH * V][64];
    __shared__ uint16_t dir_queue[kDirWaves][64];  // tokens a wavefront is about to load
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int words = (T_rows + 31) >> 5;
    // Row ownership is interleaved: workgroup b of G = 2^log2_groups owns rows b, b + G, b + 2 G, ... (at most
    // kDirRows of them). Frequent tokens have neighbouring ids (the low ids of a BPE vocabulary): consecutive rows
    // per workgroup would hand one workgroup most of the batch's tokens.
    const uint64_t group_mask = ((uint64_t)1 << log2_groups) - 1;
    auto row_of = [&](int j) { return (int64_t)blockIdx.x + ((int64_t)j << log2_groups); };
    // the first ids are on their way while the bitmap is cleared
    int64_t idv[kDirIdsPerPass];
#pragma unroll
    for (int u = 0; u < kDirIdsPerPass; ++u) {
        const int t = tid + u * kThreads;
        idv[u] = T_rows > 0 ? ids[t < T_rows ? t : T_rows - 1] : 0;
    }
    for (int i = tid; i < kDirRows * words; i += kThreads) dir_bitmap[i] = 0u;
    if (tid < kDirRows) {
        cnt[tid] = 0;
        first_tok[tid] = 0x7fffffff;
    }
    __syncthreads();
    for (int t0 = 0; t0 < T_rows; t0 += kDirIdsPerPass * kThreads) {
        if (t0 > 0) {
#pragma unroll
            for (int u = 0; u < kDirIdsPerPass; ++u) {
                const int t = t0 + tid + u * kThreads;
                idv[u] = ids[t < T_rows ? t : T_rows - 1];
            }
        }
#pragma unroll
        for (int u = 0; u < kDirIdsPerPass; ++u) {
            const int t = t0 + tid + u * kThreads;
            const uint64_t local = (uint64_t)idv[u] - (uint64_t)vocab_start;  // below V_loc exactly for ids of the slice
            const uint64_t r = local >> log2_groups;
            if (t < T_rows && local < (uint64_t)V_loc && (local & group_mask) == (uint64_t)blockIdx.x) {
                atomicOr(&dir_bitmap[(int)r * words + (t >> 5)], 1u << (t & 31));
                atomicAdd(&cnt[(int)r], 1);  // integer counts and minima: the order of the updates does not matter
                atomicMin(&first_tok[(int)r], t);
            }
        }
    }
    __syncthreads();
    int my_cnt = lane < kDirRows ? cnt[lane] : 0;
    if (row_of(lane) == skip_row) my_cnt = 0;  // its tokens are ignored: the row is written as zeros
    uint64_t light = __ballot(my_cnt > 0 && my_cnt <= kDirHeavy);  // bit j: row j is summed by one wavefront
    const uint64_t heavy = __ballot(my_cnt > kDirHeavy);
    const uint64_t empty = __ballot(my_cnt == 0 && lane < kDirRows && row_of(lane) < V_loc);
    for (int k = 0; k < wave && light != 0ull; ++k) light &= light - 1;  // this wavefront's first: the wave-th set bit

    // this wavefront's first row with tokens: the first batch of its loads goes out ahead of all zeros
    uint16_t* queue = dir_queue[wave];
    int64_t col[NV];
    float acc[NV][V];
    const int first_row = light != 0ull ? __builtin_ctzll(light) : -1;
    int early[kDirBatch], n_early = 0;  // the tokens of that batch: out of the row's bitmap while its first pass runs
#pragma unroll
    for (int b = 0; b < kDirBatch; ++b) early[b] = 0;
    {
        raw16_t raw[kDirBatch][NV];
        if (first_row >= 0) {
            // the row's first token is known from the marking pass: its loads go out without a walk over the bitmap
            // (most rows have that one token); it leaves the bitmap while the row's first pass runs
            uint32_t* bm_row = dir_bitmap + first_row * words;
            early[0] = __builtin_amdgcn_readfirstlane(first_tok[first_row]);
            n_early = 1;
            if (lane == 0) atomicAnd(&bm_row[early[0] >> 5], ~(1u << (early[0] & 31)));
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            dir_columns<T, NV>(0, lane, E, col, acc);
            dir_load_rows<T, NV, kDirBatch>(d_out, ldo, early, n_early, col, raw);
        }
        __builtin_amdgcn_s_barrier();  // no data passes here: it only keeps every wavefront's zeros behind the loads above
        if (first_row >= 0) dir_accumulate<T, NV, kDirBatch>(raw, acc);
    }
    // the rest of that row, then any further rows of this wavefront (kDirWaves set bits on each time); the
    // wavefronts without such rows are writing zeros meanwhile
    for (bool first = true; light != 0ull; first = false) {
        const int j = __builtin_ctzll(light);
        T* dst = d_weight + row_of(j) * ldw;
        uint32_t* bm_row = dir_bitmap + j * words;
        for (int64_t c0 = 0; c0 < E; c0 += (int64_t)64 * V * NV) {
            if (!(first && c0 == 0)) dir_columns<T, NV>(c0, lane, E, col, acc);  // else: the sums of the first loads
            dir_sum_tokens<T, NV, kDirBatch>(bm_row, 0, words, lane, queue, d_out, ldo, col, acc);
            dir_store_columns<T, NV>(dst, c0, lane, E, col, acc);
            if (first && c0 == 0) {  // further passes over the row's columns take all of its tokens
#pragma unroll
                for (int b = 0; b < kDirBatch; ++b)
                    if (lane == b && b < n_early) atomicOr(&bm_row[early[b] >> 5], 1u << (early[b] & 31));
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            }
        }
        for (int k = 0; k < kDirWaves && light != 0ull; ++k) light &= light - 1;
    }
    // rows that many tokens select, before the zeros (the longest job of a workgroup goes first): every wavefront
    // sums the tokens of its range of positions
    const int words_per_wave = (words + kDirWaves - 1) / kDirWaves;
    const int w_lo = wave * words_per_wave;
    const int w_hi = w_lo + words_per_wave < words ? w_lo + words_per_wave : words;
    for (uint64_t todo = heavy; todo != 0ull; todo &= todo - 1) {
        const int j = __builtin_ctzll(todo);
        T* dst = d_weight + row_of(j) * ldw;
        const uint32_t* bm_row = dir_bitmap + j * words;
        for (int64_t c0 = 0; c0 < E; c0 += (int64_t)64 * V * NVH) {
            int64_t colh[NVH];
            float acch[NVH][V];
            dir_columns<T, NVH>(c0, lane, E, colh, acch);
            dir_sum_tokens<T, NVH, 4 * kDirBatch>(bm_row, w_lo, w_hi, lane, queue, d_out, ldo, colh, acch);
            if (wave > 0) {
#pragma unroll
                for (int v = 0; v < NVH; ++v)
#pragma unroll
                    for (int e = 0; e < V; ++e) red[wave - 1][v * V + e][lane] = acch[v][e];
            }
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int v = 0; v < NVH; ++v)
#pragma unroll
                    for (int w = 0; w < kDirWaves - 1; ++w)
#pragma unroll
                        for (int e = 0; e < V; ++e) acch[v][e] += red[w][v * V + e][lane];
                dir_store_columns<T, NVH>(dst, c0, lane, E, colh, acch);
            }
            __syncthreads();
        }
    }
    // zeros: the empty rows among this wavefront's kDirRowsPerWave
#pragma unroll
    for (int q = 0; q < kDirRowsPerWave; ++q) {
        const int j = wave * kDirRowsPerWave + q;
        if (!((empty >> j) & 1ull)) continue;
        T* dst = d_weight + row_of(j) * ldw;
        for (int64_t c = (int64_t)lane * V; c < E; c += 64 * V) store_raw_stream(dst + c, raw16_t{0u, 0u, 0u, 0u});
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
    // one launch: the workgroups that clear the rows without tokens first (they carry most of the bytes), then one
    // per position of the sorted order
    const bool vec = w_vec && E % V == 0 && (T_rows == 0 || (aligned16(d_out) && ldo % V == 0));
    if (vec) {
        const int zb = zero_blocks_for(V_loc, kRunWaves);
        hipLaunchKernelGGL(embed_bwd_kernel<T>, dim3((unsigned)(zb + T_rows)), dim3(kRunWaves * 64), 0, s, T_rows, E, sorted_ids,
                           order, vocab_start, V_loc, skip_row, (const T*)d_out, ldo, (T*)d_weight, ldw, zb);
    } else {
        const int zb = zero_blocks_for(V_loc, 4);
        hipLaunchKernelGGL(embed_bwd_generic_kernel<T>, dim3((unsigned)(zb + T_rows)), dim3(256), 0, s, T_rows, E, sorted_ids,
                           order, vocab_start, V_loc, skip_row, (const T*)d_out, ldo, (T*)d_weight, ldw, zb, w_vec);
    }
    return check_launch("embed_bwd_kernel");
}

// Every workgroup of the direct kernel scans all T ids for its 32 rows: T / 4 bytes of ids per row of E elements
// written. Where that exceeds the row itself by much, the token order (one sort, then one workgroup per run) is the
// faster path; measured on a 50272-row bf16 slice: T = 16384, E = 512: 81 against 66 us, E = 1024: 86 against 76,
// E = 2048: 96 against 98; T = 8192, E = 512: 32 against 35 (up to 8192 tokens two workgroups share a compute unit,
// beyond that the token bitmaps leave room for one).
bool direct_possible(int64_t T_rows, int64_t E, const void* d_out, int64_t ldo, const void* d_weight, int64_t ldw, int V) {
    return T_rows <= kDirMaxTokens && E % V == 0 && aligned16(d_weight) && ldw % V == 0 &&
           (T_rows == 0 || (aligned16(d_out) && ldo % V == 0));
}

bool direct_ok(int64_t T_rows, int64_t E, const void* d_out, int64_t ldo, const void* d_weight, int64_t ldw, int V) {
    const int64_t row_bytes = E * (16 / V);
    const bool pays = T_rows <= (T_rows <= 8192 ? 8 : 4) * row_bytes;
    return pays && direct_possible(T_rows, E, d_out, ldo, d_weight, ldw, V);
}

template <typename T>
int bwd_direct_impl(int64_t T_rows, int64_t E, const int64_t* ids, int64_t vocab_start, int64_t V_loc, int64_t skip_row,
                    const void* d_out, int64_t ldo, void* d_weight, int64_t ldw, hipStream_t s) {
    const int words = (int)((T_rows + 31) / 32);
    const int lds = kDirRows * words * (int)sizeof(uint32_t);
    if (const int rc = ensure_dynamic_lds((const void*)embed_bwd_direct_kernel<T>, lds,
                                          "embed_bwd_direct_kernel"); rc != CW_OK) return rc;
    // a power of two of workgroups, each with between kDirRows / 2 + 1 and kDirRows interleaved rows
    int log2_groups = 0;
    while (((int64_t)kDirRows << log2_groups) < V_loc) ++log2_groups;
    hipLaunchKernelGGL(embed_bwd_direct_kernel<T>, dim3(1u << log2_groups), dim3(kDirWaves * 64), lds, s, (int)T_rows, E, ids,
                       vocab_start, V_loc, skip_row, (const T*)d_out, ldo, (T*)d_weight, ldw, log2_groups);
    return check_launch("embed_bwd_direct_kernel");
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
    if (T > INT32_MAX / 2 || V_loc > INT32_MAX / 2)
        return fail(CW_ERR_INVALID, "cw_embed_bwd: more than 2^30 tokens or rows (the grid is one launch over both)");
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

extern "C" int cw_embed_bwd_ids_supported(int64_t T, int64_t E, const void* d_out, int64_t ldo, const void* d_weight,
                                          int64_t ldw, int io_dtype) {
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16) return 0;
    return direct_ok(T, E, d_out, ldo, d_weight, ldw, io_dtype == CW_F32 ? 4 : 8) ? 1 : 0;
}

extern "C" int cw_embed_bwd_ids(int64_t T, int64_t E, const int64_t* ids, int64_t vocab_start, int64_t V_loc,
                                int64_t skip_row, const void* d_out, int64_t ldo, void* d_weight, int64_t ldw,
                                int io_dtype, void* stream) {
    if (T < 0 || E <= 0 || V_loc <= 0) return fail(CW_ERR_INVALID, "cw_embed_bwd_ids: bad shape T=%lld E=%lld V_loc=%lld", (long long)T, (long long)E, (long long)V_loc);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_embed_bwd_ids: bad io_dtype %d", io_dtype);
    if (V_loc > INT32_MAX / 2) return fail(CW_ERR_INVALID, "cw_embed_bwd_ids: more than 2^30 rows");
    if (d_weight == nullptr || ldw < E) return fail(CW_ERR_INVALID, "cw_embed_bwd_ids: d_weight is NULL or ldw < E");
    if (T > 0 && (ids == nullptr || d_out == nullptr || ldo < E))
        return fail(CW_ERR_INVALID, "cw_embed_bwd_ids: null pointer or leading dimension < E");
    if (!direct_possible(T, E, d_out, ldo, d_weight, ldw, io_dtype == CW_F32 ? 4 : 8))
        return fail(CW_ERR_UNSUPPORTED,
                    "cw_embed_bwd_ids: needs T <= %d, 16-byte aligned rows and E a multiple of the 16-byte vector; "
                    "use cw_embed_sort_ids + cw_embed_bwd", kDirMaxTokens);
    if (const int drc = require_gfx950("cw_embed_bwd_ids"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return bwd_direct_impl<std::remove_pointer_t<decltype(tag)>>(T, E, ids, vocab_start, V_loc, skip_row, d_out, ldo,
                                                                     d_weight, ldw, s);
    });
}
