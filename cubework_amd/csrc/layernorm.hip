// LayerNorm2D / LayerNorm3D per-rank kernels for gfx950: partial statistics,
// normalise (+ affine), backward partials (row sums + dgamma/dbeta column
// partials) and dx. All are HBM-streaming kernels: one 64-lane wavefront owns
// a row, every lane moves 16-byte vectors, row reductions are wavefront
// shuffles, column reductions go through registers -> LDS tree -> a small
// per-block partial in global memory (no atomics, so results are
// deterministic).
//
// Rows of up to 8 x 64 vectors (bf16: 4096 columns, fp32: 2048) take the
// "tile" kernels: a wavefront loads NR whole rows into registers with all of
// its loads in flight at once (non-temporal, each byte is used once), so a
// row is read from memory exactly once even where two passes over it are
// needed, and the memory system always sees several KiB outstanding per
// wavefront. Wider or unaligned rows take the looping kernels below them.
#include <type_traits>

#include "cw_common.h"
#include "reduce_cols.h"

namespace cw {

namespace {

constexpr int kLnBlock = 256;  // 4 wavefronts; one row per wavefront per trip

// Rows a wavefront of the tile kernels holds at a time, by chunks per row, and
// the resident blocks per compute unit the grid is capped at (measured on
// 16384 x 1024 bf16: more rows per wavefront cost registers and gained nothing).
constexpr int kRowsAt1Chunk = 2;
constexpr int kRowsAt2Chunks = 1;
constexpr int kRowsAt4Chunks = 1;
constexpr int kTileBlocksPerCu = 8;

// Sum of (x-mu) and (x-mu)^2 over one row; every lane returns the full sums.
template <typename T>
__device__ __forceinline__ void row_moments(const T* __restrict__ xr, int64_t C, float mu, bool vec_ok,
                                            int lane, float& s1, float& s2) {
    constexpr int V = elem<T>::kVec;
    float a1 = 0.0f, a2 = 0.0f;
    if (vec_ok) {
        const int64_t nvec = C / V;
        for (int64_t i = lane; i < nvec; i += 64) {
            float v[V];
            load_vec(xr + i * V, v);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float d = v[e] - mu;
                a1 += d;
                a2 += d * d;
            }
        }
        for (int64_t c = nvec * V + lane; c < C; c += 64) {
            const float d = load_elem(xr + c) - mu;
            a1 += d;
            a2 += d * d;
        }
    } else {
        for (int64_t c = lane; c < C; c += 64) {
            const float d = load_elem(xr + c) - mu;
            a1 += d;
            a2 += d * d;
        }
    }
    s1 = wave_sum(a1);
    s2 = wave_sum(a2);
}

template <typename T>
__global__ __launch_bounds__(kLnBlock) void ln_stats_kernel(int64_t R, int64_t C, const T* __restrict__ x,
                                                            int64_t ld, int mode, const float* __restrict__ mean,
                                                            float* __restrict__ stats, int vec_ok) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kLnBlock / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (kLnBlock / 64);
    for (int64_t row = wave; row < R; row += nwaves) {
        const float mu = (mode == CW_LN_TWO_PASS && mean != nullptr) ? mean[row] : 0.0f;
        float s1, s2;
        row_moments(x + row * ld, C, mu, vec_ok != 0, lane, s1, s2);
        if (lane == 0) {
            stats[2 * row] = s1;
            stats[2 * row + 1] = (mode == CW_LN_TWO_PASS && mean == nullptr) ? 0.0f : s2;
        }
    }
}

// mean / rstd from whole-hidden-size statistics.
__device__ __forceinline__ void finish_stats(int mode, float s1, float s2, float inv_h, float eps, float& mean,
                                             float& rstd) {
    float var;
    if (mode == CW_LN_ONE_PASS) {
        mean = s1 * inv_h;
        var = s2 * inv_h - mean * mean;
    } else {
        mean = s1;
        var = s2 * inv_h;
    }
    rstd = __builtin_amdgcn_rsqf(var + eps);  // hardware reciprocal square root, 1 ulp
}

template <typename T, bool FUSED>
__global__ __launch_bounds__(kLnBlock) void ln_normalize_kernel(int64_t R, int64_t C, const T* __restrict__ x,
                                                                int64_t ld, const float* __restrict__ stats,
                                                                int mode, float inv_h, float eps,
                                                                const T* __restrict__ gamma,
                                                                const T* __restrict__ beta, T* __restrict__ y,
                                                                int64_t ldy, float* __restrict__ mean_rstd,
                                                                int vec_ok) {
    constexpr int V = elem<T>::kVec;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kLnBlock / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (kLnBlock / 64);
    for (int64_t row = wave; row < R; row += nwaves) {
        const T* xr = x + row * ld;
        T* yr = y + row * ldy;
        float mean, rstd;
        if constexpr (FUSED) {
            float s1, s2;
            row_moments(xr, C, 0.0f, vec_ok != 0, lane, s1, s2);
            if (mode == CW_LN_TWO_PASS) {
                const float mu = s1 * inv_h;
                float d1, d2;
                row_moments(xr, C, mu, vec_ok != 0, lane, d1, d2);
                finish_stats(mode, mu, d2, inv_h, eps, mean, rstd);
            } else {
                finish_stats(mode, s1, s2, inv_h, eps, mean, rstd);
            }
        } else {
            finish_stats(mode, stats[2 * row], stats[2 * row + 1], inv_h, eps, mean, rstd);
        }
        if (mean_rstd != nullptr && lane == 0) {
            mean_rstd[2 * row] = mean;
            mean_rstd[2 * row + 1] = rstd;
        }
        if (vec_ok) {
            const int64_t nvec = C / V;
            for (int64_t i = lane; i < nvec; i += 64) {
                float v[V], g[V], b[V];
                load_vec(xr + i * V, v);
                if (gamma != nullptr) load_vec(gamma + i * V, g);
                if (beta != nullptr) load_vec(beta + i * V, b);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    float xh = (v[e] - mean) * rstd;
                    if (gamma != nullptr) xh *= g[e];
                    if (beta != nullptr) xh += b[e];
                    v[e] = xh;
                }
                store_vec(yr + i * V, v);
            }
            for (int64_t c = nvec * V + lane; c < C; c += 64) {
                float xh = (load_elem(xr + c) - mean) * rstd;
                if (gamma != nullptr) xh *= load_elem(gamma + c);
                if (beta != nullptr) xh += load_elem(beta + c);
                store_elem(yr + c, xh);
            }
        } else {
            for (int64_t c = lane; c < C; c += 64) {
                float xh = (load_elem(xr + c) - mean) * rstd;
                if (gamma != nullptr) xh *= load_elem(gamma + c);
                if (beta != nullptr) xh += load_elem(beta + c);
                store_elem(yr + c, xh);
            }
        }
    }
}

// ---- register-tile kernels ------------------------------------------------
// Lane l of a wavefront owns columns (j*64 + l)*V .. +V-1, j < NCH, of each of
// the NR rows the wavefront holds. C % V == 0 and 16-byte aligned rows.
//
// Loads are never predicated: a chunk past the end of the row reads column 0
// and a row past R reads row R-1, then the value is replaced by zero (chunk)
// or the result is not stored (row). A load under a branch would make the
// compiler wait for the loads before it, which serialises the memory traffic
// of the wavefront.
constexpr int kTileWaves = 4;

template <typename T>
__device__ __forceinline__ bool chunk_valid(int j, int lane, int64_t C) {
    return ((int64_t)j * 64 + lane) * elem<T>::kVec < C;
}

template <typename T, int NCH, int NR>
struct RowTile {
    static constexpr int V = elem<T>::kVec;
    raw16_t raw[NR][NCH];

    // EXACT: the row is exactly NCH chunks wide, so no chunk needs a bounds check.
    template <bool EXACT = false>
    __device__ __forceinline__ void load(const T* __restrict__ p, int64_t ld, int64_t row0, int64_t R, int64_t C,
                                         int lane) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int64_t row = (row0 + r < R) ? row0 + r : R - 1;
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                if constexpr (EXACT) {
                    raw[r][j] = load_raw_stream(p + row * ld + ((int64_t)j * 64 + lane) * V);
                    continue;
                }
                const bool ok = chunk_valid<T>(j, lane, C);
                const int64_t c0 = ok ? ((int64_t)j * 64 + lane) * V : 0;
                const raw16_t u = load_raw_stream(p + row * ld + c0);
                raw[r][j].x = ok ? u.x : 0u;
                raw[r][j].y = ok ? u.y : 0u;
                raw[r][j].z = ok ? u.z : 0u;
                raw[r][j].w = ok ? u.w : 0u;
            }
        }
    }

    // Replaces the rows past R (copies of row R-1) by zeros.
    __device__ __forceinline__ void zero_dead_rows(int64_t row0, int64_t R) {
#pragma unroll
        for (int r = 1; r < NR; ++r) {
            const bool live = row0 + r < R;
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                raw[r][j].x = live ? raw[r][j].x : 0u;
                raw[r][j].y = live ? raw[r][j].y : 0u;
                raw[r][j].z = live ? raw[r][j].z : 0u;
                raw[r][j].w = live ? raw[r][j].w : 0u;
            }
        }
    }
};

// gamma / beta chunks of a lane (zero where absent or past the end).
template <typename T, int NCH>
__device__ __forceinline__ void load_param_chunks(const T* __restrict__ p, int64_t C, int lane, raw16_t (&out)[NCH]) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        out[j] = (raw16_t){0u, 0u, 0u, 0u};
        if (p != nullptr && chunk_valid<T>(j, lane, C)) out[j] = load_raw(p + ((int64_t)j * 64 + lane) * elem<T>::kVec);
    }
}

// Sum of (x-mu) and (x-mu)^2 over row r of a tile; every lane gets the sums.
template <typename T, int NCH, int NR>
__device__ __forceinline__ void tile_moments(const RowTile<T, NCH, NR>& t, int r, int64_t C, float mu, int lane,
                                             float& s1, float& s2) {
    constexpr int V = elem<T>::kVec;
    float a1 = 0.0f, a2 = 0.0f;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const float mu_j = chunk_valid<T>(j, lane, C) ? mu : 0.0f;  // the zeros of an absent chunk add nothing
        float v[V];
        unpack_raw(t.raw[r][j], v, (const T*)nullptr);
#pragma unroll
        for (int e = 0; e < V; ++e) {
            const float d = v[e] - mu_j;
            a1 += d;
            a2 += d * d;
        }
    }
    s1 = wave_sum(a1);
    s2 = wave_sum(a2);
}

// EXACT (here and in the two kernels below): rows of exactly NCH chunks, and a grid with one tile per
// wavefront, so a wavefront issues all its loads, works and exits: no trip loop, no per-chunk bounds
// checks. On 16384 x 1024 bf16 that is the difference between 0.58 and 0.71 of the HBM peak for the
// normalise kernel; wavefronts that loop read measurably slower at these sizes, however the loop is
// pipelined.
template <typename T, int NCH, int NR, bool EXACT>
__global__ __launch_bounds__(kTileWaves * 64) void ln_stats_tile_kernel(int64_t R, int64_t C,
                                                                        const T* __restrict__ x, int64_t ld, int mode,
                                                                        const float* __restrict__ mean,
                                                                        float* __restrict__ stats) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kTileWaves + (threadIdx.x >> 6);
    const int64_t step = (int64_t)gridDim.x * kTileWaves * NR;
    const bool centred = mode == CW_LN_TWO_PASS && mean != nullptr;
    if constexpr (EXACT) {
        // plain sums (the one-pass statistics and the first exchange of the two-pass flavour): no mean to fetch
        if (!centred) {
            const int64_t row0 = wave * NR;
            if (row0 >= R) return;
            RowTile<T, NCH, NR> t;
            t.template load<true>(x, ld, row0, R, C, lane);
            float s1[NR], s2[NR];
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                tile_moments(t, r, (int64_t)NCH * 64 * elem<T>::kVec, 0.0f, lane, s1[r], s2[r]);
                if (mode == CW_LN_TWO_PASS) s2[r] = 0.0f;
            }
            if constexpr (NR % 2 == 0) {
                if ((reinterpret_cast<uintptr_t>(stats) & 15u) == 0) {
                    // every lane holds all sums: lane i stores the 16 bytes of rows 2i and 2i + 1, one instruction for
                    // the tile (four rows = one whole 32-byte sector; 8-byte stores per row measured 0.25 us slower on
                    // 16384 rows)
                    typedef float f32x4_t __attribute__((ext_vector_type(4)));
                    f32x4_t q = {s1[0], s2[0], s1[1], s2[1]};
#pragma unroll
                    for (int i = 1; i < NR / 2; ++i)
                        if (lane == i) q = (f32x4_t){s1[2 * i], s2[2 * i], s1[2 * i + 1], s2[2 * i + 1]};
                    if (lane < NR / 2) {
                        const int64_t row = row0 + 2 * lane;
                        if (row + 1 < R) *reinterpret_cast<f32x4_t*>(stats + 2 * row) = q;
                        else if (row < R) {
                            stats[2 * row] = q.x;
                            stats[2 * row + 1] = q.y;
                        }
                    }
                    return;
                }
            }
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                if (lane == 0 && row0 + r < R) {
                    typedef float f32x2_t __attribute__((ext_vector_type(2)));
                    const f32x2_t pair = {s1[r], s2[r]};
                    *reinterpret_cast<f32x2_t*>(stats + 2 * (row0 + r)) = pair;
                }
            }
            return;
        }
    }
    for (int64_t row0 = wave * NR; row0 < R; row0 += step) {
        RowTile<T, NCH, NR> t;
        t.template load<EXACT>(x, ld, row0, R, C, lane);
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int64_t row = row0 + r;
            const float mu = centred ? mean[row < R ? row : R - 1] : 0.0f;
            float s1, s2;
            tile_moments(t, r, EXACT ? (int64_t)NCH * 64 * elem<T>::kVec : C, mu, lane, s1, s2);
            if (lane == 0 && row < R) {
                typedef float f32x2_t __attribute__((ext_vector_type(2)));
                const f32x2_t pair = {s1, (mode == CW_LN_TWO_PASS && mean == nullptr) ? 0.0f : s2};
                *reinterpret_cast<f32x2_t*>(stats + 2 * row) = pair;  // one 8-byte store
            }
        }
        if constexpr (EXACT) return;  // the grid has a tile for every wavefront
    }
}

template <typename T, int NCH, int NR, bool FUSED, bool EXACT>
__global__ __launch_bounds__(kTileWaves * 64) void ln_normalize_tile_kernel(
    int64_t R, int64_t C, const T* __restrict__ x, int64_t ld, const float* __restrict__ stats, int mode, float inv_h,
    float eps, const T* __restrict__ gamma, const T* __restrict__ beta, T* __restrict__ y, int64_t ldy,
    float* __restrict__ mean_rstd) {
    constexpr int V = elem<T>::kVec;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kTileWaves + (threadIdx.x >> 6);
    const int64_t step = (int64_t)gridDim.x * kTileWaves * NR;
    // gamma and beta stay in registers across rows while they fit beside the tile; the widest tiles (8 chunk-rows)
    // read them per chunk from cache instead: with them the fp32 tile passed 256 registers and the 16-bit one ran at
    // three wavefronts per SIMD (140 registers; 8192 x 4096 bf16 fused forward 28.1 -> 26.8 us without them)
    constexpr bool kHoldParams = !(NCH * NR >= 8);
    constexpr int NP = kHoldParams ? NCH : 1;
    raw16_t g_raw[NP], b_raw[NP];
    if constexpr (kHoldParams && !EXACT) {
        load_param_chunks<T, NCH>(gamma, C, lane, g_raw);
        load_param_chunks<T, NCH>(beta, C, lane, b_raw);
    }
    if constexpr (EXACT) C = (int64_t)NCH * 64 * V;  // a compile-time width: chunk_valid() folds to true
    for (int64_t row0 = wave * NR; row0 < R; row0 += step) {
        RowTile<T, NCH, NR> t;
        t.template load<EXACT>(x, ld, row0, R, C, lane);
        if constexpr (kHoldParams && EXACT) {  // behind the row loads: the rows are what the wavefront waits for
            load_param_chunks<T, NCH>(gamma, C, lane, g_raw);
            load_param_chunks<T, NCH>(beta, C, lane, b_raw);
        }
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int64_t row = row0 + r;
            const int64_t row_c = row < R ? row : R - 1;
            float mean, rstd;
            if constexpr (FUSED) {
                float s1, s2;
                tile_moments(t, r, C, 0.0f, lane, s1, s2);
                if (mode == CW_LN_TWO_PASS) {
                    const float mu = s1 * inv_h;
                    float d1, d2;
                    tile_moments(t, r, C, mu, lane, d1, d2);
                    finish_stats(mode, mu, d2, inv_h, eps, mean, rstd);
                } else {
                    finish_stats(mode, s1, s2, inv_h, eps, mean, rstd);
                }
            } else {
                finish_stats(mode, stats[2 * row_c], stats[2 * row_c + 1], inv_h, eps, mean, rstd);
            }
            if (mean_rstd != nullptr && lane == 0 && row < R) {
                mean_rstd[2 * row] = mean;
                mean_rstd[2 * row + 1] = rstd;
            }
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                float v[V], g[V], b[V];
                unpack_raw(t.raw[r][j], v, (const T*)nullptr);
                if constexpr (kHoldParams) {
                    unpack_raw(g_raw[j], g, (const T*)nullptr);
                    unpack_raw(b_raw[j], b, (const T*)nullptr);
                } else {
                    const bool ok = chunk_valid<T>(j, lane, C);
                    const int64_t c0 = ok ? ((int64_t)j * 64 + lane) * V : 0;
                    const raw16_t zero = {0u, 0u, 0u, 0u};
                    unpack_raw(gamma != nullptr ? load_raw(gamma + c0) : zero, g, (const T*)nullptr);
                    unpack_raw(beta != nullptr ? load_raw(beta + c0) : zero, b, (const T*)nullptr);
                }
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    float xh = (v[e] - mean) * rstd;
                    if (gamma != nullptr) xh *= g[e];
                    if (beta != nullptr) xh += b[e];
                    v[e] = xh;
                }
                if (row < R && chunk_valid<T>(j, lane, C))
                    store_raw_stream(y + row * ldy + ((int64_t)j * 64 + lane) * V, pack_raw(v, (const T*)nullptr));
            }
        }
        if constexpr (EXACT) return;
    }
}

// Partial statistics of rows wider than a wavefront's registers, laid out like ln_forward_split_kernel:
// `wpr` wavefronts share a row and add their moments through LDS (one barrier per row).
template <typename T, int NCH, int MAXW>
__global__ __launch_bounds__(MAXW * 64) void ln_stats_split_kernel(int64_t R, int64_t C, const T* __restrict__ x,
                                                                   int64_t ld, int mode,
                                                                   const float* __restrict__ mean,
                                                                   float* __restrict__ stats, int wpr) {
    constexpr int V = elem<T>::kVec;
    __shared__ float lds_sums[2][MAXW][2];  // [trip parity][wavefront][moment]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nrg = (int)(blockDim.x >> 6) / wpr;
    const int rg = wave / wpr, seg = wave - rg * wpr;
    const int64_t col0 = (int64_t)seg * (NCH * 64 * V);
    const int64_t Cs = C - col0;
    x += col0;
    const bool centred = mode == CW_LN_TWO_PASS && mean != nullptr;
    const int64_t step = (int64_t)gridDim.x * nrg;
    int64_t base = (int64_t)blockIdx.x * nrg;
    RowTile<T, NCH, 1> t;
    if (base < R) t.load(x, ld, base + rg, R, Cs, lane);
    for (int trip = 0; base < R; base += step, ++trip) {
        RowTile<T, NCH, 1> next;
        const bool more = base + step < R;
        if (more) next.load(x, ld, base + step + rg, R, Cs, lane);
        const int64_t row = base + rg;
        const float mu = centred ? mean[row < R ? row : R - 1] : 0.0f;
        float s1, s2;
        tile_moments(t, 0, Cs, mu, lane, s1, s2);
        if (lane == 0) {
            lds_sums[trip & 1][wave][0] = s1;
            lds_sums[trip & 1][wave][1] = s2;
        }
        __syncthreads();
        if (seg == 0 && lane == 0 && row < R) {
            s1 = 0.0f;
            s2 = 0.0f;
            for (int w = 0; w < wpr; ++w) {
                s1 += lds_sums[trip & 1][rg * wpr + w][0];
                s2 += lds_sums[trip & 1][rg * wpr + w][1];
            }
            stats[2 * row] = s1;
            stats[2 * row + 1] = (mode == CW_LN_TWO_PASS && mean == nullptr) ? 0.0f : s2;
        }
        if (more) t = next;
    }
}

// Fused forward for rows wider than a wavefront's registers: `wpr` wavefronts share a row, NCH chunks each
// (the launcher chooses wpr so that every segment starts inside the row), and a block works on
// blockDim/64/wpr rows at a time. The segments' moments meet in LDS, one barrier per exchange: one exchange
// per row for one-pass statistics, two for two-pass; the slots alternate between trips so that a wavefront
// a trip ahead never overwrites sums that another still reads. The row is read from memory once; gamma and
// beta come from cache per chunk; the next trip's rows are loaded before the barrier.
template <typename T, int NCH, int MAXW>
__global__ __launch_bounds__(MAXW * 64) void ln_forward_split_kernel(
    int64_t R, int64_t C, const T* __restrict__ x, int64_t ld, int mode, float inv_h, float eps,
    const T* __restrict__ gamma, const T* __restrict__ beta, T* __restrict__ y, int64_t ldy,
    float* __restrict__ mean_rstd, int wpr) {
    constexpr int V = elem<T>::kVec;
    __shared__ float lds_sums[2][2][MAXW][2];  // [trip parity][exchange][wavefront][moment]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nrg = (int)(blockDim.x >> 6) / wpr;
    const int rg = wave / wpr, seg = wave - rg * wpr;
    const int64_t col0 = (int64_t)seg * (NCH * 64 * V);
    const int64_t Cs = C - col0;  // columns from the segment's start to the end of the row
    x += col0;
    y += col0;
    if (gamma != nullptr) gamma += col0;
    if (beta != nullptr) beta += col0;

    // totals of (a, b) over the wavefronts of this row group, the same in every lane of the group
    auto exchange = [&](int parity, int which, float& a, float& b) {
        if (lane == 0) {
            lds_sums[parity][which][wave][0] = a;
            lds_sums[parity][which][wave][1] = b;
        }
        __syncthreads();
        a = 0.0f;
        b = 0.0f;
        for (int w = 0; w < wpr; ++w) {
            a += lds_sums[parity][which][rg * wpr + w][0];
            b += lds_sums[parity][which][rg * wpr + w][1];
        }
    };

    const int64_t step = (int64_t)gridDim.x * nrg;
    int64_t base = (int64_t)blockIdx.x * nrg;  // the same for every wavefront of the block: uniform trip count
    RowTile<T, NCH, 1> t;
    if (base < R) t.load(x, ld, base + rg, R, Cs, lane);
    for (int trip = 0; base < R; base += step, ++trip) {
        RowTile<T, NCH, 1> next;
        const bool more = base + step < R;
        if (more) next.load(x, ld, base + step + rg, R, Cs, lane);
        const int64_t row = base + rg;
        const bool live = row < R;
        float s1, s2, mean, rstd;
        tile_moments(t, 0, Cs, 0.0f, lane, s1, s2);
        exchange(trip & 1, 0, s1, s2);
        if (mode == CW_LN_TWO_PASS) {
            const float mu = s1 * inv_h;
            float d1, d2;
            tile_moments(t, 0, Cs, mu, lane, d1, d2);
            exchange(trip & 1, 1, d1, d2);
            finish_stats(mode, mu, d2, inv_h, eps, mean, rstd);
        } else {
            finish_stats(mode, s1, s2, inv_h, eps, mean, rstd);
        }
        if (mean_rstd != nullptr && seg == 0 && lane == 0 && live) {
            mean_rstd[2 * row] = mean;
            mean_rstd[2 * row + 1] = rstd;
        }
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const bool ok = chunk_valid<T>(j, lane, Cs);
            const int64_t c0 = ok ? ((int64_t)j * 64 + lane) * V : 0;
            const raw16_t zero = {0u, 0u, 0u, 0u};
            float v[V], g[V], b[V];
            unpack_raw(t.raw[0][j], v, (const T*)nullptr);
            unpack_raw(gamma != nullptr ? load_raw(gamma + c0) : zero, g, (const T*)nullptr);
            unpack_raw(beta != nullptr ? load_raw(beta + c0) : zero, b, (const T*)nullptr);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float xh = (v[e] - mean) * rstd;
                if (gamma != nullptr) xh *= g[e];
                if (beta != nullptr) xh += b[e];
                v[e] = xh;
            }
            if (live && ok) store_raw_stream(y + row * ldy + c0, pack_raw(v, (const T*)nullptr));
        }
        if (more) t = next;
    }
}

template <typename T, int NCH, int NR, bool EXACT>
__global__ __launch_bounds__(kTileWaves * 64) void ln_bwd_dx_tile_kernel(
    int64_t R, int64_t C, const T* __restrict__ dY, int64_t ld_dy, const T* __restrict__ x, int64_t ld_x,
    const float* __restrict__ mean_rstd, const T* __restrict__ gamma, const float* __restrict__ row_sums, float inv_h,
    T* __restrict__ dx, int64_t ld_dx, const FinishCols fin) {
    constexpr int V = elem<T>::kVec;
    if (fin.blocks > 0 && (int)blockIdx.x < fin.blocks) {  // the leading workgroups finish the column sums
        __shared__ float fin_red[kTileWaves * 64];
        finish_cols_block<kTileWaves * 64>(fin, (int)blockIdx.x, fin_red);
        return;
    }
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)((int)blockIdx.x - fin.blocks) * kTileWaves + (threadIdx.x >> 6);
    const int64_t step = (int64_t)((int)gridDim.x - fin.blocks) * kTileWaves * NR;
    raw16_t g_raw[NCH];
    if constexpr (!EXACT) load_param_chunks<T, NCH>(gamma, C, lane, g_raw);
    if constexpr (EXACT) C = (int64_t)NCH * 64 * V;
    for (int64_t row0 = wave * NR; row0 < R; row0 += step) {
        RowTile<T, NCH, NR> tdy, tx;
        tdy.template load<EXACT>(dY, ld_dy, row0, R, C, lane);
        tx.template load<EXACT>(x, ld_x, row0, R, C, lane);
        if constexpr (EXACT) load_param_chunks<T, NCH>(gamma, C, lane, g_raw);
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int64_t row = row0 + r;
            const int64_t row_c = row < R ? row : R - 1;
            const float mean = mean_rstd[2 * row_c], rstd = mean_rstd[2 * row_c + 1];
            const float c1 = row_sums[2 * row_c] * inv_h, c2 = row_sums[2 * row_c + 1] * inv_h;
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                float dy[V], xv[V], g[V];
                unpack_raw(tdy.raw[r][j], dy, (const T*)nullptr);
                unpack_raw(tx.raw[r][j], xv, (const T*)nullptr);
                unpack_raw(g_raw[j], g, (const T*)nullptr);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float xh = (xv[e] - mean) * rstd;
                    const float gg = gamma != nullptr ? dy[e] * g[e] : dy[e];
                    dy[e] = (gg - xh * c2 - c1) * rstd;
                }
                if (row < R && chunk_valid<T>(j, lane, C))
                    store_raw_stream(dx + row * ld_dx + ((int64_t)j * 64 + lane) * V, pack_raw(dy, (const T*)nullptr));
            }
        }
        if constexpr (EXACT) return;
    }
}

// Number of 64-vector chunks a row of C columns spans.
template <typename T>
int64_t row_chunks(int64_t C) {
    return (C + 64 * elem<T>::kVec - 1) / (64 * elem<T>::kVec);
}

// Calls f(NCH, NR) with compile-time constants chosen for `nch` (<= 8) chunks.
template <typename F>
int dispatch_tile(int64_t nch, F&& f) {
    if (nch <= 1) return f(std::integral_constant<int, 1>{}, std::integral_constant<int, kRowsAt1Chunk>{});
    if (nch <= 2) return f(std::integral_constant<int, 2>{}, std::integral_constant<int, kRowsAt2Chunks>{});
    if (nch <= 4) return f(std::integral_constant<int, 4>{}, std::integral_constant<int, kRowsAt4Chunks>{});
    return f(std::integral_constant<int, 8>{}, std::integral_constant<int, 1>{});
}

// Calls f(NCH, NR) for rows of exactly `nch` (1, 2, 4 or 8) chunks with NR = max(1, LOADS / NCH) rows per
// wavefront, LOADS being the 16-byte loads per lane and operand that the kernel wants in flight (measured
// on 16384 x 1024 bf16, one tile per wavefront: 8 for the statistics (7.1 us with 4, 6.9 with 8, 7.4 with 16), 8
// for normalise, 2 for each of dx's two operands).
template <int LOADS, typename F>
int dispatch_exact(int64_t nch, F&& f) {
    if (nch == 1) return f(std::integral_constant<int, 1>{}, std::integral_constant<int, (LOADS >= 4 ? 4 : LOADS)>{});
    if (nch == 2) return f(std::integral_constant<int, 2>{}, std::integral_constant<int, (LOADS / 2 >= 1 ? LOADS / 2 : 1)>{});
    if (nch == 4) return f(std::integral_constant<int, 4>{}, std::integral_constant<int, (LOADS / 4 >= 1 ? LOADS / 4 : 1)>{});
    return f(std::integral_constant<int, 8>{}, std::integral_constant<int, 1>{});
}

template <typename T>
bool exact_chunks(int64_t C, int64_t nch) {
    return (nch == 1 || nch == 2 || nch == 4 || nch == 8) && C == nch * 64 * elem<T>::kVec;
}

// One tile of nr rows per wavefront.
int exact_grid(int64_t R, int nr) {
    const int64_t rows_per_block = (int64_t)kTileWaves * nr;
    return (int)((R + rows_per_block - 1) / rows_per_block);
}

int tile_grid(int64_t R, int nr) {
    const int64_t rows_per_block = (int64_t)kTileWaves * nr;
    const int64_t blocks = (R + rows_per_block - 1) / rows_per_block;
    const int64_t cap = 256 * kTileBlocksPerCu;
    return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

// Backward partials, vector path. Lane `l` owns the columns of chunks
// (j*64 + l)*V .. +V-1, j < NCH, for every row its wavefront visits, so the
// dgamma/dbeta accumulators stay in registers for the whole kernel. A
// wavefront holds NR rows of dY and x at a time.
// FUSE_DX != 0: the rows are complete on this rank (C is the whole hidden size), so the row sums are final and
// dx is written from the registers that hold the row, in the same pass. FUSE_DX == 2: the same rows of dx_add
// (the gradient arriving along a residual branch) are loaded with the tiles and added before the store; an
// instantiation of its own, so that the kernel without an addend carries neither the loads nor a test for them.
template <typename T, int NCH, int NWAVES, int NR, int FUSE_DX>
__global__ __launch_bounds__(NWAVES * 64) void ln_bwd_partials_kernel(
    int64_t R, int64_t C, const T* __restrict__ dY, int64_t ld_dy, const T* __restrict__ x, int64_t ld_x,
    const float* __restrict__ mean_rstd, const T* __restrict__ gamma, float* __restrict__ row_sums,
    float* __restrict__ col_ws, int want_cols, T* __restrict__ dx, int64_t ld_dx, float inv_h,
    const T* __restrict__ dx_add, int64_t ld_add) {
    constexpr int V = elem<T>::kVec;
    extern __shared__ float lds_red[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;

    raw16_t g_raw[NCH];
    load_param_chunks<T, NCH>(gamma, C, lane, g_raw);
    float acc[2 * NCH * V];  // [0, NCH*V): dgamma, [NCH*V, 2*NCH*V): dbeta
#pragma unroll
    for (int i = 0; i < 2 * NCH * V; ++i) acc[i] = 0.0f;

    const int64_t step = (int64_t)gridDim.x * NWAVES * NR;
    for (int64_t row0 = ((int64_t)blockIdx.x * NWAVES + wave) * NR; row0 < R; row0 += step) {
        RowTile<T, NCH, NR> tdy, tx, tadd;
        tdy.load(dY, ld_dy, row0, R, C, lane);
        tx.load(x, ld_x, row0, R, C, lane);
        if constexpr (FUSE_DX == 2) tadd.load(dx_add, ld_add, row0, R, C, lane);
        tdy.zero_dead_rows(row0, R);  // a zero dY row adds nothing to the column sums
#pragma unroll
        for (int r = 0; r < NR; ++r) {            const int64_t row = row0 + r;
            const int64_t row_c = row < R ? row : R - 1;
            const float mean = mean_rstd[2 * row_c];
            const float rstd = mean_rstd[2 * row_c + 1];
            float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                float dy[V], xv[V], g[V];
                unpack_raw(tdy.raw[r][j], dy, (const T*)nullptr);
                unpack_raw(tx.raw[r][j], xv, (const T*)nullptr);
                unpack_raw(g_raw[j], g, (const T*)nullptr);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float d = dy[e];
                    const float xh = (xv[e] - mean) * rstd;
                    const float gd = gamma != nullptr ? d * g[e] : d;
                    s1 += gd;
                    s2 += gd * xh;
                    acc[j * V + e] += d * xh;
                    acc[NCH * V + j * V + e] += d;
                }
            }
            s1 = wave_sum(s1);
            s2 = wave_sum(s2);
            if (lane == 0 && row < R) {
                row_sums[2 * row] = s1;
                row_sums[2 * row + 1] = s2;
            }
            if (FUSE_DX) {
                const float c1 = s1 * inv_h, c2 = s2 * inv_h;
#pragma unroll
                for (int j = 0; j < NCH; ++j) {
                    float dy[V], xv[V], g[V];
                    unpack_raw(tdy.raw[r][j], dy, (const T*)nullptr);
                    unpack_raw(tx.raw[r][j], xv, (const T*)nullptr);
                    unpack_raw(g_raw[j], g, (const T*)nullptr);
#pragma unroll
                    for (int e = 0; e < V; ++e) {
                        const float xh = (xv[e] - mean) * rstd;
                        const float gg = gamma != nullptr ? dy[e] * g[e] : dy[e];
                        dy[e] = (gg - xh * c2 - c1) * rstd;
                    }
                    if constexpr (FUSE_DX == 2) {  // the gradient arriving along the residual branch
                        float av[V];
                        unpack_raw(tadd.raw[r][j], av, (const T*)nullptr);
#pragma unroll
                        for (int e = 0; e < V; ++e) dy[e] += av[e];
                    }
                    if (row < R && chunk_valid<T>(j, lane, C))
                        store_raw_stream(dx + row * ld_dx + ((int64_t)j * 64 + lane) * V, pack_raw(dy, (const T*)nullptr));
                }
            }
        }
    }
    if (!want_cols) return;

    // accumulator i: set i / (NCH*V) (0 = dgamma, 1 = dbeta), chunk j = (i % (NCH*V)) / V, element e = i % V
    float* out = col_ws + (int64_t)blockIdx.x * 2 * C;
    block_flat_reduce<2 * NCH * V, NWAVES>(acc, lds_red, wave, lane, [&](int i, int l, float total) {
        const int set = i / (NCH * V), rem = i - set * (NCH * V);
        const int64_t c = ((int64_t)(rem / V) * 64 + l) * V + (rem % V);
        if (c < C) out[(int64_t)set * C + c] = total;
    });
}

// Backward partials for rows too wide for one wavefront's registers: `wpr` wavefronts share a row, each
// owning a segment of NCH chunks (kSeg columns), and a block works on blockDim/64/wpr rows at a time. The
// segments' row sums meet in LDS (one barrier per trip, slots alternating between trips so that no second
// barrier is needed), after which every wavefront has the row's totals and, with FUSE_DX, writes its
// segment of dx from the registers that hold the row. The next trip's rows are loaded before the barrier.
// The dgamma/dbeta accumulators of the row groups are added through LDS at the end, in a fixed order.
// The launcher chooses wpr so that every segment starts inside the row.
template <typename T, int NCH, int MAXW, int FUSE_DX>
__global__ __launch_bounds__(MAXW * 64, 4) void ln_bwd_split_kernel(
    int64_t R, int64_t C, const T* __restrict__ dY, int64_t ld_dy, const T* __restrict__ x, int64_t ld_x,
    const float* __restrict__ mean_rstd, const T* __restrict__ gamma, float* __restrict__ row_sums,
    float* __restrict__ col_ws, int want_cols, T* __restrict__ dx, int64_t ld_dx, float inv_h, int wpr,
    const T* __restrict__ dx_add, int64_t ld_add) {
    constexpr int V = elem<T>::kVec;
    constexpr int kSeg = NCH * 64 * V;
    constexpr int NA = NCH * V;  // accumulators of one set (dgamma or dbeta) in a lane
    // 16-bit rows and segments of more than two chunks leave no registers for a second pair of tiles
    constexpr bool kPrefetch = sizeof(T) == 4 && NCH <= 2;
    extern __shared__ float lds_red[];
    __shared__ float lds_sums[2][MAXW][2];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nrg = (int)(blockDim.x >> 6) / wpr;
    const int rg = wave / wpr, seg = wave - rg * wpr;
    const int64_t col0 = (int64_t)seg * kSeg;
    const int64_t Cs = C - col0;  // columns from the segment's start to the end of the row
    dY += col0;
    x += col0;
    if (gamma != nullptr) gamma += col0;
    if (FUSE_DX) dx += col0;
    if constexpr (FUSE_DX == 2) dx_add += col0;

    raw16_t g_raw[NCH];
    load_param_chunks<T, NCH>(gamma, Cs, lane, g_raw);
    float acc[2 * NA];  // [0, NA): dgamma, [NA, 2*NA): dbeta
#pragma unroll
    for (int i = 0; i < 2 * NA; ++i) acc[i] = 0.0f;

    const int64_t step = (int64_t)gridDim.x * nrg;
    int64_t base = (int64_t)blockIdx.x * nrg;  // the same for every wavefront of the block: uniform trip count
    RowTile<T, NCH, 1> tdy, tx;
    if (base < R) {
        tdy.load(dY, ld_dy, base + rg, R, Cs, lane);
        tx.load(x, ld_x, base + rg, R, Cs, lane);
    }
    for (int trip = 0; base < R; base += step, ++trip) {
        RowTile<T, NCH, 1> ndy, nx;
        const bool more = kPrefetch && base + step < R;
        if (more) {
            ndy.load(dY, ld_dy, base + step + rg, R, Cs, lane);
            nx.load(x, ld_x, base + step + rg, R, Cs, lane);
        }
        const int64_t row = base + rg;
        const bool live = row < R;
        const int64_t row_c = live ? row : R - 1;
        const float mean = mean_rstd[2 * row_c];
        const float rstd = mean_rstd[2 * row_c + 1];
        // the residual branch's gradient of this row: on its way while the row sums are formed and exchanged
        RowTile<T, NCH, 1> tadd;
        if constexpr (FUSE_DX == 2) tadd.load(dx_add, ld_add, row, R, Cs, lane);
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            float dy[V], xv[V], g[V];
            unpack_raw(tdy.raw[0][j], dy, (const T*)nullptr);
            unpack_raw(tx.raw[0][j], xv, (const T*)nullptr);
            unpack_raw(g_raw[j], g, (const T*)nullptr);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float d = live ? dy[e] : 0.0f;  // a row past the end adds nothing to the column sums
                const float xh = (xv[e] - mean) * rstd;
                const float gd = gamma != nullptr ? d * g[e] : d;
                s1 += gd;
                s2 += gd * xh;
                acc[j * V + e] += d * xh;
                acc[NA + j * V + e] += d;
            }
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        if (lane == 0) {
            lds_sums[trip & 1][wave][0] = s1;
            lds_sums[trip & 1][wave][1] = s2;
        }
        __syncthreads();
        s1 = 0.0f;
        s2 = 0.0f;
        for (int w = 0; w < wpr; ++w) {
            s1 += lds_sums[trip & 1][rg * wpr + w][0];
            s2 += lds_sums[trip & 1][rg * wpr + w][1];
        }
        if (seg == 0 && lane == 0 && live) {
            row_sums[2 * row] = s1;
            row_sums[2 * row + 1] = s2;
        }
        if (FUSE_DX) {
            const float c1 = s1 * inv_h, c2 = s2 * inv_h;
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                float dy[V], xv[V], g[V];
                unpack_raw(tdy.raw[0][j], dy, (const T*)nullptr);
                unpack_raw(tx.raw[0][j], xv, (const T*)nullptr);
                unpack_raw(g_raw[j], g, (const T*)nullptr);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float xh = (xv[e] - mean) * rstd;
                    const float gg = gamma != nullptr ? dy[e] * g[e] : dy[e];
                    dy[e] = (gg - xh * c2 - c1) * rstd;
                }
                if constexpr (FUSE_DX == 2) {  // the gradient arriving along the residual branch
                    float av[V];
                    unpack_raw(tadd.raw[0][j], av, (const T*)nullptr);
#pragma unroll
                    for (int e = 0; e < V; ++e) dy[e] += av[e];
                }
                if (live && chunk_valid<T>(j, lane, Cs))
                    store_raw_stream(dx + row * ld_dx + ((int64_t)j * 64 + lane) * V, pack_raw(dy, (const T*)nullptr));
            }
        }
        if (more) {
            tdy = ndy;
            tx = nx;
        } else if (!kPrefetch && base + step < R) {
            tdy.load(dY, ld_dy, base + step + rg, R, Cs, lane);
            tx.load(x, ld_x, base + step + rg, R, Cs, lane);
        }
    }
    if (!want_cols) return;

    // row groups 1.. hand their accumulators to group 0, one set and one group at a time
    float* red = lds_red + ((int64_t)seg * NA) * 64 + lane;
    for (int set = 0; set < 2; ++set) {
        for (int g = 1; g < nrg; ++g) {
            __syncthreads();
            if (rg == g) {
#pragma unroll
                for (int i = 0; i < NA; ++i) red[i * 64] = acc[set * NA + i];
            }
            __syncthreads();
            if (rg == 0) {
#pragma unroll
                for (int i = 0; i < NA; ++i) acc[set * NA + i] += red[i * 64];
            }
        }
    }
    if (rg != 0) return;
    float* out = col_ws + (int64_t)blockIdx.x * 2 * C + col0;
#pragma unroll
    for (int set = 0; set < 2; ++set)
#pragma unroll
        for (int j = 0; j < NCH; ++j)
            if (chunk_valid<T>(j, lane, Cs)) {
#pragma unroll
                for (int e = 0; e < V; ++e) out[(int64_t)set * C + ((int64_t)j * 64 + lane) * V + e] = acc[set * NA + j * V + e];
            }
}

// Backward partials for shapes the vector kernel does not take (ragged C,
// unaligned rows, very wide rows). Row sums only; the column sums of this
// path come from ln_bwd_cols_generic_kernel.
template <typename T>
__global__ __launch_bounds__(kLnBlock) void ln_bwd_rows_generic_kernel(
    int64_t R, int64_t C, const T* __restrict__ dY, int64_t ld_dy, const T* __restrict__ x, int64_t ld_x,
    const float* __restrict__ mean_rstd, const T* __restrict__ gamma, float* __restrict__ row_sums) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kLnBlock / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (kLnBlock / 64);
    for (int64_t row = wave; row < R; row += nwaves) {
        const float mean = mean_rstd[2 * row];
        const float rstd = mean_rstd[2 * row + 1];
        float s1 = 0.0f, s2 = 0.0f;
        for (int64_t c = lane; c < C; c += 64) {
            const float xh = (load_elem(x + row * ld_x + c) - mean) * rstd;
            const float g = load_elem(dY + row * ld_dy + c) * (gamma != nullptr ? load_elem(gamma + c) : 1.0f);
            s1 += g;
            s2 += g * xh;
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        if (lane == 0) {
            row_sums[2 * row] = s1;
            row_sums[2 * row + 1] = s2;
        }
    }
}

// Column partials of the generic path: thread = one column, block.y = a slab
// of rows. ws[slab][2][C].
template <typename T>
__global__ __launch_bounds__(kLnBlock) void ln_bwd_cols_generic_kernel(
    int64_t R, int64_t C, const T* __restrict__ dY, int64_t ld_dy, const T* __restrict__ x, int64_t ld_x,
    const float* __restrict__ mean_rstd, float* __restrict__ col_ws, int64_t rows_per_slab) {
    const int64_t c = (int64_t)blockIdx.x * kLnBlock + threadIdx.x;
    if (c >= C) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_slab;
    const int64_t r1 = (r0 + rows_per_slab < R) ? r0 + rows_per_slab : R;
    float dg = 0.0f, db = 0.0f;
    for (int64_t row = r0; row < r1; ++row) {
        const float xh = (load_elem(x + row * ld_x + c) - mean_rstd[2 * row]) * mean_rstd[2 * row + 1];
        const float dy = load_elem(dY + row * ld_dy + c);
        dg += dy * xh;
        db += dy;
    }
    col_ws[(int64_t)blockIdx.y * 2 * C + c] = dg;
    col_ws[(int64_t)blockIdx.y * 2 * C + C + c] = db;
}

template <typename T>
__global__ __launch_bounds__(kLnBlock) void ln_bwd_dx_kernel(int64_t R, int64_t C, const T* __restrict__ dY,
                                                             int64_t ld_dy, const T* __restrict__ x, int64_t ld_x,
                                                             const float* __restrict__ mean_rstd,
                                                             const T* __restrict__ gamma,
                                                             const float* __restrict__ row_sums, float inv_h,
                                                             T* __restrict__ dx, int64_t ld_dx, int vec_ok,
                                                             const FinishCols fin) {
    constexpr int V = elem<T>::kVec;
    if (fin.blocks > 0 && (int)blockIdx.x < fin.blocks) {  // the leading workgroups finish the column sums
        __shared__ float fin_red[kLnBlock];
        finish_cols_block<kLnBlock>(fin, (int)blockIdx.x, fin_red);
        return;
    }
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)((int)blockIdx.x - fin.blocks) * (kLnBlock / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)((int)gridDim.x - fin.blocks) * (kLnBlock / 64);
    for (int64_t row = wave; row < R; row += nwaves) {
        const float mean = mean_rstd[2 * row];
        const float rstd = mean_rstd[2 * row + 1];
        const float c1 = row_sums[2 * row] * inv_h;
        const float c2 = row_sums[2 * row + 1] * inv_h;
        const T* dyr = dY + row * ld_dy;
        const T* xr = x + row * ld_x;
        T* dxr = dx + row * ld_dx;
        if (vec_ok) {
            const int64_t nvec = C / V;
            for (int64_t i = lane; i < nvec; i += 64) {
                float dy[V], xv[V], g[V];
                load_vec(dyr + i * V, dy);
                load_vec(xr + i * V, xv);
                if (gamma != nullptr) load_vec(gamma + i * V, g);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float xh = (xv[e] - mean) * rstd;
                    const float gg = gamma != nullptr ? dy[e] * g[e] : dy[e];
                    dy[e] = (gg - xh * c2 - c1) * rstd;
                }
                store_vec(dxr + i * V, dy);
            }
            for (int64_t c = nvec * V + lane; c < C; c += 64) {
                const float xh = (load_elem(xr + c) - mean) * rstd;
                const float gg = load_elem(dyr + c) * (gamma != nullptr ? load_elem(gamma + c) : 1.0f);
                store_elem(dxr + c, (gg - xh * c2 - c1) * rstd);
            }
        } else {
            for (int64_t c = lane; c < C; c += 64) {
                const float xh = (load_elem(xr + c) - mean) * rstd;
                const float gg = load_elem(dyr + c) * (gamma != nullptr ? load_elem(gamma + c) : 1.0f);
                store_elem(dxr + c, (gg - xh * c2 - c1) * rstd);
            }
        }
    }
}


int ln_grid(int64_t R) {
    const int64_t blocks = (R + (kLnBlock / 64) - 1) / (kLnBlock / 64);
    const int64_t cap = 256 * 8;  // 8 resident blocks of 4 wavefronts per CU
    return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

template <typename T>
bool rows_vec_ok(const void* p, int64_t ld) {
    return aligned16(p) && (ld % elem<T>::kVec) == 0;
}

// Chunks per wavefront and wavefronts per block of the forward-side split kernels (statistics, fused
// forward) for rows of more than 8 chunks; blocks of as many wavefronts as a row needs, up to 16, for the
// widest rows.
constexpr int kFwdSplitChunks = 4;
constexpr int kFwdSplitBlockWaves = 8;

struct FwdSplitShape {
    int wpr, nrg;
    int64_t blocks;
    bool takes, wide;
};

FwdSplitShape fwd_split_shape(int64_t R, int64_t nch) {
    FwdSplitShape sh;
    sh.wpr = (int)((nch + kFwdSplitChunks - 1) / kFwdSplitChunks);
    sh.takes = nch > 8 && sh.wpr <= 16;
    sh.nrg = sh.wpr >= kFwdSplitBlockWaves ? 1 : kFwdSplitBlockWaves / sh.wpr;
    sh.wide = sh.wpr * sh.nrg > kFwdSplitBlockWaves;
    sh.blocks = (R + sh.nrg - 1) / sh.nrg;
    const int64_t cap = sh.takes ? 256 * (16 / (sh.wpr * sh.nrg)) : 1;  // 16 wavefronts per CU
    if (sh.blocks > cap) sh.blocks = cap;
    if (sh.blocks < 1) sh.blocks = 1;
    return sh;
}

template <typename T>
int stats_impl(int64_t R, int64_t C, const void* x, int64_t ld, int mode, const float* mean, float* stats,
               hipStream_t s) {
    const int vec_ok = rows_vec_ok<T>(x, ld);
    const int64_t nch = row_chunks<T>(C);
    if (vec_ok && exact_chunks<T>(C, nch) && R <= (int64_t)1 << 30) {
        return dispatch_exact<8>(nch, [&](auto nch_c, auto nr_c) {
            constexpr int NCH = decltype(nch_c)::value, NR = decltype(nr_c)::value;
            hipLaunchKernelGGL((ln_stats_tile_kernel<T, NCH, NR, true>), dim3(exact_grid(R, NR)), dim3(kTileWaves * 64),
                               0, s, R, C, (const T*)x, ld, mode, mean, stats);
            return check_launch("ln_stats_tile_kernel");
        });
    }
    if (vec_ok && (C % elem<T>::kVec) == 0 && nch <= 8) {
        return dispatch_tile(nch, [&](auto nch_c, auto nr_c) {
            constexpr int NCH = decltype(nch_c)::value, NR = decltype(nr_c)::value;
            hipLaunchKernelGGL((ln_stats_tile_kernel<T, NCH, NR, false>), dim3(tile_grid(R, NR)), dim3(kTileWaves * 64),
                               0, s, R, C, (const T*)x, ld, mode, mean, stats);
            return check_launch("ln_stats_tile_kernel");
        });
    }
    const FwdSplitShape sh = fwd_split_shape(R, nch);
    if (vec_ok && (C % elem<T>::kVec) == 0 && sh.takes) {
        const dim3 grid((unsigned)sh.blocks), block(sh.wpr * sh.nrg * 64);
        if (sh.wide)
            hipLaunchKernelGGL((ln_stats_split_kernel<T, kFwdSplitChunks, 16>), grid, block, 0, s, R, C, (const T*)x,
                               ld, mode, mean, stats, sh.wpr);
        else
            hipLaunchKernelGGL((ln_stats_split_kernel<T, kFwdSplitChunks, kFwdSplitBlockWaves>), grid, block, 0, s,
                               R, C, (const T*)x, ld, mode, mean, stats, sh.wpr);
        return check_launch("ln_stats_split_kernel");
    }
    hipLaunchKernelGGL(ln_stats_kernel<T>, dim3(ln_grid(R)), dim3(kLnBlock), 0, s, R, C, (const T*)x, ld, mode,
                       mean, stats, vec_ok);
    return check_launch("ln_stats_kernel");
}

template <typename T, bool FUSED>
int normalize_impl(int64_t R, int64_t C, const void* x, int64_t ld, const float* stats, int mode, int64_t H,
                   float eps, const void* gamma, const void* beta, void* y, int64_t ldy, float* mean_rstd,
                   hipStream_t s) {
    const int vec_ok = rows_vec_ok<T>(x, ld) && rows_vec_ok<T>(y, ldy) && (gamma == nullptr || aligned16(gamma)) &&
                       (beta == nullptr || aligned16(beta));
    const int64_t nch = row_chunks<T>(C);
    if (vec_ok && exact_chunks<T>(C, nch) && R <= (int64_t)1 << 30) {
        // rows per wavefront, by measurement (one tile per wavefront, 16-bit rows): four rows of one chunk (12.8 us
        // on 32768 x 512 against 14.8 with two and 14.5 with eight), two rows of two chunks (16384 x 1024: 11.9
        // against 12.8 us with four; fused 12.4 against 14.6), two rows of four chunks (8192 x 2048 fused: 13.6
        // against 15.5 us with one)
        return dispatch_exact<8>(nch, [&](auto nch_c, auto nr_c) {
            constexpr int NCH = decltype(nch_c)::value;
            constexpr int NR = NCH == 2 ? 2 : decltype(nr_c)::value;
            hipLaunchKernelGGL((ln_normalize_tile_kernel<T, NCH, NR, FUSED, true>), dim3(exact_grid(R, NR)),
                               dim3(kTileWaves * 64), 0, s, R, C, (const T*)x, ld, stats, mode, 1.0f / (float)H, eps,
                               (const T*)gamma, (const T*)beta, (T*)y, ldy, mean_rstd);
            return check_launch("ln_normalize_tile_kernel");
        });
    }
    if (vec_ok && (C % elem<T>::kVec) == 0 && nch <= 8) {
        return dispatch_tile(nch, [&](auto nch_c, auto nr_c) {
            constexpr int NCH = decltype(nch_c)::value, NR = decltype(nr_c)::value;
            hipLaunchKernelGGL((ln_normalize_tile_kernel<T, NCH, NR, FUSED, false>), dim3(tile_grid(R, NR)),
                               dim3(kTileWaves * 64), 0, s, R, C, (const T*)x, ld, stats, mode, 1.0f / (float)H, eps,
                               (const T*)gamma, (const T*)beta, (T*)y, ldy, mean_rstd);
            return check_launch("ln_normalize_tile_kernel");
        });
    }
    if constexpr (FUSED) {
        const FwdSplitShape sh = fwd_split_shape(R, nch);
        if (vec_ok && (C % elem<T>::kVec) == 0 && sh.takes) {
            const dim3 grid((unsigned)sh.blocks), block(sh.wpr * sh.nrg * 64);
            if (sh.wide)
                hipLaunchKernelGGL((ln_forward_split_kernel<T, kFwdSplitChunks, 16>), grid, block, 0, s, R, C,
                                   (const T*)x, ld, mode, 1.0f / (float)H, eps, (const T*)gamma, (const T*)beta,
                                   (T*)y, ldy, mean_rstd, sh.wpr);
            else
                hipLaunchKernelGGL((ln_forward_split_kernel<T, kFwdSplitChunks, kFwdSplitBlockWaves>), grid, block, 0,
                                   s, R, C, (const T*)x, ld, mode, 1.0f / (float)H, eps, (const T*)gamma,
                                   (const T*)beta, (T*)y, ldy, mean_rstd, sh.wpr);
            return check_launch("ln_forward_split_kernel");
        }
    }
    hipLaunchKernelGGL((ln_normalize_kernel<T, FUSED>), dim3(ln_grid(R)), dim3(kLnBlock), 0, s, R, C, (const T*)x,
                       ld, stats, mode, 1.0f / (float)H, eps, (const T*)gamma, (const T*)beta, (T*)y, ldy,
                       mean_rstd, vec_ok);
    return check_launch("ln_normalize_kernel");
}

// The gradient that reaches x along a residual branch, added to dx by the kernels that write dx from the row they
// hold (p == nullptr: none).
struct DxAdd {
    const void* p = nullptr;
    int64_t ld = 0;
};

// Number of blocks (= column partials) of the vector backward kernel.
int64_t bwd_blocks(int64_t R, int nwaves) {
    int64_t nb = (R + nwaves - 1) / nwaves;
    if (nb > 256) nb = 256;
    if (nb < 1) nb = 1;
    return nb;
}

template <typename T, int NCH, int NWAVES, int NR, int FUSE_DX>
int bwd_partials_launch_as(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                           const float* mean_rstd, const void* gamma, float* row_sums, float* ws, int want_cols,
                           void* dx, int64_t ld_dx, hipStream_t s, DxAdd add = {}) {
    constexpr int V = elem<T>::kVec;
    const int64_t nb = bwd_blocks(R, NWAVES * NR);
    const size_t lds = flat_reduce_lds_bytes(2 * NCH * V, NWAVES);
    auto kern = ln_bwd_partials_kernel<T, NCH, NWAVES, NR, FUSE_DX>;
    if (lds > 48 * 1024) {
        if (const int lrc = ensure_dynamic_lds((const void*)kern, (int)((int)lds), "ln_bwd_partials"); lrc != CW_OK) return lrc;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nb), dim3(NWAVES * 64), lds, s, R, C, (const T*)dY, ld_dy, (const T*)x,
                       ld_x, mean_rstd, (const T*)gamma, row_sums, ws, want_cols, (T*)dx, ld_dx, 1.0f / (float)C,
                       (const T*)add.p, add.ld);
    return check_launch("ln_bwd_partials_kernel");
}

template <typename T, int NCH, int NWAVES, int NR>
int bwd_partials_launch(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                        const float* mean_rstd, const void* gamma, float* row_sums, float* ws, int want_cols,
                        void* dx, int64_t ld_dx, hipStream_t s, DxAdd add = {}) {
    if (dx != nullptr && add.p != nullptr)
        return bwd_partials_launch_as<T, NCH, NWAVES, NR, 2>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws,
                                                             want_cols, dx, ld_dx, s, add);
    if (dx != nullptr)
        return bwd_partials_launch_as<T, NCH, NWAVES, NR, 1>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws,
                                                             want_cols, dx, ld_dx, s);
    return bwd_partials_launch_as<T, NCH, NWAVES, NR, 0>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws,
                                                         want_cols, nullptr, 0, s);
}

// Rows of more than kSplitMinChunks chunks go to the split kernel: kSplitChunks chunks per wavefront (three
// or four for fp32 rows too wide for 16 such wavefronts), blocks of kSplitBlockWaves wavefronts (of as many
// as a row needs, up to 16, for the widest rows).
constexpr int kSplitChunks = 2;
constexpr int kSplitBlockWaves = 8;
constexpr int64_t kSplitMaxBlocks = 512;

constexpr int kSplitMinChunks = 4;

// chunks per wavefront of the split kernel for rows of nch chunks, 0 if it does not take them
template <typename T>
int split_chunks(int64_t nch) {
    if (nch <= kSplitMinChunks) return 0;
    if ((nch + kSplitChunks - 1) / kSplitChunks <= 16) return kSplitChunks;
    if (sizeof(T) == 4 && (nch + 2) / 3 <= 16) return 3;
    if (sizeof(T) == 4 && (nch + 3) / 4 <= 16) return 4;
    return 0;
}

struct SplitShape {
    int chunks, wpr, nrg;
    int64_t blocks;
};

SplitShape split_shape(int64_t R, int64_t nch, int chunks) {
    SplitShape sh;
    sh.chunks = chunks;
    sh.wpr = (int)((nch + chunks - 1) / chunks);
    sh.nrg = sh.wpr >= kSplitBlockWaves ? 1 : kSplitBlockWaves / sh.wpr;
    sh.blocks = (R + sh.nrg - 1) / sh.nrg;
    const int64_t cap = 256 * (16 / (sh.wpr * sh.nrg));  // 16 wavefronts per CU; at most kSplitMaxBlocks
    if (sh.blocks > cap) sh.blocks = cap;
    if (sh.blocks > kSplitMaxBlocks) sh.blocks = kSplitMaxBlocks;
    if (sh.blocks < 1) sh.blocks = 1;
    return sh;
}

template <typename T, int NCH, int MAXW, int FUSE_DX>
int bwd_split_launch_as(const SplitShape& sh, int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x,
                        int64_t ld_x, const float* mean_rstd, const void* gamma, float* row_sums, float* ws,
                        int want_cols, void* dx, int64_t ld_dx, hipStream_t s, DxAdd add = {}) {
    constexpr int V = elem<T>::kVec;
    const size_t lds = sh.nrg > 1 ? (size_t)sh.wpr * NCH * V * 64 * sizeof(float) : 0;
    hipLaunchKernelGGL((ln_bwd_split_kernel<T, NCH, MAXW, FUSE_DX>), dim3((unsigned)sh.blocks),
                       dim3(sh.wpr * sh.nrg * 64), lds, s, R, C, (const T*)dY, ld_dy, (const T*)x, ld_x, mean_rstd,
                       (const T*)gamma, row_sums, ws, want_cols, (T*)dx, ld_dx, 1.0f / (float)C, sh.wpr,
                       (const T*)(FUSE_DX == 2 ? add.p : nullptr), add.ld);
    return check_launch("ln_bwd_split_kernel");
}

template <typename T>
int bwd_split_launch(const SplitShape& sh, int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x,
                     int64_t ld_x, const float* mean_rstd, const void* gamma, float* row_sums, float* ws,
                     int want_cols, void* dx, int64_t ld_dx, hipStream_t s, DxAdd add = {}) {
    const bool wide = sh.wpr * sh.nrg > kSplitBlockWaves;
#define CW_SPLIT(NCH, MAXW, FUSE)                                                                               \
    bwd_split_launch_as<T, NCH, MAXW, FUSE>(sh, R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws, want_cols, \
                                            dx, ld_dx, s, add)
#define CW_SPLIT_MODE(NCH, MAXW) \
    (dx == nullptr ? CW_SPLIT(NCH, MAXW, 0) : (add.p != nullptr ? CW_SPLIT(NCH, MAXW, 2) : CW_SPLIT(NCH, MAXW, 1)))
    if constexpr (sizeof(T) == 4) {
        // three or four chunks: only rows that need more than eight such wavefronts, in one row group
        if (sh.chunks == 3) return CW_SPLIT_MODE(3, 16);
        if (sh.chunks == 4) return CW_SPLIT_MODE(4, 16);
    }
    return wide ? CW_SPLIT_MODE(kSplitChunks, 16) : CW_SPLIT_MODE(kSplitChunks, kSplitBlockWaves);
#undef CW_SPLIT_MODE
#undef CW_SPLIT
}

constexpr int64_t kGenericSlabRows = 64;

// dx != nullptr asks for the fused backward (C is the whole hidden size); *dx_done tells whether the
// kernel chosen wrote dx or the caller still has to run the dx kernel.
template <typename T>
int bwd_partials_impl(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                      const float* mean_rstd, const void* gamma, float* row_sums, void* dgamma, void* dbeta,
                      int param_dtype, void* workspace, int64_t workspace_bytes, hipStream_t s, void* dx = nullptr,
                      int64_t ld_dx = 0, bool* dx_done = nullptr, int64_t* open_parts = nullptr, DxAdd add = {}) {
    // open_parts: the column partials are left in the workspace, their count is reported, and whoever launches next
    // on the stream adds them up (bwd_dx_impl with a FinishCols)
    constexpr int V = elem<T>::kVec;
    if (dx_done != nullptr) *dx_done = false;
    const int want_cols = (dgamma != nullptr || dbeta != nullptr || open_parts != nullptr) ? 1 : 0;
    const bool vec = rows_vec_ok<T>(dY, ld_dy) && rows_vec_ok<T>(x, ld_x) && (gamma == nullptr || aligned16(gamma)) &&
                     (C % V) == 0 && (add.p == nullptr || rows_vec_ok<T>(add.p, add.ld));
    const int64_t nch = (C + 64 * V - 1) / (64 * V);
    int64_t nparts = 0;
    int rc;
    if (vec && split_chunks<T>(nch) != 0) {
        const SplitShape sh = split_shape(R, nch, split_chunks<T>(nch));
        nparts = sh.blocks;
        if (want_cols && workspace_bytes < nparts * 2 * C * (int64_t)sizeof(float))
            return fail(CW_ERR_INVALID, "cw_ln_bwd_partials: workspace too small (%lld bytes)", (long long)workspace_bytes);
        void* fdx = (dx != nullptr && rows_vec_ok<T>(dx, ld_dx)) ? dx : nullptr;
        rc = bwd_split_launch<T>(sh, R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, (float*)workspace, want_cols,
                                 fdx, ld_dx, s, add);
        if (rc != CW_OK) return rc;
        if (dx_done != nullptr) *dx_done = fdx != nullptr;
    } else if (vec && nch <= 8) {
        const int rows_per_trip = nch <= 1 ? 16 * 2 : (nch <= 2 ? 16 : (nch <= 4 ? 8 : 4));
        nparts = bwd_blocks(R, rows_per_trip);
        if (want_cols && workspace_bytes < nparts * 2 * C * (int64_t)sizeof(float))
            return fail(CW_ERR_INVALID, "cw_ln_bwd_partials: workspace too small (%lld bytes)", (long long)workspace_bytes);
        float* ws = (float*)workspace;
        void* fdx = (dx != nullptr && rows_vec_ok<T>(dx, ld_dx)) ? dx : nullptr;
        if (nch <= 1)
            rc = bwd_partials_launch<T, 1, 16, 2>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws, want_cols, fdx, ld_dx, s, add);
        else if (nch <= 2)
            rc = bwd_partials_launch<T, 2, 16, 1>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws, want_cols, fdx, ld_dx, s, add);
        else if (nch <= 4)
            rc = bwd_partials_launch<T, 4, 8, 1>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws, want_cols, fdx, ld_dx, s, add);
        else
            rc = bwd_partials_launch<T, 8, 4, 1>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, ws, want_cols, fdx, ld_dx, s, add);
        if (rc != CW_OK) return rc;
        if (dx_done != nullptr) *dx_done = fdx != nullptr;
    } else {
        nparts = (R + kGenericSlabRows - 1) / kGenericSlabRows;
        if (want_cols && workspace_bytes < nparts * 2 * C * (int64_t)sizeof(float))  // before anything is launched
            return fail(CW_ERR_INVALID, "cw_ln_bwd_partials: workspace too small (%lld bytes)", (long long)workspace_bytes);
        hipLaunchKernelGGL(ln_bwd_rows_generic_kernel<T>, dim3(ln_grid(R)), dim3(kLnBlock), 0, s, R, C,
                           (const T*)dY, ld_dy, (const T*)x, ld_x, mean_rstd, (const T*)gamma, row_sums);
        rc = check_launch("ln_bwd_rows_generic_kernel");
        if (rc != CW_OK) return rc;
        if (want_cols) {
            dim3 grid((unsigned)((C + kLnBlock - 1) / kLnBlock), (unsigned)nparts);
            hipLaunchKernelGGL(ln_bwd_cols_generic_kernel<T>, grid, dim3(kLnBlock), 0, s, R, C, (const T*)dY, ld_dy,
                               (const T*)x, ld_x, mean_rstd, (float*)workspace, kGenericSlabRows);
            rc = check_launch("ln_bwd_cols_generic_kernel");
            if (rc != CW_OK) return rc;
        }
    }
    if (open_parts != nullptr) {
        *open_parts = nparts;
        return rc;
    }
    if (want_cols) {
        // ws is [nparts][2][C]: dgamma partials are rows 2p, dbeta partials rows 2p+1.
        rc = finalize_col_partials((const float*)workspace, nparts, 2 * C, 2, C, dgamma, dbeta, param_dtype, s);
    }
    return rc;
}

template <typename T>
int bwd_dx_impl(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                const float* mean_rstd, const void* gamma, const float* row_sums, int64_t H, void* dx, int64_t ld_dx,
                hipStream_t s, const FinishCols* finish = nullptr) {
    const int vec_ok = rows_vec_ok<T>(dY, ld_dy) && rows_vec_ok<T>(x, ld_x) && rows_vec_ok<T>(dx, ld_dx) &&
                       (gamma == nullptr || aligned16(gamma));
    const FinishCols fin = finish != nullptr ? *finish : FinishCols{};
    const unsigned fb = (unsigned)fin.blocks;
    const int64_t nch = row_chunks<T>(C);
    // rows of more than 4 chunks are faster on the looping kernel (the 8-chunk tile needs 160-240 registers)
    if (vec_ok && exact_chunks<T>(C, nch) && nch <= 4 && R <= (int64_t)1 << 30) {
        return dispatch_exact<2>(nch, [&](auto nch_c, auto nr_c) {
            constexpr int NCH = decltype(nch_c)::value, NR = decltype(nr_c)::value;
            hipLaunchKernelGGL((ln_bwd_dx_tile_kernel<T, NCH, NR, true>), dim3(exact_grid(R, NR) + fb), dim3(kTileWaves * 64),
                               0, s, R, C, (const T*)dY, ld_dy, (const T*)x, ld_x, mean_rstd, (const T*)gamma, row_sums,
                               1.0f / (float)H, (T*)dx, ld_dx, fin);
            return check_launch("ln_bwd_dx_tile_kernel");
        });
    }
    if (vec_ok && (C % elem<T>::kVec) == 0 && nch <= 4) {
        return dispatch_tile(nch, [&](auto nch_c, auto nr_c) {
            constexpr int NCH = decltype(nch_c)::value, NR = decltype(nr_c)::value;
            hipLaunchKernelGGL((ln_bwd_dx_tile_kernel<T, NCH, NR, false>), dim3(tile_grid(R, NR) + fb), dim3(kTileWaves * 64),
                               0, s, R, C, (const T*)dY, ld_dy, (const T*)x, ld_x, mean_rstd, (const T*)gamma, row_sums,
                               1.0f / (float)H, (T*)dx, ld_dx, fin);
            return check_launch("ln_bwd_dx_tile_kernel");
        });
    }
    hipLaunchKernelGGL(ln_bwd_dx_kernel<T>, dim3(ln_grid(R) + fb), dim3(kLnBlock), 0, s, R, C, (const T*)dY, ld_dy,
                       (const T*)x, ld_x, mean_rstd, (const T*)gamma, row_sums, 1.0f / (float)H, (T*)dx, ld_dx,
                       vec_ok, fin);
    return check_launch("ln_bwd_dx_kernel");
}

int check_rc(const char* fn, int64_t R, int64_t C, int io_dtype) {
    if (R < 0 || C <= 0) return fail(CW_ERR_INVALID, "%s: bad shape R=%lld C=%lld", fn, (long long)R, (long long)C);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "%s: bad io_dtype %d", fn, io_dtype);
    return CW_OK;
}

}  // namespace

// Upper bound of the column-partial scratch cw_ln_bwd_partials can need.
int64_t ln_bwd_workspace_bytes(int64_t R, int64_t C) {
    int64_t parts = (R + kGenericSlabRows - 1) / kGenericSlabRows;
    if (parts < kSplitMaxBlocks) parts = kSplitMaxBlocks;
    return parts * 2 * C * (int64_t)sizeof(float);
}

}  // namespace cw

using namespace cw;

extern "C" int cw_ln_partial_stats(int64_t R, int64_t C, const void* x, int64_t ld, int mode, const float* mean,
                                   float* stats, int io_dtype, void* stream) {
    int rc = check_rc("cw_ln_partial_stats", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (mode != CW_LN_ONE_PASS && mode != CW_LN_TWO_PASS) return fail(CW_ERR_INVALID, "cw_ln_partial_stats: bad mode %d", mode);
    if (R == 0) return CW_OK;
    if (x == nullptr || stats == nullptr || ld < C) return fail(CW_ERR_INVALID, "cw_ln_partial_stats: null pointer or ld < C");
    if (const int drc = require_gfx950("cw_ln_partial_stats"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return stats_impl<std::remove_pointer_t<decltype(tag)>>(R, C, x, ld, mode, mean, stats, s);
    });
}

extern "C" int cw_ln_normalize(int64_t R, int64_t C, const void* x, int64_t ld, const float* stats, int mode,
                               int64_t H, float eps, const void* gamma, const void* beta, void* y, int64_t ldy,
                               float* mean_rstd, int io_dtype, void* stream) {
    int rc = check_rc("cw_ln_normalize", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (mode != CW_LN_ONE_PASS && mode != CW_LN_TWO_PASS) return fail(CW_ERR_INVALID, "cw_ln_normalize: bad mode %d", mode);
    if (H < C) return fail(CW_ERR_INVALID, "cw_ln_normalize: hidden size H=%lld smaller than local C=%lld", (long long)H, (long long)C);
    if (R == 0) return CW_OK;
    if (x == nullptr || y == nullptr || stats == nullptr || ld < C || ldy < C)
        return fail(CW_ERR_INVALID, "cw_ln_normalize: null pointer or leading dimension < C");
    if (const int drc = require_gfx950("cw_ln_normalize"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return normalize_impl<std::remove_pointer_t<decltype(tag)>, false>(R, C, x, ld, stats, mode, H, eps, gamma, beta,
                                                                           y, ldy, mean_rstd, s);
    });
}

extern "C" int cw_ln_forward_fused(int64_t R, int64_t C, const void* x, int64_t ld, int mode, float eps,
                                   const void* gamma, const void* beta, void* y, int64_t ldy, float* mean_rstd,
                                   int io_dtype, void* stream) {
    int rc = check_rc("cw_ln_forward_fused", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (mode != CW_LN_ONE_PASS && mode != CW_LN_TWO_PASS) return fail(CW_ERR_INVALID, "cw_ln_forward_fused: bad mode %d", mode);
    if (R == 0) return CW_OK;
    if (x == nullptr || y == nullptr || ld < C || ldy < C)
        return fail(CW_ERR_INVALID, "cw_ln_forward_fused: null pointer or leading dimension < C");
    if (const int drc = require_gfx950("cw_ln_forward_fused"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return normalize_impl<std::remove_pointer_t<decltype(tag)>, true>(R, C, x, ld, nullptr, mode, C, eps, gamma, beta,
                                                                          y, ldy, mean_rstd, s);
    });
}

extern "C" int cw_ln_bwd_partials(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                                  const float* mean_rstd, const void* gamma, float* row_sums, void* dgamma,
                                  void* dbeta, int param_dtype, void* workspace, int64_t workspace_bytes, int io_dtype,
                                  void* stream) {
    int rc = check_rc("cw_ln_bwd_partials", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (dgamma != nullptr && !col_out_dtype_ok(param_dtype))
        return fail(CW_ERR_INVALID, "cw_ln_bwd_partials: bad param_dtype %d", param_dtype);
    if ((dgamma == nullptr) != (dbeta == nullptr))
        return fail(CW_ERR_INVALID, "cw_ln_bwd_partials: dgamma and dbeta must both be given or both be NULL");
    if (R == 0) return CW_OK;
    if (dY == nullptr || x == nullptr || mean_rstd == nullptr || row_sums == nullptr || ld_dy < C || ld_x < C)
        return fail(CW_ERR_INVALID, "cw_ln_bwd_partials: null pointer or leading dimension < C");
    if (dgamma != nullptr && workspace == nullptr) return fail(CW_ERR_INVALID, "cw_ln_bwd_partials: workspace is NULL");
    if (const int drc = require_gfx950("cw_ln_bwd_partials"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return bwd_partials_impl<std::remove_pointer_t<decltype(tag)>>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums,
                                                                       dgamma, dbeta, param_dtype, workspace,
                                                                       workspace_bytes, s);
    });
}

namespace cw {
namespace {
template <typename T>
int backward_fused_impl(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                        const float* mean_rstd, const void* gamma, float* row_sums, void* dx, int64_t ld_dx,
                        void* dgamma, void* dbeta, int param_dtype, void* workspace, int64_t workspace_bytes,
                        hipStream_t s, DxAdd add) {
    // the residual gradient rides only the kernels that write dx from the row they hold: shapes that take the
    // two-kernel path are refused before anything is launched (the caller adds it itself)
    if (add.p != nullptr) {
        constexpr int V = elem<T>::kVec;
        const int64_t nch = (C + 64 * V - 1) / (64 * V);
        const bool one_pass = rows_vec_ok<T>(dY, ld_dy) && rows_vec_ok<T>(x, ld_x) && rows_vec_ok<T>(dx, ld_dx) &&
                              rows_vec_ok<T>(add.p, add.ld) && (gamma == nullptr || aligned16(gamma)) && (C % V) == 0 &&
                              (split_chunks<T>(nch) != 0 || nch <= 8);
        if (!one_pass)
            return fail(CW_ERR_UNSUPPORTED, "cw_ln_backward_fused: dx_addend is taken by the one-pass kernels only (16-byte "
                                            "aligned rows, C a multiple of the 16-byte vector, rows within their width)");
    }
    bool dx_done = false;
    int rc = bwd_partials_impl<T>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, dgamma, dbeta, param_dtype,
                                  workspace, workspace_bytes, s, dx, ld_dx, &dx_done, nullptr, add);
    if (rc != CW_OK || dx_done) return rc;
    if (add.p != nullptr)  // the check above and the choice of kernel have come apart: never drop the addend silently
        return fail(CW_ERR_UNSUPPORTED, "cw_ln_backward_fused: this shape took the two-kernel path, which does not add dx_addend");
    return bwd_dx_impl<T>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, C, dx, ld_dx, s);
}
}  // namespace
}  // namespace cw

extern "C" int cw_ln_backward_fused(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                                    const float* mean_rstd, const void* gamma, float* row_sums, void* dx,
                                    int64_t ld_dx, const void* dx_addend, int64_t ld_add, void* dgamma, void* dbeta,
                                    int param_dtype, void* workspace, int64_t workspace_bytes, int io_dtype,
                                    void* stream) {
    int rc = check_rc("cw_ln_backward_fused", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (dx_addend != nullptr && ld_add < C)
        return fail(CW_ERR_INVALID, "cw_ln_backward_fused: ld_add < C");
    if (dgamma != nullptr && !col_out_dtype_ok(param_dtype))
        return fail(CW_ERR_INVALID, "cw_ln_backward_fused: bad param_dtype %d", param_dtype);
    if ((dgamma == nullptr) != (dbeta == nullptr))
        return fail(CW_ERR_INVALID, "cw_ln_backward_fused: dgamma and dbeta must both be given or both be NULL");
    if (R == 0) return CW_OK;
    if (dY == nullptr || x == nullptr || mean_rstd == nullptr || row_sums == nullptr || dx == nullptr || ld_dy < C ||
        ld_x < C || ld_dx < C)
        return fail(CW_ERR_INVALID, "cw_ln_backward_fused: null pointer or leading dimension < C");
    if (dgamma != nullptr && workspace == nullptr) return fail(CW_ERR_INVALID, "cw_ln_backward_fused: workspace is NULL");
    if (const int drc = require_gfx950("cw_ln_backward_fused"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    DxAdd add;
    add.p = R > 0 ? dx_addend : nullptr;
    add.ld = ld_add;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return backward_fused_impl<std::remove_pointer_t<decltype(tag)>>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums,
                                                                         dx, ld_dx, dgamma, dbeta, param_dtype,
                                                                         workspace, workspace_bytes, s, add);
    });
}

extern "C" int cw_ln_bwd_dx(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                            const float* mean_rstd, const void* gamma, const float* row_sums, int64_t H, void* dx,
                            int64_t ld_dx, int io_dtype, void* stream) {
    int rc = check_rc("cw_ln_bwd_dx", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (H < C) return fail(CW_ERR_INVALID, "cw_ln_bwd_dx: hidden size H=%lld smaller than local C=%lld", (long long)H, (long long)C);
    if (R == 0) return CW_OK;
    if (dY == nullptr || x == nullptr || mean_rstd == nullptr || row_sums == nullptr || dx == nullptr || ld_dy < C ||
        ld_x < C || ld_dx < C)
        return fail(CW_ERR_INVALID, "cw_ln_bwd_dx: null pointer or leading dimension < C");
    if (const int drc = require_gfx950("cw_ln_bwd_dx"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return bwd_dx_impl<std::remove_pointer_t<decltype(tag)>>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, H, dx,
                                                                 ld_dx, s);
    });
}

extern "C" int cw_ln_bwd_partials_open(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                                       const float* mean_rstd, const void* gamma, float* row_sums, void* workspace,
                                       int64_t workspace_bytes, int64_t* n_parts, int io_dtype, void* stream) {
    int rc = check_rc("cw_ln_bwd_partials_open", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (n_parts == nullptr) return fail(CW_ERR_INVALID, "cw_ln_bwd_partials_open: n_parts is NULL");
    *n_parts = 0;
    if (R == 0) return CW_OK;
    if (dY == nullptr || x == nullptr || mean_rstd == nullptr || row_sums == nullptr || workspace == nullptr || ld_dy < C ||
        ld_x < C)
        return fail(CW_ERR_INVALID, "cw_ln_bwd_partials_open: null pointer or leading dimension < C");
    if (const int drc = require_gfx950("cw_ln_bwd_partials_open"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return bwd_partials_impl<std::remove_pointer_t<decltype(tag)>>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums,
                                                                       nullptr, nullptr, CW_F32, workspace,
                                                                       workspace_bytes, s, nullptr, 0, nullptr, n_parts);
    });
}

extern "C" int cw_ln_bwd_dx_close(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                                  const float* mean_rstd, const void* gamma, const float* row_sums, int64_t H, void* dx,
                                  int64_t ld_dx, const void* workspace, int64_t n_parts, void* dgamma, void* dbeta,
                                  int param_dtype, int io_dtype, void* stream) {
    int rc = check_rc("cw_ln_bwd_dx_close", R, C, io_dtype);
    if (rc != CW_OK) return rc;
    if (!col_out_dtype_ok(param_dtype)) return fail(CW_ERR_INVALID, "cw_ln_bwd_dx_close: bad param_dtype %d", param_dtype);
    if (H < C) return fail(CW_ERR_INVALID, "cw_ln_bwd_dx_close: hidden size H=%lld smaller than local C=%lld", (long long)H, (long long)C);
    if (dgamma == nullptr || dbeta == nullptr) return fail(CW_ERR_INVALID, "cw_ln_bwd_dx_close: dgamma and dbeta are both needed");
    if (n_parts < 0 || n_parts > (1 << 20) || (n_parts > 0 && workspace == nullptr) || C > ((int64_t)1 << 30))
        return fail(CW_ERR_INVALID, "cw_ln_bwd_dx_close: bad partial count %lld, NULL workspace or C too large", (long long)n_parts);
    if (const int drc = require_gfx950("cw_ln_bwd_dx_close"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (R == 0 || n_parts == 0) {
        // no rows: the column sums are zero (the finalize kernel over zero partial rows writes them)
        rc = finalize_col_partials(nullptr, 0, 2 * C, 2, C, dgamma, dbeta, param_dtype, s);
        if (rc != CW_OK || R == 0) return rc;
    }
    if (dY == nullptr || x == nullptr || mean_rstd == nullptr || row_sums == nullptr || dx == nullptr || ld_dy < C ||
        ld_x < C || ld_dx < C)
        return fail(CW_ERR_INVALID, "cw_ln_bwd_dx_close: null pointer or leading dimension < C");
    FinishCols fin;
    fin.ws = (const float*)workspace;
    fin.nparts = n_parts;
    fin.part_stride = 2 * C;
    fin.C = C;
    fin.out0 = dgamma;
    fin.out1 = dbeta;
    fin.out_dtype = param_dtype;
    fin.blocks = n_parts > 0 ? 2 * (int)((C + 63) / 64) : 0;
    return with_elem_type(io_dtype, [&](auto* tag) {
        return bwd_dx_impl<std::remove_pointer_t<decltype(tag)>>(R, C, dY, ld_dy, x, ld_x, mean_rstd, gamma, row_sums, H, dx,
                                                                 ld_dx, s, &fin);
    });
}
