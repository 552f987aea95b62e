// Deterministic column reductions shared by the bias-gradient and LayerNorm
// backward kernels: register accumulators -> LDS tree across the block's
// wavefronts -> one partial row per block in global memory -> finalize kernel.
#pragma once

#include "cw_common.h"

namespace cw {

inline size_t tree_reduce_lds_bytes(int nreg, int nwaves) {
    return (size_t)(nwaves / 2 > 0 ? nwaves / 2 : 1) * nreg * 64 * sizeof(float);
}

// Sums acc[] element-wise over the NWAVES wavefronts of a block into
// wavefront 0, in a fixed order. Must be reached by every thread of the block.
template <int NREG, int NWAVES>
__device__ __forceinline__ void block_tree_reduce(float (&acc)[NREG], float* lds, int wave, int lane) {
#pragma unroll
    for (int half = NWAVES / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
            float* region = lds + (size_t)(wave - half) * NREG * 64;
#pragma unroll
            for (int i = 0; i < NREG; ++i) region[i * 64 + lane] = acc[i];
        }
        __syncthreads();
        if (wave < half) {
            const float* region = lds + (size_t)wave * NREG * 64;
#pragma unroll
            for (int i = 0; i < NREG; ++i) acc[i] += region[i * 64 + lane];
        }
        __syncthreads();
    }
}

// Flat variant for wide accumulator sets: every wavefront writes its NREG x 64 accumulators to LDS once
// ([wave][reg][lane], NWAVES * NREG * 256 bytes), one barrier, then thread t adds the NWAVES values of
// accumulator slots t, t + NWAVES*64, ... in wavefront order and hands each total to sink(reg, lane, total).
inline size_t flat_reduce_lds_bytes(int nreg, int nwaves) { return (size_t)nwaves * nreg * 64 * sizeof(float); }

template <int NREG, int NWAVES, typename Sink>
__device__ __forceinline__ void block_flat_reduce(const float (&acc)[NREG], float* lds, int wave, int lane, Sink&& sink) {
    float* mine = lds + (size_t)wave * NREG * 64;
#pragma unroll
    for (int i = 0; i < NREG; ++i) mine[i * 64 + lane] = acc[i];
    __syncthreads();
    const int tid = wave * 64 + lane;
    for (int o = tid; o < NREG * 64; o += NWAVES * 64) {
        float total = lds[o];
#pragma unroll
        for (int w = 1; w < NWAVES; ++w) total += lds[(size_t)w * NREG * 64 + o];
        sink(o >> 6, o & 63, total);
    }
}

// The column finalize as the leading workgroups of another launch: the first `blocks` workgroups of a kernel that
// was handed a FinishCols add the partial rows (out_k[c] = sum_p ws[p*part_stride + k*C + c], k < 2) and return, the
// others do the kernel's own work with their index shifted. blocks = 2 * ceil(C / 64); 0 = nothing to finish.
struct FinishCols {
    const float* ws;
    int64_t nparts, part_stride, C;
    void* out0;
    void* out1;
    int blocks;
    int out_dtype;  // CW_F32 / CW_BF16 / CW_F16: the type the totals are stored in (rounded once, to nearest even)
};

// One finished column total into an output vector of the given element type.
__device__ __forceinline__ void store_col_total(void* out, int64_t c, float total, int out_dtype) {
    if (out_dtype == CW_F32) reinterpret_cast<float*>(out)[c] = total;
    else if (out_dtype == CW_BF16) store_elem(reinterpret_cast<bf16_t*>(out) + c, total);
    else store_elem(reinterpret_cast<f16_t*>(out) + c, total);
}

// Workgroup `block` (< f.blocks) of THREADS threads: 64 columns of one of the two sets. The THREADS / 64 groups
// of 64 threads split the partial rows, 16 independent loads in flight each, and are combined in index order.
// red: THREADS floats of LDS. Must be reached by every thread of the workgroup.
template <int THREADS>
__device__ __forceinline__ void finish_cols_block(const FinishCols& f, int block, float* red) {
    constexpr int G = THREADS / 64;
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int col_blocks = f.blocks / 2;
    const int k = block / col_blocks;
    const int64_t c = (int64_t)(block - k * col_blocks) * 64 + lane;
    float acc = 0.0f;
    if (c < f.C) {
        const float* base = f.ws + (int64_t)k * f.C + c;
        for (int64_t p = grp; p < f.nparts; p += 16 * G) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int64_t q = p + u * G;
                v[u] = base[(q < f.nparts ? q : f.nparts - 1) * f.part_stride];
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) acc += (p + u * G < f.nparts) ? v[u] : 0.0f;
        }
    }
    red[grp * 64 + lane] = acc;
    __syncthreads();
    if (grp == 0 && c < f.C) {
        float total = red[lane];
#pragma unroll
        for (int g = 1; g < G; ++g) total += red[g * 64 + lane];
        void* out = (k == 0) ? f.out0 : f.out1;
        if (out != nullptr) store_col_total(out, c, total, f.out_dtype);
    }
}

// out_k[c] = sum_p ws[p*part_stride + k*C + c], k < nsets (nsets is 1 or 2;
// out1 is ignored when nsets == 1), stored as out_dtype. Enqueued on `s`.
int finalize_col_partials(const float* ws, int64_t nparts, int64_t part_stride, int nsets, int64_t C, void* out0,
                          void* out1, int out_dtype, hipStream_t s);

inline bool col_out_dtype_ok(int dt) { return dt == CW_F32 || dt == CW_BF16 || dt == CW_F16; }

// Scratch bounds of the two users, combined by cw_colsum_workspace_bytes.
int64_t colsum_workspace_bytes(int64_t M, int64_t N);
int64_t ln_bwd_workspace_bytes(int64_t R, int64_t C);

}  // namespace cw
