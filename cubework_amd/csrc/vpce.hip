// Vocab-parallel cross-entropy, one rank's vocabulary slice, for gfx950.
// forward: one online pass (running max + rescaled sum of exponentials) over a
// row per 256-thread block, 16-byte loads, wavefront-shuffle reductions, plus
// the bit-exact target mask / shifted index / gather. backward: recomputes the
// softmax from the logits and the global (max, sum) and writes the gradient;
// the logits are never modified.
#include <type_traits>

#include "cw_common.h"

namespace cw {

namespace {

constexpr int kCeBlock = 256;
constexpr int kCeUnroll = 3;     // 16-byte loads in flight per thread, forward
// Backward: one block of 16 wavefronts per row, every thread's share of the row requested at once. Measured on
// 8192 x 12568 bf16 -> fp32 (8-byte loads, 16-byte stores): 256 threads per row 118 us, 512: 116, 1024: 107.
constexpr int kCeBwdBlock = 1024;
constexpr float kNegInf = -__builtin_huge_valf();

// Running (max m, sum s of exp(x - m)) kept in the exp2 domain: m2 = m*log2(e).
struct OnlineLse {
    float m;   // running maximum of the logits seen (exact input value)
    float m2;  // m * log2(e), or 0 while m is -inf
    float s;   // sum of exp2(x*log2e - m2)
};

template <int V>
__device__ __forceinline__ float chunk_max(const float (&v)[V]) {
    float cm = v[0];
#pragma unroll
    for (int e = 1; e < V; ++e) cm = fmaxf(cm, v[e]);
    return cm;
}

// Adds U chunks with one rescale of the running sum.
template <int V, int U>
__device__ __forceinline__ void lse_add_chunks(OnlineLse& st, const float (&v)[U][V]) {
    float cm = chunk_max<V>(v[0]);
#pragma unroll
    for (int u = 1; u < U; ++u) cm = fmaxf(cm, chunk_max<V>(v[u]));
    const float m_new = fmaxf(st.m, cm);
    const float m2_new = (m_new == kNegInf) ? 0.0f : m_new * kLog2e;
    const float scale = (st.m == kNegInf) ? 0.0f : __builtin_amdgcn_exp2f(st.m2 - m2_new);
    float s = st.s * scale;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        float su = 0.0f;  // per-chunk partial sums keep the add chains short
#pragma unroll
        for (int e = 0; e < V; ++e) su += __builtin_amdgcn_exp2f(__builtin_fmaf(v[u][e], kLog2e, -m2_new));
        s += su;
    }
    st.m = m_new;
    st.m2 = m2_new;
    st.s = s;
}

template <int V>
__device__ __forceinline__ void lse_add_chunk(OnlineLse& st, const float (&v)[V]) {
    const float cm = chunk_max<V>(v);
    const float m_new = fmaxf(st.m, cm);
    const float m2_new = (m_new == kNegInf) ? 0.0f : m_new * kLog2e;
    // rescale the old sum; an empty state (m == -inf) has s == 0 and stays 0
    const float scale = (st.m == kNegInf) ? 0.0f : __builtin_amdgcn_exp2f(st.m2 - m2_new);
    float s = st.s * scale;
#pragma unroll
    for (int e = 0; e < V; ++e) s += __builtin_amdgcn_exp2f(__builtin_fmaf(v[e], kLog2e, -m2_new));
    st.m = m_new;
    st.m2 = m2_new;
    st.s = s;
}

__device__ __forceinline__ void lse_add_one(OnlineLse& st, float x) {
    const float v[1] = {x};
    lse_add_chunk<1>(st, v);
}

// Merge (m_b, s_b) into (m_a, s_a).
__device__ __forceinline__ void lse_merge(float& m_a, float& s_a, float m_b, float s_b) {
    const float m = fmaxf(m_a, m_b);
    const float fa = (m_a == kNegInf) ? 0.0f : __builtin_amdgcn_exp2f((m_a - m) * kLog2e);
    const float fb = (m_b == kNegInf) ? 0.0f : __builtin_amdgcn_exp2f((m_b - m) * kLog2e);
    s_a = s_a * fa + s_b * fb;
    m_a = m;
}

template <typename T>
__global__ __launch_bounds__(kCeBlock) void vpce_fwd_kernel(int64_t T_rows, int64_t V_cols,
                                                            const T* __restrict__ logits, int64_t ld,
                                                            const int64_t* __restrict__ targets, int64_t vocab_start,
                                                            float* __restrict__ out_max, float* __restrict__ out_sumexp,
                                                            float* __restrict__ out_pred, uint8_t* __restrict__ out_mask,
                                                            int vec_ok) {
    constexpr int V = elem<T>::kVec;
    __shared__ float red_m[kCeBlock / 64];
    __shared__ float red_s[kCeBlock / 64];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    for (int64_t row = blockIdx.x; row < T_rows; row += gridDim.x) {
        const T* xr = logits + row * ld;
        OnlineLse st{kNegInf, 0.0f, 0.0f};
        if (vec_ok) {
            const int64_t nvec = V_cols / V;
            int64_t i = tid;
            // kCeUnroll independent 16-byte streaming loads in flight per trip
            for (; i + (kCeUnroll - 1) * kCeBlock < nvec; i += kCeUnroll * kCeBlock) {
                raw16_t raw[kCeUnroll];
#pragma unroll
                for (int u = 0; u < kCeUnroll; ++u) raw[u] = load_raw_stream(xr + (i + u * kCeBlock) * V);
                float v[kCeUnroll][V];
#pragma unroll
                for (int u = 0; u < kCeUnroll; ++u) unpack_raw(raw[u], v[u], (const T*)nullptr);
                lse_add_chunks<V, kCeUnroll>(st, v);
            }
            for (; i < nvec; i += kCeBlock) {
                float v0[V];
                unpack_raw(load_raw_stream(xr + i * V), v0, (const T*)nullptr);
                lse_add_chunk<V>(st, v0);
            }
            for (int64_t c = nvec * V + tid; c < V_cols; c += kCeBlock) lse_add_one(st, load_elem(xr + c));
        } else {
            for (int64_t c = tid; c < V_cols; c += kCeBlock) lse_add_one(st, load_elem(xr + c));
        }
        // wavefront, then block
        float m = st.m, s = st.s;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float mo = __shfl_xor(m, off, 64);
            const float so = __shfl_xor(s, off, 64);
            lse_merge(m, s, mo, so);
        }
        if (lane == 0) {
            red_m[wave] = m;
            red_s[wave] = s;
        }
        __syncthreads();
        if (tid == 0) {
            float gm = red_m[0], gs = red_s[0];
#pragma unroll
            for (int w = 1; w < kCeBlock / 64; ++w) lse_merge(gm, gs, red_m[w], red_s[w]);
            out_max[row] = gm;
            out_sumexp[row] = gs;
            // target bookkeeping: integer-exact
            const int64_t t = targets[row];
            const bool masked = (t < vocab_start) || (t >= vocab_start + V_cols);
            const int64_t idx = masked ? 0 : (t - vocab_start);
            out_mask[row] = masked ? 1 : 0;
            out_pred[row] = masked ? 0.0f : load_elem(xr + idx);
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void vpce_finalize_kernel(int64_t T_rows, int n_ranks,
                                                            const float* __restrict__ max_all,
                                                            const float* __restrict__ sumexp_all,
                                                            const float* __restrict__ pred_all,
                                                            const uint8_t* __restrict__ mask_all,
                                                            float* __restrict__ loss, float* __restrict__ gmax,
                                                            float* __restrict__ gsum) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= T_rows) return;
    float m = max_all[t];
    for (int r = 1; r < n_ranks; ++r) m = fmaxf(m, max_all[(int64_t)r * T_rows + t]);
    float s = 0.0f, p = 0.0f;
    for (int r = 0; r < n_ranks; ++r) {
        const float mr = max_all[(int64_t)r * T_rows + t];
        const float f = (mr == kNegInf) ? 0.0f : expf(mr - m);
        s += sumexp_all[(int64_t)r * T_rows + t] * f;
        if (mask_all[(int64_t)r * T_rows + t] == 0) p += pred_all[(int64_t)r * T_rows + t] - m;
    }
    loss[t] = logf(s) - p;
    if (gmax != nullptr) gmax[t] = m;
    if (gsum != nullptr) gsum[t] = s;
}

// The gradient is written once and not read again by this kernel: streaming stores.
template <int V>
__device__ __forceinline__ void store_grad(bf16_t* p, const float (&v)[V]) {
    static_assert(V == 8, "bf16 gradients are written 8 at a time");
    store_raw_stream(p, pack_raw(v, (const bf16_t*)nullptr));
}
template <int V>
__device__ __forceinline__ void store_grad(f16_t* p, const float (&v)[V]) {
    static_assert(V == 8, "fp16 gradients are written 8 at a time");
    store_raw_stream(p, pack_raw(v, (const f16_t*)nullptr));
}
template <int V>
__device__ __forceinline__ void store_grad(float* p, const float (&v)[V]) {
#pragma unroll
    for (int e = 0; e < V; e += 4) {
        const float q[4] = {v[e], v[e + 1], v[e + 2], v[e + 3]};
        store_raw_stream(p + e, pack_raw(q, (const float*)nullptr));
    }
}

// One 16-byte vector of the gradient row: softmax * scale, minus dl at the target column.
template <typename T, typename G, int V>
__device__ __forceinline__ void grad_vector(raw16_t raw, int64_t i, int64_t tcol, float m2, float scale, float dl,
                                            G* __restrict__ gr) {
    float v[V];
    unpack_raw(raw, v, (const T*)nullptr);
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(v[e], kLog2e, -m2)) * scale;
    const int64_t rel = tcol - i * V;
    if (rel >= 0 && rel < V) {
#pragma unroll
        for (int e = 0; e < V; ++e)
            if (e == rel) v[e] -= dl;
    }
    store_grad<V>(gr + i * V, v);
}

// fp32 gradient of 16-bit logits: four logits (8 bytes) in, four floats (16 bytes) out per lane, so that the
// stores of one instruction cover one contiguous 1 KB span. With 16-byte loads a lane would write 32
// bytes in two stores that each leave every other 16 bytes to the next instruction.
typedef uint32_t raw8_t __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ void grad_quad(raw8_t raw, int64_t i, int64_t tcol, float m2, float scale, float dl,
                                          float* __restrict__ gr) {
    float v[4] = {half_conv<T>::lo(raw.x), half_conv<T>::hi(raw.x), half_conv<T>::lo(raw.y), half_conv<T>::hi(raw.y)};
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(v[e], kLog2e, -m2)) * scale;
    const int64_t rel = tcol - i * 4;
    if (rel >= 0 && rel < 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e == rel) v[e] -= dl;
    }
    store_raw_stream(gr + i * 4, pack_raw(v, (const float*)nullptr));
}

// Per-row scalars of the backward: fetched after the row's first loads have been issued.
struct CeRowScalars {
    float m2, dl, scale;
    int64_t tcol;
};
__device__ __forceinline__ CeRowScalars ce_row_scalars(int64_t row, int64_t V_cols, const int64_t* __restrict__ targets,
                                                       int64_t vocab_start, const float* __restrict__ gmax,
                                                       const float* __restrict__ gsum,
                                                       const float* __restrict__ dloss_rows, float dloss_scale) {
    CeRowScalars r;
    r.m2 = gmax[row] * kLog2e;
    r.dl = (dloss_rows != nullptr ? dloss_rows[row] : 1.0f) * dloss_scale;
    r.scale = r.dl / gsum[row];
    const int64_t t = targets[row];
    const bool masked = (t < vocab_start) || (t >= vocab_start + V_cols);
    r.tcol = masked ? -1 : (t - vocab_start);
    return r;
}

template <typename T, typename G>
__global__ __launch_bounds__(kCeBwdBlock) void vpce_bwd_kernel(int64_t T_rows, int64_t V_cols,
                                                               const T* __restrict__ logits, int64_t ld,
                                                               const int64_t* __restrict__ targets, int64_t vocab_start,
                                                               const float* __restrict__ gmax,
                                                               const float* __restrict__ gsum,
                                                               const float* __restrict__ dloss_rows, float dloss_scale,
                                                               G* __restrict__ grad, int64_t ld_grad, int vec_ok) {
    constexpr int V = elem<T>::kVec;
    constexpr int B = kCeBwdBlock;
    const int tid = threadIdx.x;
    for (int64_t row = blockIdx.x; row < T_rows; row += gridDim.x) {
        const T* xr = logits + row * ld;
        G* gr = grad + row * ld_grad;
        if constexpr (sizeof(T) == 2 && std::is_same<G, float>::value) {
          if (vec_ok) {
            // fp32 gradient of 16-bit logits: batches of U quads (8 bytes in, 16 out) per thread, all requested
            // before the first is worked on; a position past the end of the row re-reads the last quad (no
            // load under a branch) and stores nothing
            constexpr int U = 4;
            const int64_t nq = V_cols / 4;
            const uint16_t* xb = reinterpret_cast<const uint16_t*>(xr);
            float* gf = reinterpret_cast<float*>(gr);
            CeRowScalars rs;
            for (int64_t base = tid; base < nq; base += (int64_t)U * B) {
                raw8_t raw[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t i = base + (int64_t)u * B;
                    raw[u] = __builtin_nontemporal_load(reinterpret_cast<const raw8_t*>(xb + (i < nq ? i : nq - 1) * 4));
                }
                if (base == tid) rs = ce_row_scalars(row, V_cols, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale);
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t i = base + (int64_t)u * B;
                    if (i < nq) grad_quad<T>(raw[u], i, rs.tcol, rs.m2, rs.scale, rs.dl, gf);
                }
            }
            if (nq * 4 < V_cols) {
                rs = ce_row_scalars(row, V_cols, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale);
                for (int64_t c = nq * 4 + tid; c < V_cols; c += B) {
                    float y = __builtin_amdgcn_exp2f(__builtin_fmaf(load_elem(xr + c), kLog2e, -rs.m2)) * rs.scale;
                    if (c == rs.tcol) y -= rs.dl;
                    store_elem(gr + c, y);
                }
            }
            continue;
          }
        }
        if (vec_ok) {
            const int64_t nvec = V_cols / V;
            CeRowScalars rs;
            if constexpr (sizeof(T) == 2) {
                // 16-bit in, 16-bit out: one vector per thread and trip. Sixteen wavefronts per row and two rows
                // per compute unit keep enough loads in flight; batching loads per thread measured slower here.
                rs = ce_row_scalars(row, V_cols, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale);
                for (int64_t i = tid; i < nvec; i += B)
                    grad_vector<T, G, V>(load_raw_stream(xr + i * V), i, rs.tcol, rs.m2, rs.scale, rs.dl, gr);
            } else {
                constexpr int U = 4;  // 16-byte vectors per thread and batch
                for (int64_t base = tid; base < nvec; base += (int64_t)U * B) {
                    raw16_t raw[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int64_t i = base + (int64_t)u * B;
                        raw[u] = load_raw_stream(xr + (i < nvec ? i : nvec - 1) * V);
                    }
                    if (base == tid) rs = ce_row_scalars(row, V_cols, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale);
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int64_t i = base + (int64_t)u * B;
                        if (i < nvec) grad_vector<T, G, V>(raw[u], i, rs.tcol, rs.m2, rs.scale, rs.dl, gr);
                    }
                }
            }
            if (nvec * V < V_cols) {
                rs = ce_row_scalars(row, V_cols, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale);
                for (int64_t c = nvec * V + tid; c < V_cols; c += B) {
                    float y = __builtin_amdgcn_exp2f(__builtin_fmaf(load_elem(xr + c), kLog2e, -rs.m2)) * rs.scale;
                    if (c == rs.tcol) y -= rs.dl;
                    store_elem(gr + c, y);
                }
            }
        } else {
            const CeRowScalars rs = ce_row_scalars(row, V_cols, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale);
            for (int64_t c = tid; c < V_cols; c += B) {
                float y = __builtin_amdgcn_exp2f(__builtin_fmaf(load_elem(xr + c), kLog2e, -rs.m2)) * rs.scale;
                if (c == rs.tcol) y -= rs.dl;
                store_elem(gr + c, y);
            }
        }
    }
}

int ce_grid(int64_t T_rows) {
    const int64_t cap = (int64_t)1 << 20;  // one block per row: finished blocks are replaced one by one
    return (int)(T_rows < cap ? T_rows : cap);
}

template <typename T, typename G>
int bwd_impl(int64_t T_rows, int64_t V_cols, const void* logits, int64_t ld, const int64_t* targets,
             int64_t vocab_start, const float* gmax, const float* gsum, const float* dloss_rows, float dloss_scale,
             void* grad, int64_t ld_grad, hipStream_t s) {
    const int vec_ok = aligned16(logits) && (ld % elem<T>::kVec) == 0 && aligned16(grad) &&
                       (ld_grad % (16 / (int)sizeof(G))) == 0;
    hipLaunchKernelGGL((vpce_bwd_kernel<T, G>), dim3(ce_grid(T_rows)), dim3(kCeBwdBlock), 0, s, T_rows, V_cols,
                       (const T*)logits, ld, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale, (G*)grad,
                       ld_grad, vec_ok);
    return check_launch("vpce_bwd_kernel");
}

}  // namespace
}  // namespace cw

using namespace cw;

extern "C" int cw_vpce_fwd_local(int64_t T, int64_t V, const void* logits, int64_t ld, const int64_t* targets,
                                 int64_t vocab_start, float* out_max, float* out_sumexp, float* out_pred,
                                 uint8_t* out_mask, int io_dtype, void* stream) {
    if (T < 0 || V <= 0) return fail(CW_ERR_INVALID, "cw_vpce_fwd_local: bad shape T=%lld V=%lld", (long long)T, (long long)V);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_vpce_fwd_local: bad io_dtype %d", io_dtype);
    if (vocab_start < 0) return fail(CW_ERR_INVALID, "cw_vpce_fwd_local: negative vocab_start");
    if (T == 0) return CW_OK;
    if (logits == nullptr || targets == nullptr || out_max == nullptr || out_sumexp == nullptr ||
        out_pred == nullptr || out_mask == nullptr || ld < V)
        return fail(CW_ERR_INVALID, "cw_vpce_fwd_local: null pointer or ld < V");
    if (const int drc = require_gfx950("cw_vpce_fwd_local"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (io_dtype == CW_BF16) {
        const int vec_ok = aligned16(logits) && (ld % 8) == 0;
        hipLaunchKernelGGL(vpce_fwd_kernel<bf16_t>, dim3(ce_grid(T)), dim3(kCeBlock), 0, s, T, V,
                           (const bf16_t*)logits, ld, targets, vocab_start, out_max, out_sumexp, out_pred, out_mask,
                           vec_ok);
    } else if (io_dtype == CW_F16) {
        const int vec_ok = aligned16(logits) && (ld % 8) == 0;
        hipLaunchKernelGGL(vpce_fwd_kernel<f16_t>, dim3(ce_grid(T)), dim3(kCeBlock), 0, s, T, V,
                           (const f16_t*)logits, ld, targets, vocab_start, out_max, out_sumexp, out_pred, out_mask,
                           vec_ok);
    } else {
        const int vec_ok = aligned16(logits) && (ld % 4) == 0;
        hipLaunchKernelGGL(vpce_fwd_kernel<float>, dim3(ce_grid(T)), dim3(kCeBlock), 0, s, T, V,
                           (const float*)logits, ld, targets, vocab_start, out_max, out_sumexp, out_pred, out_mask,
                           vec_ok);
    }
    return check_launch("vpce_fwd_kernel");
}

extern "C" int cw_vpce_finalize(int64_t T, int n_ranks, const float* max_all, const float* sumexp_all,
                                const float* pred_all, const uint8_t* mask_all, float* loss, float* gmax,
                                float* gsum, void* stream) {
    if (T < 0 || n_ranks < 1) return fail(CW_ERR_INVALID, "cw_vpce_finalize: bad T=%lld or n_ranks=%d", (long long)T, n_ranks);
    if (T == 0) return CW_OK;
    if (max_all == nullptr || sumexp_all == nullptr || pred_all == nullptr || mask_all == nullptr || loss == nullptr)
        return fail(CW_ERR_INVALID, "cw_vpce_finalize: null pointer");
    if (const int drc = require_gfx950("cw_vpce_finalize"); drc != CW_OK) return drc;
    hipLaunchKernelGGL(vpce_finalize_kernel, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, (hipStream_t)stream, T,
                       n_ranks, max_all, sumexp_all, pred_all, mask_all, loss, gmax, gsum);
    return check_launch("vpce_finalize_kernel");
}

extern "C" int cw_vpce_bwd(int64_t T, int64_t V, const void* logits, int64_t ld, const int64_t* targets,
                           int64_t vocab_start, const float* gmax, const float* gsum, const float* dloss_rows,
                           float dloss_scale, void* grad, int64_t ld_grad, int io_dtype, int grad_dtype,
                           void* stream) {
    if (T < 0 || V <= 0) return fail(CW_ERR_INVALID, "cw_vpce_bwd: bad shape T=%lld V=%lld", (long long)T, (long long)V);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_vpce_bwd: bad io_dtype %d", io_dtype);
    if (grad_dtype != CW_BF16 && grad_dtype != CW_F32 && grad_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_vpce_bwd: bad grad_dtype %d", grad_dtype);
    if (grad_dtype != CW_F32 && grad_dtype != io_dtype)
        return fail(CW_ERR_UNSUPPORTED, "cw_vpce_bwd: the gradient is fp32 or of the logits' type");
    if (T == 0) return CW_OK;
    if (logits == nullptr || targets == nullptr || gmax == nullptr || gsum == nullptr || grad == nullptr || ld < V ||
        ld_grad < V)
        return fail(CW_ERR_INVALID, "cw_vpce_bwd: null pointer or leading dimension < V");
    if (const int drc = require_gfx950("cw_vpce_bwd"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    if (io_dtype == CW_F16 && grad_dtype == CW_F16)
        return bwd_impl<f16_t, f16_t>(T, V, logits, ld, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale, grad, ld_grad, s);
    if (io_dtype == CW_F16)
        return bwd_impl<f16_t, float>(T, V, logits, ld, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale, grad, ld_grad, s);
    if (io_dtype == CW_BF16 && grad_dtype == CW_BF16)
        return bwd_impl<bf16_t, bf16_t>(T, V, logits, ld, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale, grad, ld_grad, s);
    if (io_dtype == CW_BF16)
        return bwd_impl<bf16_t, float>(T, V, logits, ld, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale, grad, ld_grad, s);
    return bwd_impl<float, float>(T, V, logits, ld, targets, vocab_start, gmax, gsum, dloss_rows, dloss_scale, grad, ld_grad, s);
}
