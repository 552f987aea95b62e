/*
 * cubework_hip.h — C ABI of libcubework_hip.so (gfx950 / MI355X).
 *
 * One rank's share of the compute inside Cubework's tensor-parallel layers:
 * the SUMMA block-GEMM accumulation loop (+ bias + activation), LayerNorm
 * partial statistics / normalise / backward, vocab-parallel cross-entropy.
 * Operands a collective would have delivered are passed as extra device
 * pointers ("pre-staged" peers); the library never communicates.
 *
 * Conventions for every entry point
 *   - returns 0 on success, a negative cw_status on failure; the message for
 *     the calling thread is available from cw_last_error();
 *   - every data pointer is a DEVICE pointer owned by the caller, row-major,
 *     with explicit leading dimensions counted in ELEMENTS;
 *   - no allocation, no synchronisation, nothing on the null stream: work is
 *     enqueued on `stream` (a hipStream_t passed as void*) and the call returns;
 *   - re-entrant and callable from any thread (the autograd engine calls the
 *     backward entry points from its own device thread);
 *   - io_dtype selects the storage type of activations/weights (CW_BF16,
 *     CW_F32 or CW_F16); statistics, losses and all
 *     accumulation are fp32.
 *
 * Citations name the reference code (kurisusnowdeng/Cubework) each entry
 * point stands in for; paths are relative to the reference tree.
 */
#ifndef CUBEWORK_HIP_H
#define CUBEWORK_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    CW_OK = 0,
    CW_ERR_INVALID = -1,     /* bad argument (shape, enum, null pointer) */
    CW_ERR_ALIGNMENT = -2,   /* pointer / leading dimension not usable   */
    CW_ERR_UNSUPPORTED = -3, /* valid request this build cannot serve    */
    CW_ERR_LAUNCH = -4,      /* HIP reported an error at launch          */
    CW_ERR_DEVICE = -5       /* current device is not gfx950             */
} cw_status;

/* CW_F16 (IEEE half) is the type the reference's GEMM-type Functions cast to under autocast
 * (custom_fwd(cast_inputs=torch.float16), cubework/module/parallel_2d/_operation.py:17,96,176,255,363) and
 * the type of every tensor of a model converted with .half(), where nothing casts. Every entry point
 * takes it. Under autocast the reference runs LayerNorm in fp32 on the fp32 residual stream (CW_F32
 * here) and casts the logits of its loss to fp32 first, which reading them as 16-bit values and computing
 * in fp32 reproduces without the copy. */
typedef enum { CW_BF16 = 0, CW_F32 = 1, CW_F16 = 2 } cw_dtype;

/* Operand orientation of the block GEMM, per k-step i:
 *   CW_NN: C[M,N] += A_i[M,K] * B_i[K,N]      (summa_AB,  Linear2D/3D forward)
 *   CW_NT: C[M,N] += A_i[M,K] * B_i[N,K]^T    (summa_ABT, F.linear, dX, classifiers)
 *   CW_TN: C[M,N] += A_i[K,M]^T * B_i[K,N]    (summa_ATB, dW)                       */
typedef enum { CW_NN = 0, CW_NT = 1, CW_TN = 2 } cw_layout;

typedef enum {
    CW_EPI_NONE = 0,       /* C = acc (+ addends)                    */
    CW_EPI_BIAS = 1,       /* C = acc + bias[N]                      */
    CW_EPI_BIAS_GELU_TANH = 2,
    CW_EPI_BIAS_GELU_ERF = 3,
    CW_EPI_BIAS_RELU = 4
} cw_epilogue;

typedef enum { CW_ACT_NONE = 0, CW_ACT_GELU_TANH = 2, CW_ACT_GELU_ERF = 3, CW_ACT_RELU = 4 } cw_activation;

/* LayerNorm statistics convention.
 *   CW_LN_ONE_PASS : partials are (sum x, sum x^2); var = E[x^2] - E[x]^2
 *                    (LayerNorm2D, parallel_2d/module.py:142-153)
 *   CW_LN_TWO_PASS : first exchange gives the mean, second partial is
 *                    sum (x-mean)^2 (LayerNorm3D, parallel_3d/_operation.py:273-276) */
typedef enum { CW_LN_ONE_PASS = 0, CW_LN_TWO_PASS = 1 } cw_ln_mode;

#define CW_MAX_KSTEPS 16
#define CW_MAX_ADDENDS 8

/* ---- sanity ------------------------------------------------------------ */
const char* cw_version(void);
/* gcnArchName of the current device ("gfx950:..."), or "" without a device. */
const char* cw_device_arch(void);
/* Message of the last failing call made by this thread ("" if none). */
const char* cw_last_error(void);

/* ---- block GEMM with k-step accumulation ------------------------------- */
/*
 * C = act( sum_{i<n_steps} op(A_i) * op(B_i) + sum_{j<n_addends} addend_j + bias )
 *
 * Replaces the per-rank math of
 *   _SUMMA_AB.forward   cubework/module/parallel_2d/_operation.py:41-47  (CW_NN)
 *   _SUMMA_ABT.forward  cubework/module/parallel_2d/_operation.py:117-125 (CW_NT)
 *   _SUMMA_ATB.forward  cubework/module/parallel_2d/_operation.py:197-204 (CW_TN)
 *   _SUMMAbias.forward  cubework/module/parallel_2d/_operation.py:271-274 (bias)
 *   F.linear            cubework/module/parallel_1d/module.py:147,209,269,338 (CW_NT)
 *   _Linear3D fwd/bwd   cubework/module/parallel_3d/_operation.py:34,39,53,65
 *   _Classifier2D       cubework/module/parallel_2d/_operation.py:383,387,408-410
 *   activation after the linear: benchmark/gpt2/gpt2.py:116-117, benchmark/opt/opt.py:200
 * with A_steps[i]/B_steps[i] standing for what the row/column broadcast of
 * step i delivers, and addends[j] for the peers' partial products a reduce
 * delivers. A_steps/B_steps/addends are HOST arrays of device pointers.
 * K is the reduction length of ONE step. bias (length N, io_dtype) may be
 * NULL for any epilogue. preact (optional, [M,N], ld = ldp) receives the value
 * before the activation, for the backward of a fused activation. Accumulation
 * across k and across steps is fp32; the result is rounded once. C and preact
 * must not overlap the operands, the addends or each other (an element may be
 * computed and stored by two workgroups, with identical bits).
 */
int cw_gemm_ksteps(int layout, int64_t M, int64_t N, int64_t K, int n_steps,
                   const void* const* A_steps, int64_t lda,
                   const void* const* B_steps, int64_t ldb,
                   const void* bias, int epilogue,
                   void* C, int64_t ldc,
                   void* preact, int64_t ldp,
                   const void* const* addends, int n_addends, int64_t ldadd,
                   int io_dtype, void* stream);

/*
 * cw_gemm_ksteps with caller-provided scratch. When the output has too few
 * tiles to occupy the chip and the reduction is long -- the weight-gradient
 * products X^T dY of _SUMMA_AB.backward / _SUMMA_ABT.backward
 * (parallel_2d/_operation.py:63-66, 141-144, through _SUMMA_ATB.forward
 * :197-204), of F.linear's backward (parallel_1d/module.py:147,209,269,338) and
 * of _Linear3D.backward (parallel_3d/_operation.py:53) -- the k range of every
 * step is split over several workgroups per tile, whose fp32 partial sums go
 * through `workspace` and are added in a fixed order (bit-reproducible; the
 * reference leaves this choice, and its scratch, to the BLAS library inside
 * torch.matmul). The scratch also serves a large product whose reduction
 * length is not a multiple of the kernel's k tile and whose B is stored [K, N]
 * (the input gradient dC W of the vocabulary-slice classifiers,
 * parallel_2d/_operation.py:408, parallel_1d/module.py:209: K = 12568): 32 rows
 * of B are copied there, zero-padded, for one short extra k step.
 * cw_gemm_workspace_bytes gives the size that enables either (0 when the shape
 * uses neither); with workspace NULL or smaller the call behaves exactly like
 * cw_gemm_ksteps (same results, a slower kernel). The scratch must not be
 * shared by calls that may overlap on the device.
 */
int64_t cw_gemm_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps, int io_dtype);
int cw_gemm_ksteps_ws(int layout, int64_t M, int64_t N, int64_t K, int n_steps,
                      const void* const* A_steps, int64_t lda,
                      const void* const* B_steps, int64_t ldb,
                      const void* bias, int epilogue,
                      void* C, int64_t ldc,
                      void* preact, int64_t ldp,
                      const void* const* addends, int n_addends, int64_t ldadd,
                      void* workspace, int64_t workspace_bytes,
                      int io_dtype, void* stream);

/* ---- bias / activation backward ---------------------------------------- */
/*
 * Number of bytes of scratch cw_colsum / cw_act_bwd_colsum / cw_ln_bwd_partials / cw_ln_backward_fused
 * need for an [M,N] operand.
 */
int64_t cw_colsum_workspace_bytes(int64_t M, int64_t N);

/*
 * out[N] = sum over rows of dY[M,N], accumulated in fp32 and stored as out_dtype
 * (CW_F32, or CW_BF16 / CW_F16 rounded once to nearest even: the parameter's own
 * type, so that no cast launch follows, as the reference's sum in the tensors'
 * dtype leaves none).
 * Replaces torch.sum(output_grad, dim=reduce_dim) in _SUMMAbias.backward
 * (parallel_2d/_operation.py:285-286), _Classifier2D.backward (:414),
 * _Linear3D.backward (parallel_3d/_operation.py:59). Two deterministic stages
 * through `workspace` (no atomics).
 */
int cw_colsum(int64_t M, int64_t N, const void* dY, int64_t ld, void* out, int out_dtype,
              void* workspace, int64_t workspace_bytes, int io_dtype, void* stream);

/*
 * cw_colsum for callers that cannot allocate device memory or hand over scratch (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference,
 * whose torch.sum allocates through torch's caching allocator. Same kernels and same bits as cw_colsum;
 * the partial sums go through a 4 MiB array that is part of the library's code object (one copy per GPU,
 * held until the process ends; cw_colsum_static_max_bytes returns its size). Shapes whose partial sums do
 * not fit are refused with CW_ERR_UNSUPPORTED: with 16-byte aligned dY and ld, N % (16 / element size)
 * == 0 the limit is N <= 1048576, otherwise ceil(M / 64) * N <= 1048576. Calls on one GPU share the array:
 * calls that may overlap on the device (two streams, two threads) race; calls on one stream do not. The
 * first call on a device looks the array's address up (hipGetSymbolAddress): make it outside a capture (a first
 * call on a capturing stream is refused with CW_ERR_UNSUPPORTED and records nothing).
 * No hipMalloc / hipFree / allocating library routine on any call.
 */
int64_t cw_colsum_static_max_bytes(void);
int cw_colsum_static(int64_t M, int64_t N, const void* dY, int64_t ld, void* out, int out_dtype, int io_dtype,
                     void* stream);

/*
 * dPre[M,N] = dY * act'(preact); optionally dbias[N] = column sums of dPre, fp32
 * sums stored as dbias_dtype like cw_colsum's (dbias may be NULL, then workspace
 * may be NULL and dbias_dtype is ignored). Backward of the fused
 * activation epilogue of cw_gemm_ksteps; the reference runs it as autograd of
 * nn.functional.gelu / nn.ReLU (benchmark/gpt2/gpt2.py:117, benchmark/opt/opt.py:200)
 * followed by _SUMMAbias.backward.
 */
int cw_act_bwd_colsum(int activation, int64_t M, int64_t N,
                      const void* dY, int64_t ld_dy, const void* preact, int64_t ld_pre,
                      void* dPre, int64_t ld_dpre, void* dbias, int dbias_dtype,
                      void* workspace, int64_t workspace_bytes, int io_dtype, void* stream);

/* ---- LayerNorm ---------------------------------------------------------- */
/*
 * Local partial statistics of x[R,C] (this rank's C of the H hidden columns).
 *   CW_LN_ONE_PASS: stats[r] = (sum_c x, sum_c x^2)
 *   CW_LN_TWO_PASS: stats[r] = (sum_c (x-mean[r]), sum_c (x-mean[r])^2); mean == NULL
 *                   means "first exchange": stats[r] = (sum_c x, 0).
 * Replaces torch.sum(x), torch.sum(x*x) in LayerNorm2D.forward
 * (parallel_2d/module.py:144,148) and torch.sum(input_), torch.sum(mu**2) in
 * _Layernorm3D.forward (parallel_3d/_operation.py:273,275).
 */
int cw_ln_partial_stats(int64_t R, int64_t C, const void* x, int64_t ld, int mode,
                        const float* mean, float* stats, int io_dtype, void* stream);

/*
 * y = gamma * (x - mean) * rstd + beta from statistics summed over the whole
 * hidden size H (after the peers' partials were added):
 *   CW_LN_ONE_PASS: stats[r] = (sum x, sum x^2) over H
 *   CW_LN_TWO_PASS: stats[r] = (mean, sum (x-mean)^2 over H)
 * gamma/beta (length C, io_dtype) may be NULL (no affine). mean_rstd[R,2]
 * (fp32, optional) receives (mean, rstd) for the backward.
 * Replaces parallel_2d/module.py:145-153,170 + _Layernorm_2D.forward
 * (parallel_2d/_operation.py:321-324) and parallel_3d/_operation.py:273-281.
 */
int cw_ln_normalize(int64_t R, int64_t C, const void* x, int64_t ld, const float* stats,
                    int mode, int64_t H, float eps, const void* gamma, const void* beta,
                    void* y, int64_t ldy, float* mean_rstd, int io_dtype, void* stream);

/*
 * Statistics and normalise in one launch for the case with no peers (H == C):
 * what LayerNorm2D/3D compute at tensor-parallel size 1.
 */
int cw_ln_forward_fused(int64_t R, int64_t C, const void* x, int64_t ld, int mode, float eps,
                        const void* gamma, const void* beta, void* y, int64_t ldy,
                        float* mean_rstd, int io_dtype, void* stream);

/*
 * Backward partials. With g = dY * gamma and xhat = (x - mean) * rstd:
 *   row_sums[r] = (sum_c g, sum_c g*xhat)                 (fp32 [R,2])
 *   dgamma[c]   = sum_r dY*xhat, dbeta[c] = sum_r dY      ([C] each, optional; fp32 sums stored as
 *                                                          param_dtype: CW_F32, CW_BF16 or CW_F16)
 * Replaces _Layernorm_2D.backward sums (parallel_2d/_operation.py:334,338), the
 * autograd of torch.addcmul (parallel_2d/module.py:170) and the bias_grad /
 * weight_grad sums of _Layernorm3D.backward (parallel_3d/_operation.py:294-301).
 * dgamma == dbeta == NULL skips the column part (and needs no workspace).
 */
int cw_ln_bwd_partials(int64_t R, int64_t C, const void* dY, int64_t ld_dy,
                       const void* x, int64_t ld_x, const float* mean_rstd, const void* gamma,
                       float* row_sums, void* dgamma, void* dbeta, int param_dtype,
                       void* workspace, int64_t workspace_bytes, int io_dtype, void* stream);

/*
 * dx = (g - xhat * S2/H - S1/H) * rstd with (S1, S2) = row_sums summed over
 * the whole hidden size H. Replaces parallel_2d/_operation.py:336-345 and
 * parallel_3d/_operation.py:303-311.
 */
int cw_ln_bwd_dx(int64_t R, int64_t C, const void* dY, int64_t ld_dy,
                 const void* x, int64_t ld_x, const float* mean_rstd, const void* gamma,
                 const float* row_sums, int64_t H, void* dx, int64_t ld_dx,
                 int io_dtype, void* stream);
/*
 * cw_ln_bwd_partials and cw_ln_bwd_dx with the column finalize moved from a launch of its own (the second launch of
 * cw_ln_bwd_partials, 3 - 5 us between the two kernels) into the dx launch: cw_ln_bwd_partials_open writes row_sums
 * and leaves *n_parts unfinished column partial rows in `workspace` (sized by cw_ln_bwd_workspace_bytes; *n_parts
 * is a host value, set before the call returns); the caller all-reduces row_sums as before
 * (parallel_2d/_operation.py:335,339) and cw_ln_bwd_dx_close writes dx and, from its leading workgroups, dgamma and
 * dbeta ([C], stored as param_dtype) out of those rows, which must still be in `workspace`. Same arithmetic as the pair above; the
 * column sums are added in a fixed order (bit-reproducible) that differs from cw_ln_bwd_partials' in the last bits.
 */
int cw_ln_bwd_partials_open(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                            const float* mean_rstd, const void* gamma, float* row_sums, void* workspace,
                            int64_t workspace_bytes, int64_t* n_parts, int io_dtype, void* stream);
int cw_ln_bwd_dx_close(int64_t R, int64_t C, const void* dY, int64_t ld_dy, const void* x, int64_t ld_x,
                       const float* mean_rstd, const void* gamma, const float* row_sums, int64_t H, void* dx,
                       int64_t ld_dx, const void* workspace, int64_t n_parts, void* dgamma, void* dbeta,
                       int param_dtype, int io_dtype, void* stream);

/*
 * cw_ln_bwd_partials + cw_ln_bwd_dx with H = C in one pass over dY and x, for rows that are complete on
 * this rank: what _Layernorm_2D.backward (parallel_2d/_operation.py:330-347) and
 * _Layernorm3D.backward (parallel_3d/_operation.py:294-311) compute when the group their sums are
 * all-reduced over has one member. The counterpart of cw_ln_forward_fused. row_sums ([R,2] fp32) is
 * written as by cw_ln_bwd_partials; shapes the one-pass kernel does not take run the two kernels.
 * dx_addend (may be NULL; [R,C] of the io dtype, leading dimension ld_add): the gradient that reaches x along
 * a residual branch around the layer (benchmark/opt/opt.py:170,184 and :193,206), added to dx before its one
 * rounding: what autograd's accumulation of the two branches computes with a pass of its own. Taken by the
 * one-pass kernels only; a shape that runs the two kernels is refused with CW_ERR_UNSUPPORTED before any launch.
 */
int cw_ln_backward_fused(int64_t R, int64_t C, const void* dY, int64_t ld_dy,
                         const void* x, int64_t ld_x, const float* mean_rstd, const void* gamma,
                         float* row_sums, void* dx, int64_t ld_dx, const void* dx_addend, int64_t ld_add,
                         void* dgamma, void* dbeta, int param_dtype,
                         void* workspace, int64_t workspace_bytes, int io_dtype, void* stream);

/* ---- vocab-parallel cross-entropy -------------------------------------- */
/*
 * One online pass over this rank's vocabulary slice logits[T,V] (columns
 * [vocab_start, vocab_start+V) of the full vocabulary):
 *   out_max[t]    = max_c logits[t,c]
 *   out_sumexp[t] = sum_c exp(logits[t,c] - out_max[t])
 *   out_mask[t]   = 1 if targets[t] is outside the slice else 0
 *   out_pred[t]   = logits[t, targets[t]-vocab_start] as fp32 (0 where masked)
 * Replaces loss_1d.py:17,23-42,47-49; loss_2d.py:39,45-59,62-63;
 * loss_3d.py:43,48-60,64-65 (cubework/module/loss/). logits are not modified.
 */
int cw_vpce_fwd_local(int64_t T, int64_t V, const void* logits, int64_t ld,
                      const int64_t* targets, int64_t vocab_start,
                      float* out_max, float* out_sumexp, float* out_pred, uint8_t* out_mask,
                      int io_dtype, void* stream);

/*
 * Combine the n_ranks slices' statistics (row r of *_all is rank r's output of
 * cw_vpce_fwd_local; they stand for the MAX / SUM / SUM all-reduces of
 * loss_1d.py:18,44,50):
 *   gmax = max_r max_r[t];  gsum = sum_r sumexp_r[t] * exp(max_r[t] - gmax)
 *   loss = log(gsum) - sum_r (mask_r ? 0 : pred_r[t] - gmax)      (loss_1d.py:53)
 */
int cw_vpce_finalize(int64_t T, int n_ranks, const float* max_all, const float* sumexp_all,
                     const float* pred_all, const uint8_t* mask_all,
                     float* loss, float* gmax, float* gsum, void* stream);

/*
 * grad[t,c] = (exp(logits[t,c]-gmax[t]) / gsum[t] - [c == target column, in slice]) * dloss
 * with dloss = dloss_rows[t] * dloss_scale (dloss_rows may be NULL = all ones).
 * Recomputes the softmax instead of keeping it (loss_1d.py:55-56,61-79).
 * grad_dtype selects the storage type of grad: CW_F32 or the logits' type.
 */
int cw_vpce_bwd(int64_t T, int64_t V, const void* logits, int64_t ld,
                const int64_t* targets, int64_t vocab_start,
                const float* gmax, const float* gsum,
                const float* dloss_rows, float dloss_scale,
                void* grad, int64_t ld_grad, int io_dtype, int grad_dtype, void* stream);

/* ---- vocab-parallel embedding -------------------------------------------- */
/*
 * out[t, :] = (vocab_start <= ids[t] < vocab_start + V_loc) ? weight[ids[t] - vocab_start, :] : 0
 * Replaces the mask / shifted index / F.embedding / zeroing of masked rows in
 * VocabParallelEmbedding1D.forward (cubework/module/parallel_1d/module.py:441-452),
 * VocabParallelEmbedding2D.forward (parallel_2d/module.py:345-353),
 * VocabParallelEmbedding3D.forward (parallel_3d/module.py:455-466), and, with
 * vocab_start = 0 and V_loc = num_embeddings, F.embedding in Embedding1D/2D/3D
 * (parallel_1d/module.py:390, parallel_2d/module.py:290, parallel_3d/module.py:396).
 * The index arithmetic is integer-exact; the copy is bit-exact.
 */
int cw_embed_fwd(int64_t T, int64_t E, const int64_t* ids, int64_t vocab_start, int64_t V_loc,
                 const void* weight, int64_t ldw, void* out, int64_t ldo, int io_dtype, void* stream);

/*
 * d_weight[r, :] = sum over tokens t with ids[t] - vocab_start == r of d_out[t, :] (fp32 sum, rounded
 * once); rows without tokens, and row skip_row (F.embedding's padding_idx, -1 for none), are zero.
 * Autograd of the F.embedding call above. sorted_ids / order: the ids in ascending order and the
 * token position of each (a stable sort by the caller); runs of equal ids are summed in that order,
 * without atomics, so the result is bit-reproducible. One launch: the rows without tokens are found by a
 * search in sorted_ids and cleared by workgroups of the same grid. T, V_loc <= 2^30.
 */
int cw_embed_bwd(int64_t T, int64_t E, const int64_t* sorted_ids, const int64_t* order,
                 int64_t vocab_start, int64_t V_loc, int64_t skip_row,
                 const void* d_out, int64_t ldo, void* d_weight, int64_t ldw, int io_dtype, void* stream);

/*
 * The token order cw_embed_bwd takes, made on the device: sorted_ids[i] / order[i] = id and position of
 * the i-th token in ascending order of the selected row, ties in token order (a stable sort by id for
 * the ids in range). Ids outside [vocab_start, vocab_start + V_loc) are written as
 * vocab_start + V_loc and come last, so cw_embed_bwd skips them. Replaces the sort inside the
 * autograd of F.embedding (the reference's backward of parallel_1d/module.py:390,452 and its 2D / 3D
 * counterparts sorts the indices through torch's embedding_dense_backward). Integer-exact.
 * T <= 16384 needs no workspace (one launch places every token by counting the tokens ahead of it);
 * above that a sorting network runs over `workspace` of cw_embed_sort_workspace_bytes(T) bytes.
 * T <= 2^30, V_loc < 2^32 - 1.
 */
int64_t cw_embed_sort_workspace_bytes(int64_t T);
int cw_embed_sort_ids(int64_t T, const int64_t* ids, int64_t vocab_start, int64_t V_loc,
                      int64_t* sorted_ids, int64_t* order, void* workspace, int64_t workspace_bytes,
                      void* stream);

/*
 * The same gradient as cw_embed_bwd straight from the unsorted ids, in one launch and one pass over the
 * data: no token order is made first and the zeros of the rows without tokens are written by the launch
 * that sums the others (every row of d_weight is written exactly once). Replaces the whole backward of
 * the F.embedding call (parallel_1d/module.py:452, parallel_2d/module.py:353, parallel_3d/module.py:466)
 * for a batch of up to 16384 tokens whose rows are 16-byte aligned (E a multiple of the 16-byte vector).
 * A row's tokens are added in an order that the ids and the shape alone fix (the same bits on every call):
 * the row's token positions are walked in blocks of 32, round by round the lowest remaining token of every
 * block, blocks ascending (a workgroup's first row per wavefront takes its lowest token ahead of the walk).
 * That is ascending token position (the order of cw_embed_sort_ids + cw_embed_bwd, hence the same bits) when
 * no two of the row's tokens share a block of 32 positions, and another fixed order, equal up to fp32
 * reassociation, when some do. A row that more than 8 tokens select is summed over 8 contiguous ranges of
 * token positions (the same walk inside each) whose partial sums are added in order. No atomics on global
 * memory: bit-reproducible. A row that n tokens select is summed by one
 * workgroup at about 70 ns per token, so a batch dominated by one id is better served by the token order,
 * which shares a long run among several workgroups. Every workgroup scans all T ids for its 32 rows, so the
 * launch pays while a row is not much smaller than T / 4 bytes: cw_embed_bwd_ids_supported returns 1 when the
 * shapes and pointers qualify and T <= 8 row sizes in bytes (4 beyond 8192 tokens); cw_embed_bwd_ids itself
 * refuses only what it cannot do (CW_ERR_UNSUPPORTED: more than 16384 tokens, unaligned rows), and the caller
 * then goes through cw_embed_sort_ids + cw_embed_bwd.
 */
int cw_embed_bwd_ids_supported(int64_t T, int64_t E, const void* d_out, int64_t ldo, const void* d_weight,
                               int64_t ldw, int io_dtype);
int cw_embed_bwd_ids(int64_t T, int64_t E, const int64_t* ids, int64_t vocab_start, int64_t V_loc,
                     int64_t skip_row, const void* d_out, int64_t ldo, void* d_weight, int64_t ldw,
                     int io_dtype, void* stream);

/* ---- gradient-norm clipping ---------------------------------------------- */
/*
 * out2[0] = sum over tensors with groups[i] == 0 of |g|^p, out2[1] = sum over tensors with
 * groups[i] == 1 of factors[i] * |g|^p (p = norm_type; for norm_type = +inf both are maxima of |g|
 * and factors are not used). Replaces the per-tensor torch.norm(...) ** norm_type, the
 * num_partitions weighting and the two torch.stack / torch.sum of clip_grad_norm
 * (cubework/utils/clip_grad.py:31-46); group 1 = parameters tagged with NUM_PARTITIONS, whose sum
 * the caller all-reduces and divides by the tensor-parallel size (:48-49) before taking the root.
 * grads / numels / factors / groups are HOST arrays; all tensors share io_dtype and are contiguous.
 * Two deterministic stages through `workspace` (cw_multi_norm_workspace_bytes), no atomics: the first leaves
 * cw_multi_norm_partial_count (value, group) fp32 pairs at the start of `workspace`, the second combines them
 * into out2. With out2 == NULL the second stage is left out and the pairs are the result, for cw_clip_scale
 * (a caller with several dtypes gives each call the workspace address behind the previous call's pairs, so
 * that all pairs are contiguous).
 */
int64_t cw_multi_norm_workspace_bytes(int n_tensors, const int64_t* numels);
int64_t cw_multi_norm_partial_count(int n_tensors, const int64_t* numels);
int cw_multi_norm_partials(int n_tensors, const void* const* grads, const int64_t* numels,
                           const float* factors, const unsigned char* groups, float norm_type,
                           float* out2, void* workspace, int64_t workspace_bytes,
                           int io_dtype, void* stream);
/*
 * Total norm and clamped coefficient from the results of n_sets cw_multi_norm_partials calls (one per
 * dtype), `sets` = [n_sets][2] fp32 in device memory: out2[0] = (sum_i sets[i][0] + tp_scale *
 * sum_i sets[i][1]) ^ (1 / norm_type) (for +inf: the maximum of all entries), out2[1] =
 * min(max_norm / (out2[0] + 1e-6), 1). Replaces clip_grad.py:46-50,57-61 (tensor-parallel sum divided
 * by the group size, the root, clip_coef and its clamp) with one launch; a caller with a
 * tensor-parallel group larger than 1 all-reduces the second column first and passes
 * tp_scale = 1 / size.
 */
int cw_clip_coef(int n_sets, const float* sets, float tp_scale, float norm_type, float max_norm,
                 float* out2, void* stream);
/*
 * g *= coef[0] for every tensor, coef in device memory (clip_grad.py:64-68: the clamped
 * coefficient is applied without a host round trip).
 */
int cw_multi_scale(int n_tensors, void* const* grads, const int64_t* numels, const float* coef,
                   int io_dtype, void* stream);
/*
 * cw_clip_coef and cw_multi_scale in one launch (clip_grad.py:46-50,57-68): every workgroup of the scaling
 * launch combines `sets` ([n_sets][2] finished results, as for cw_clip_coef; n_sets may be 0) and `partials`
 * (n_partials unfinished (value, group) pairs left by cw_multi_norm_partials calls with out2 == NULL; may be 0)
 * in one fixed order, takes the root and the clamp, and multiplies its share of the gradients; out2 receives
 * (total norm, coefficient) as from cw_clip_coef. With partials, a clipping call that needs no exchange between
 * ranks is two launches per dtype (three beyond 2048 pairs, i.e. 134 M elements: every workgroup of the scaling launch
 * reads all pairs, so more of them are combined by one launch of their own first). out2 must not overlap sets or partials; a caller with several dtypes calls
 * it once per dtype with the same sets / partials (out2 is rewritten with the same values).
 */
int cw_clip_scale(int n_tensors, void* const* grads, const int64_t* numels, int io_dtype, int n_sets,
                  const float* sets, int64_t n_partials, const float* partials, float tp_scale,
                  float norm_type, float max_norm, float* out2, void* stream);

/* ---- attention core ------------------------------------------------------ */
/*
 * out[b, s, h, :] = softmax_j(scale * q[b,s,h,:] . k[b,j,h,:] + causal mask) . v[b,j,h,:]
 * Replaces OPTAttention.forward's scaled bmm / mask / softmax / bmm
 * (benchmark/opt/opt.py:84-117) in one pass; the probabilities are never
 * written. q, k, v are views into the qkv projection's output: element
 * (b, s, h, c) at b*stride_b + s*stride_s + h*stride_h + c (elements, unit
 * stride in c; opt.py:72-76 makes them [b, s, heads, 3*d] slices), out
 * likewise with its own strides ([b, s, heads*d] as opt.py:123-128 leaves it).
 * lse (optional, [B,H,S] fp32) receives log sum_j exp(scale * q.k_j) for the
 * backward. D = 64 or 128, CW_BF16 or CW_F16 in this build (CW_ERR_UNSUPPORTED
 * else); token strides below 2^23 elements.
 */
int cw_attn_fwd(int64_t B, int64_t H, int64_t S, int64_t D,
                const void* q, const void* k, const void* v,
                int64_t stride_b, int64_t stride_s, int64_t stride_h,
                float scale, int causal,
                void* out, int64_t out_stride_b, int64_t out_stride_s, int64_t out_stride_h,
                float* lse, int io_dtype, void* stream);

/*
 * Backward of cw_attn_fwd: dq, dk, dv from q, k, v, out, d_out and the forward's lse; what
 * autograd derives for benchmark/opt/opt.py:84-117 (bmm, mask, softmax, bmm), with the
 * probabilities recomputed instead of saved. out / d_out share one set of strides, dq / dk /
 * dv another (e.g. the three slices of one [b, s, heads, 3*d] gradient buffer, so that the
 * gradient of the qkv projection's output needs no concatenation). workspace:
 * cw_attn_bwd_workspace_bytes(B, H, S) bytes. No atomics: bit-reproducible.
 */
int64_t cw_attn_bwd_workspace_bytes(int64_t B, int64_t H, int64_t S);
int cw_attn_bwd(int64_t B, int64_t H, int64_t S, int64_t D,
                const void* q, const void* k, const void* v,
                int64_t stride_b, int64_t stride_s, int64_t stride_h,
                const void* out, const void* d_out,
                int64_t out_stride_b, int64_t out_stride_s, int64_t out_stride_h,
                const float* lse, float scale, int causal,
                void* dq, void* dk, void* dv,
                int64_t grad_stride_b, int64_t grad_stride_s, int64_t grad_stride_h,
                void* workspace, int64_t workspace_bytes, int io_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CUBEWORK_HIP_H */
