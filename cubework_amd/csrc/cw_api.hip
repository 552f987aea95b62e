// Host side of the block-GEMM entry points: argument checks of cw_gemm_ksteps(_ws) and the scratch size they
// ask for. The other entry points live beside their kernels; error text and device checks in cw_runtime.hip.
#include <cstring>

#include "cw_common.h"
#include "gemm.h"

using namespace cw;

extern "C" int64_t cw_gemm_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps, int io_dtype) {
    if (layout != CW_NN && layout != CW_NT && layout != CW_TN) return 0;
    if (io_dtype != CW_BF16 && io_dtype != CW_F16) return 0;  // the fp32 GEMM is not split
    const int slices = gemm_bf16_split_slices(M, N, K, n_steps);
    if (slices > 1) {
        // shapes the 128 x 128 ring kernel takes in preference to the split (gemm_half_launch) need none
        const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
        if (tiles128 >= 192 && K * n_steps < 12288) return 0;
        return (int64_t)slices * M * N * (int64_t)sizeof(float);
    }
    return gemm_bf16_ktail_workspace_bytes(layout, M, N, K, n_steps);
}

extern "C" int cw_gemm_ksteps(int layout, int64_t M, int64_t N, int64_t K, int n_steps, const void* const* A_steps,
                              int64_t lda, const void* const* B_steps, int64_t ldb, const void* bias, int epilogue,
                              void* C, int64_t ldc, void* preact, int64_t ldp, const void* const* addends,
                              int n_addends, int64_t ldadd, int io_dtype, void* stream) {
    return cw_gemm_ksteps_ws(layout, M, N, K, n_steps, A_steps, lda, B_steps, ldb, bias, epilogue, C, ldc, preact, ldp,
                             addends, n_addends, ldadd, nullptr, 0, io_dtype, stream);
}

extern "C" int cw_gemm_ksteps_ws(int layout, int64_t M, int64_t N, int64_t K, int n_steps,
                                 const void* const* A_steps, int64_t lda, const void* const* B_steps, int64_t ldb,
                                 const void* bias, int epilogue, void* C, int64_t ldc, void* preact, int64_t ldp,
                                 const void* const* addends, int n_addends, int64_t ldadd, void* workspace,
                                 int64_t workspace_bytes, int io_dtype, void* stream) {
    if (layout != CW_NN && layout != CW_NT && layout != CW_TN)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    if (epilogue < CW_EPI_NONE || epilogue > CW_EPI_BIAS_RELU)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad io_dtype %d", io_dtype);
    if (M < 0 || N < 0 || K < 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                    (long long)K);
    if (n_steps < 0 || n_steps > CW_MAX_KSTEPS)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: n_steps=%d outside [0, %d]", n_steps, CW_MAX_KSTEPS);
    if (n_addends < 0 || n_addends > CW_MAX_ADDENDS)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: n_addends=%d outside [0, %d]", n_addends, CW_MAX_ADDENDS);
    if (M == 0 || N == 0) return CW_OK;
    if (C == nullptr || ldc < N) return fail(CW_ERR_INVALID, "cw_gemm_ksteps: C is NULL or ldc < N");
    if (preact != nullptr && ldp < N) return fail(CW_ERR_INVALID, "cw_gemm_ksteps: ldp < N");
    if (K == 0) n_steps = 0;
    if (n_steps > 0) {
        if (A_steps == nullptr || B_steps == nullptr)
            return fail(CW_ERR_INVALID, "cw_gemm_ksteps: operand pointer tables are NULL");
        const int64_t a_cols = (layout == CW_TN) ? M : K;  // contiguous extent of A's rows
        const int64_t b_cols = (layout == CW_NT) ? K : N;
        if (lda < a_cols || ldb < b_cols)
            return fail(CW_ERR_INVALID, "cw_gemm_ksteps: leading dimension smaller than the row (lda=%lld ldb=%lld)",
                        (long long)lda, (long long)ldb);
    }
    if (n_addends > 0 && (addends == nullptr || ldadd < N))
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: addends table is NULL or ldadd < N");

    GemmArgs args;
    memset(&args, 0, sizeof(args));
    const int vec = (io_dtype == CW_F32) ? 4 : 8;        // elements per 16 bytes
    const uintptr_t out_mask = 15u;                      // outputs / addends move 16 bytes at a time
    const int out_vec = (io_dtype == CW_F32) ? 4 : 8;    // elements per 16 bytes
    args.vec_a = args.vec_b = 1;
    for (int i = 0; i < n_steps; ++i) {
        if (A_steps[i] == nullptr || B_steps[i] == nullptr)
            return fail(CW_ERR_INVALID, "cw_gemm_ksteps: operand pointer of step %d is NULL", i);
        args.A[i] = A_steps[i];
        args.B[i] = B_steps[i];
        if (!aligned16(A_steps[i])) args.vec_a = 0;
        if (!aligned16(B_steps[i])) args.vec_b = 0;
    }
    if (lda % vec != 0) args.vec_a = 0;
    if (ldb % vec != 0) args.vec_b = 0;
    args.vec_add = 1;
    for (int j = 0; j < n_addends; ++j) {
        if (addends[j] == nullptr) return fail(CW_ERR_INVALID, "cw_gemm_ksteps: addend %d is NULL", j);
        args.addend[j] = addends[j];
        if ((reinterpret_cast<uintptr_t>(addends[j]) & out_mask) != 0) args.vec_add = 0;
    }
    if (ldadd % out_vec != 0) args.vec_add = 0;
    args.bias = bias;
    args.vec_bias = (bias == nullptr || (reinterpret_cast<uintptr_t>(bias) & 7u) == 0) ? 1 : 0;
    args.C = C;
    args.vec_c = ((reinterpret_cast<uintptr_t>(C) & out_mask) == 0 && ldc % out_vec == 0) ? 1 : 0;
    args.preact = preact;
    args.vec_p = (preact == nullptr || ((reinterpret_cast<uintptr_t>(preact) & out_mask) == 0 && ldp % out_vec == 0)) ? 1 : 0;
    args.lda = lda;
    args.ldb = ldb;
    args.ldc = ldc;
    args.ldp = ldp;
    args.ldadd = ldadd;
    args.M = (int)M;
    args.N = (int)N;
    args.K = (int)K;
    args.n_steps = n_steps;
    args.n_addends = n_addends;
    args.workspace = workspace_bytes > 0 ? workspace : nullptr;
    args.workspace_bytes = workspace != nullptr ? workspace_bytes : 0;
    if (const int drc = require_gfx950("cw_gemm_ksteps_ws"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return io_dtype == CW_F32 ? gemm_f32_launch(args, layout, epilogue, s)
                              : gemm_half_launch(args, layout, epilogue, io_dtype == CW_F16, s);
}
