// Host side of the block-GEMM entry points: argument checks of cw_gemm_ksteps(_ws) and the scratch size they
// ask for. The other entry points live beside their kernels; error text and device checks in cw_runtime.hip.
#include "cw_common.h"
#include "gemm_plan.h"

using namespace cw;

extern "C" int64_t cw_gemm_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps, int io_dtype) {
    return gemm_workspace_bytes(layout, M, N, K, n_steps, io_dtype);
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
    GemmArgs args;
    bool nothing_to_do = false;
    if (const int rc = gemm_prepare_args(layout, M, N, K, n_steps, A_steps, lda, B_steps, ldb, bias, epilogue, C, ldc, preact,
                                         ldp, addends, n_addends, ldadd, workspace, workspace_bytes, io_dtype, &args,
                                         &nothing_to_do);
        rc != CW_OK || nothing_to_do)
        return rc;
    if (const int drc = require_gfx950("cw_gemm_ksteps_ws"); drc != CW_OK) return drc;
    hipStream_t s = (hipStream_t)stream;
    return io_dtype == CW_F32 ? gemm_f32_launch(args, layout, epilogue, s)
                              : gemm_half_launch(args, layout, epilogue, io_dtype == CW_F16, s);
}
