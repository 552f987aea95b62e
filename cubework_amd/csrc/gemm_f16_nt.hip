// fp16 block GEMM, orientation NT (C += A[M,K] * B[N,K]^T: both operands are k-contiguous).
#include "gemm_bf16_kernel.h"

namespace cw {

int gemm_f16_launch_nt(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s) {
    return gemm_bf16::launch_orientation<false, false, f16_t>(args, epilogue, big, exact, s);
}

}  // namespace cw
