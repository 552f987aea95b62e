// fp16 block GEMM, orientation TN (C += A[K,M]^T * B[K,N]: both operands are transposed on their way to LDS).
#include "gemm_bf16_kernel.h"

namespace cw {

int gemm_f16_launch_tn(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s) {
    return gemm_bf16::launch_orientation<true, true, f16_t>(args, epilogue, big, exact, s);
}

}  // namespace cw
