// fp16 block GEMM, orientation NN (C += A[M,K] * B[K,N]: B is transposed on its way to LDS).
#include "gemm_bf16_kernel.h"

namespace cw {

int gemm_f16_launch_nn(const GemmArgs& args, int epilogue, bool big, bool exact, hipStream_t s) {
    return gemm_bf16::launch_orientation<false, true, f16_t>(args, epilogue, big, exact, s);
}

}  // namespace cw
