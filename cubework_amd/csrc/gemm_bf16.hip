// bf16 block GEMM: choice of tile configuration and kernel variant.
#include "gemm_bf16_kernel.h"

namespace cw {

int gemm_bf16_launch(const GemmArgs& args, int layout, int epilogue, hipStream_t s) {
    // the unguarded kernels address operands with 32-bit byte offsets
    const int64_t max_dim = args.M > args.N ? (args.M > args.K ? args.M : args.K) : (args.N > args.K ? args.N : args.K);
    const bool fits32 = (max_dim + 64) * (args.lda > args.ldb ? args.lda : args.ldb) * 2 < ((int64_t)1 << 32);
    const bool all_vec = fits32 && args.vec_a && args.vec_b && args.vec_c && (args.preact == nullptr || args.vec_p) &&
                         (args.bias == nullptr || args.vec_bias) && (args.n_addends == 0 || args.vec_add);
    // Large problems: 256x256 tiles (one per CU at 8192x2048). Small ones: 128x128.
    const int64_t tiles256 = (int64_t)((args.M + 255) / 256) * ((args.N + 255) / 256);
    const bool big = tiles256 >= 128;
    const int tile = big ? 256 : 128;
    const bool exact = all_vec && (args.M % tile) == 0 && (args.N % tile) == 0 && (args.K % gemm_bf16::kBK) == 0;
    switch (layout) {
        case CW_NN: return gemm_bf16_launch_nn(args, epilogue, big, exact, s);
        case CW_NT: return gemm_bf16_launch_nt(args, epilogue, big, exact, s);
        case CW_TN: return gemm_bf16_launch_tn(args, epilogue, big, exact, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

}  // namespace cw
