// bf16 block GEMM: choice of kernel and tile configuration.
//   - large tile-aligned problems (>= 128 tiles of 256x256, K a multiple of 64,
//     16-byte aligned rows, at most 4 k-steps and 2 addends): the LDS-DMA
//     kernel (gemm_bf16_dma.h);
//   - everything else: the register-staged kernel (gemm_bf16_kernel.h), with
//     256x256 or 128x128 tiles, guarded when the shape is ragged or unaligned.
// CW_GEMM_IMPL=staged in the environment forces the register-staged kernel.
#include <cstdlib>
#include <cstring>

#include "gemm_bf16_kernel.h"

namespace cw {

int gemm_bf16_dma_launch_nn(const GemmArgs& args, int epilogue, hipStream_t s);
int gemm_bf16_dma_launch_nt(const GemmArgs& args, int epilogue, hipStream_t s);
int gemm_bf16_dma_launch_tn(const GemmArgs& args, int epilogue, hipStream_t s);

static bool dma_kernel_enabled() {
    static const bool enabled = [] {
        const char* v = std::getenv("CW_GEMM_IMPL");
        return !(v != nullptr && std::strcmp(v, "staged") == 0);
    }();
    return enabled;
}

int gemm_bf16_launch(const GemmArgs& args, int layout, int epilogue, hipStream_t s) {
    // the unguarded kernels address operands with 32-bit byte offsets
    const int64_t max_dim = args.M > args.N ? (args.M > args.K ? args.M : args.K) : (args.N > args.K ? args.N : args.K);
    const bool fits32 = (max_dim + 64) * (args.lda > args.ldb ? args.lda : args.ldb) * 2 < ((int64_t)1 << 32);
    const bool all_vec = fits32 && args.vec_a && args.vec_b && args.vec_c && (args.preact == nullptr || args.vec_p) &&
                         (args.bias == nullptr || args.vec_bias) && (args.n_addends == 0 || args.vec_add);
    const int64_t tiles256 = (int64_t)((args.M + 255) / 256) * ((args.N + 255) / 256);
    const bool big = tiles256 >= 128;
    const int tile = big ? 256 : 128;
    const bool exact = all_vec && (args.M % tile) == 0 && (args.N % tile) == 0 && (args.K % gemm_bf16::kBK) == 0;
    if (big && exact && args.n_steps > 0 && args.n_steps <= kRingMaxSteps && args.n_addends <= kRingMaxAddends &&
        dma_kernel_enabled()) {
        switch (layout) {
            case CW_NN: return gemm_bf16_dma_launch_nn(args, epilogue, s);
            case CW_NT: return gemm_bf16_dma_launch_nt(args, epilogue, s);
            case CW_TN: return gemm_bf16_dma_launch_tn(args, epilogue, s);
            default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
        }
    }
    switch (layout) {
        case CW_NN: return gemm_bf16_launch_nn(args, epilogue, big, exact, s);
        case CW_NT: return gemm_bf16_launch_nt(args, epilogue, big, exact, s);
        case CW_TN: return gemm_bf16_launch_tn(args, epilogue, big, exact, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    }
}

}  // namespace cw
