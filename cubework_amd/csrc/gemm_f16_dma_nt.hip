// fp16 block GEMM, LDS-DMA kernel, orientation NT.
#include "gemm_bf16_dma.h"

namespace cw {

int gemm_f16_dma_launch_nt(const GemmArgs& args, int epilogue, hipStream_t s, const void* tail_a, const void* tail_b) {
    return gemm_dma::launch_dma<false, false, f16_t>(args, epilogue, s, tail_a, tail_b);
}

int gemm_f16_dma_split_launch_nt(const GemmArgs& args, int slices, hipStream_t s) {
    return gemm_dma::launch_dma_split<false, false, f16_t>(args, slices, s);
}

}  // namespace cw
