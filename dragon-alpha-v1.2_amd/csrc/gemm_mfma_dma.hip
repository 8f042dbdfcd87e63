// The three products through the direct-to-LDS kernel of gemm_mfma_kernel.h, in its tile shapes.
#include "gemm_mfma_kernel.h"

namespace dragon {

hipError_t gemm_launch_dma(int variant, const GemmParams& p, int tile, hipStream_t stream) {
    switch (variant) {
        case GEMM_NN: return launch_variant_dma<true, false, false>(p, tile, stream);
        case GEMM_T1: return launch_variant_dma<false, false, false>(p, tile, stream);
        case GEMM_T2: return launch_variant_dma<true, true, false>(p, tile, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace dragon
