// Implicit-GEMM convolution: the A * B^T kernel of gemm_mfma_kernel.h with the A operand gathered
// from the image tensor (ConvInner), with and without the bias row in the epilogue.
#include "gemm_mfma_kernel.h"

namespace dragon {

hipError_t gemm_launch_conv(const GemmParams& p, int tile, hipStream_t stream) {
    if (tile < 0 || gemm_tile_is_dma(tile & ~TILE_PAIRED)) return hipErrorInvalidValue;
    if (p.bias != nullptr) return launch_variant<true, true, true, true>(p, tile, stream);
    return launch_variant<true, true, false, true>(p, tile, stream);
}

}  // namespace dragon
