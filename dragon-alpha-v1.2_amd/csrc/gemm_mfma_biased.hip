// C = A*B + bias row in one launch: the NN product of gemm_mfma_kernel.h with the bias added in
// the epilogue, in every tile shape; and the same for A*B^T.
#include "gemm_mfma_kernel.h"

namespace dragon {

hipError_t gemm_launch_nn_biased(const GemmParams& p, int tile, hipStream_t stream) {
    if (gemm_tile_is_dma(tile)) return launch_variant_dma<true, false, true>(p, tile, stream);
    return launch_variant<true, false, true>(p, tile, stream);
}

// C = A*B^T + bias row: what a 1 x 1 convolution with a bias is (tile-per-workgroup shapes that stage through registers)
hipError_t gemm_launch_t2_biased(const GemmParams& p, int tile, hipStream_t stream) {
    if (tile < 0 || gemm_tile_is_dma(tile & ~TILE_PAIRED) || (tile & ~TILE_PAIRED) > TILE_64x128_K32) return hipErrorInvalidValue;
    return launch_variant<true, true, true>(p, tile, stream);
}

}  // namespace dragon
