// C = A*B + bias row in one launch: the NN product of gemm_mfma_kernel.h with the bias added in
// the epilogue, in every tile shape.
#include "gemm_mfma_kernel.h"

namespace dragon {

hipError_t gemm_launch_nn_biased(const GemmParams& p, int tile, hipStream_t stream) {
    if (gemm_tile_is_dma(tile)) return launch_variant_dma<true, false, true>(p, tile, stream);
    return launch_variant<true, false, true>(p, tile, stream);
}

}  // namespace dragon
