// Implicit-GEMM convolution: the A * B^T kernel of gemm_mfma_kernel.h with the A operand gathered
// from the image tensor (ConvInner), with and without the bias row in the epilogue.
#include "gemm_mfma_kernel.h"

namespace dragon {

hipError_t gemm_launch_conv(const GemmParams& p, int tile, hipStream_t stream) {
    if (gemm_tile_is_streamk(tile)) {
        // where the convolution cannot take the balanced kernel (channels no multiple of 32, a capturing stream,
        // a very large image) a tile-per-workgroup kernel takes over
        const hipError_t e = gemm_launch_streamk_conv(p, tile, stream);
        if (e != hipErrorOutOfMemory) return e;
        (void)hipGetLastError();
        const int num_cu = gemm_device_num_cu();
        if (num_cu <= 0) return hipErrorNoDevice;
        tile = gemm_choose_tile_per_workgroup(p.rows, p.cols, 1, p.k_total, num_cu) & ~TILE_PAIRED;
        if (gemm_tile_is_dma(tile))
            tile = (tile == TILE_DMA_128x128_S4) ? TILE_128x128 : (tile == TILE_DMA_64x64_S4) ? TILE_64x64 : TILE_64x64_K32;
    }
    if (tile < 0 || gemm_tile_is_dma(tile & ~TILE_PAIRED)) return hipErrorInvalidValue;
    if (p.bias != nullptr) return launch_variant<true, true, true, true>(p, tile, stream);
    return launch_variant<true, true, false, true>(p, tile, stream);
}

}  // namespace dragon
