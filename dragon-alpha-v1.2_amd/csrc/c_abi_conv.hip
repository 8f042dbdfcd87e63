// C ABI of the forward convolution (declared in include/dragon_hip_conv.h): argument checks and
// the mapping of the convolution geometry onto the implicit-GEMM launch.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/dragon_hip_conv.h"
#include "../../include/dragon_hip_gemm.h"
#include "gemm_mfma.h"
#include "runtime_internal.h"

using namespace dragon;

namespace {

inline bool aligned16(int64_t a) { return (a & 15) == 0; }

int conv_forward(const int64_t* streams, int length, int64_t dX, int IH, int IW, int64_t dW, int FH, int FW,
                 int64_t dY, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                 int64_t dBias = 0, int lengthv = 0, int width = 0) {
    if (streams == nullptr || length < 1 || length > 10) return hipErrorInvalidValue;
    if (dX == 0 || dW == 0 || dY == 0 || !aligned16(dX) || !aligned16(dW) || !aligned16(dY))
        return hipErrorInvalidValue;
    if (IH <= 0 || IW <= 0 || FH <= 0 || FW <= 0 || OH <= 0 || OW <= 0 || N <= 0 || IC <= 0 || OC <= 0 ||
        sh <= 0 || sw <= 0 || ph < 0 || pw < 0 || (IC & 3) || (OC & 3))
        return hipErrorInvalidValue;
    const long long GM = (long long)N * OH * OW, GK = (long long)FH * FW * IC;
    const long long sizeX = (long long)N * IH * IW * IC;
    if (GM > 0x7fffffffLL || GK >= (1LL << 24) || sizeX >= (1LL << 29) || GM * OC > 0x7fffffffLL)
        return hipErrorInvalidValue;
    split_ledger_touch((const void*)(intptr_t)dY, (size_t)(GM * OC) * 4);
    GemmParams p = {};
    p.A = (const float*)(intptr_t)dX;
    p.B = (const float*)(intptr_t)dW;
    p.C = (float*)(intptr_t)dY;
    p.rows = (int)GM; p.cols = OC; p.k_total = (int)GK;
    p.lda = (int)GK; p.a_outer = (int)GM; p.a_inner = (int)GK;     // A exists only as a gather
    p.ldb = (int)GK; p.b_outer = OC; p.b_inner = (int)GK;
    p.ldc = OC;
    p.nz = 1;
    p.cv_IH = IH; p.cv_IW = IW; p.cv_IC = IC; p.cv_FW = FW; p.cv_OH = OH; p.cv_OW = OW;
    p.cv_sh = sh; p.cv_sw = sw; p.cv_ph = ph; p.cv_pw = pw;
    p.cv_rcp_IC = 1.0f / (float)IC;
    p.cv_rcp_FW = 1.0f / (float)FW;
    p.cv_walk = 1;
    if (dBias != 0) {
        if (!aligned16(dBias) || width <= 0 || width > OC || lengthv <= 0 || lengthv % OC != 0 ||
            lengthv / OC > GM)
            return hipErrorInvalidValue;
        p.bias = (const float*)(intptr_t)dBias;
        p.bias_rows = lengthv / OC;
        p.bias_width = width;
    }
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    // A 1 x 1 filter at stride 1 without padding gathers nothing: Y[N*IH*IW][OC] = X[N*IH*IW][IC] * W[OC][IC]^T is the
    // plain A * B^T product, whose loaders have no tap arithmetic (128 x 32 x 32 x 256 -> 256: 137 -> 131 us).
    if (FH == 1 && FW == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && OH == IH && OW == IW &&
        gemm_forced_tile() == TILE_AUTO) {
        GemmParams q = {};
        q.A = p.A; q.B = p.B; q.C = p.C;
        q.rows = (int)GM; q.cols = OC; q.k_total = IC;
        q.lda = IC; q.a_outer = (int)GM; q.a_inner = IC;
        q.ldb = IC; q.b_outer = OC; q.b_inner = IC;
        q.ldc = OC;
        q.nz = 1;
        if (dBias == 0)
            return gemm_launch(GEMM_T2, q, gemm_choose_tile(q.rows, q.cols, 1, q.k_total, num_cu, GEMM_T2), (hipStream_t)(intptr_t)streams[0]);
        // with a bias row: the tile-per-workgroup kernels' epilogue (the shapes that stage through registers)
        q.bias = p.bias; q.bias_rows = p.bias_rows; q.bias_width = p.bias_width;
        const int t = gemm_choose_tile_per_workgroup(q.rows, q.cols, 1, q.k_total, num_cu, GEMM_T2);
        if (!gemm_tile_is_dma(t & ~TILE_PAIRED) && (t & ~TILE_PAIRED) <= TILE_64x128_K32)
            return gemm_launch_t2_biased(q, t, (hipStream_t)(intptr_t)streams[0]);
    }
    int tile = gemm_forced_tile() != TILE_AUTO ? gemm_forced_tile() : gemm_choose_tile_per_workgroup(p.rows, p.cols, 1, p.k_total, num_cu);
    const bool free_choice = gemm_forced_tile() == TILE_AUTO;   // a forced shape (tests, sweeps) is taken as it is
    if (free_choice) tile &= ~TILE_PAIRED;   // decided below, on the convolution's own measurements
    if (gemm_tile_is_dma(tile)) {   // the direct-to-LDS shapes have no gathering loader: nearest classic shape
        tile = (tile == TILE_DMA_128x128_S4) ? TILE_128x128 : (tile == TILE_DMA_64x64_S4) ? TILE_64x64 : TILE_64x64_K32;
    }
    // the stage depth is decided below, where the channel count is known: back to the 16-k shapes first
    if (free_choice)
        tile = tile == TILE_128x128_K32 ? TILE_128x128 : tile == TILE_128x64_K32 ? TILE_128x64
             : tile == TILE_64x128_K32 ? TILE_64x128 : tile;
    // 256 gathered rows per workgroup cost the loader four rows' worth of registers per lane and the
    // kernel spills; 128 x 64 measures the same or better on every layer tried
    if (free_choice && tile == TILE_256x64) tile = TILE_128x64;
    // a gathered row of A costs the loader more than a row of W: of the two 8192-element shapes take the
    // one with fewer A rows when the filters fill it
    if (free_choice && tile == TILE_128x64 && OC > 64) tile = TILE_64x128;
    // 32 k per stage halve the per-stage instructions; worth it while the larger LDS footprint does not
    // cost co-resident workgroups (2 of 128x128, 3 of the 8192-element shapes fit a compute unit)
    if (free_choice && (IC & 31) == 0) {
        const int bm = (tile == TILE_128x128 || tile == TILE_128x64) ? 128 : 64;
        const int bn = (tile == TILE_128x128 || tile == TILE_64x128) ? 128 : 64;
        const long long tiles = ((GM + bm - 1) / bm) * ((OC + bn - 1) / bn);
        const long long per_cu = (tiles + num_cu - 1) / num_cu;
        if (tile == TILE_128x128 && per_cu <= 2) tile = TILE_128x128_K32;
        else if (tile == TILE_64x128 && per_cu <= 3) tile = TILE_64x128_K32;
        else if (tile == TILE_128x64 && per_cu <= 3) tile = TILE_128x64_K32;
    }
    // the paired-stage form pays later here than in the plain products (the gathering loader needs the
    // registers): 3-5 % faster on 7x7x64 and 3x3x512 filters, 4-8 % slower on 3x3x64 and 1x1x256
    if (free_choice && GK >= 3072 && tile != TILE_256x64 && tile != TILE_64x256) tile |= TILE_PAIRED;
    // Large layers whose output channels fill 128-wide tiles take the balanced kernel (the gather staged straight
    // into LDS, a filter tap at a time; channels in multiples of 32): 3x3 layers with 128 ... 512 channels 5 - 13 %
    // faster (290 -> 276, 298 -> 267, 302 -> 263 us), level for a K below 768, and behind with 64 output
    // channels, where its 128 x 64 tiles lose to the paired tile-per-workgroup kernel (823 against 782 us on the
    // 7x7 layer).  gemm_launch_conv falls back where the stream has no workspace and may not make one.
    // Where the products' choice for this shape is one of the balanced kernel's smaller tiles (fewer 128 x 128 tiles
    // than compute units: 128 images of 7 x 7 with 512 -> 512 channels, 196 tiles), that tile is taken as well from
    // K = 768 on and more than 64 output channels: 298 -> 217 - 222 us on that layer.
    const int sk = (free_choice && (IC & 31) == 0 && FH <= 32 && FW <= 32)
                       ? gemm_choose_streamk(p.rows, p.cols, 1, p.k_total, num_cu, GEMM_T2) : -1;
    const int sk_conv = sk == TILE_SK_128x64_O2 ? TILE_SK_128x64 : sk == TILE_SK_64x64_O2 ? TILE_SK_64x64 : sk;
    if (sk == TILE_SK_128x128)
        tile = TILE_SK_128x128;
    else if (OC > 64 && GK >= 768 && (sk_conv == TILE_SK_128x64 || sk_conv == TILE_SK_64x128 || sk_conv == TILE_SK_64x64))
        tile = sk_conv;
    // ... and with up to 64 output channels the 256 x 64 shape of the same kernel, which has the 128 x 128 tile's
    // ratio of matrix work to LDS traffic (the 7x7 layer of the reference's speed test: 784 -> 767 us; 3x3 layers
    // with 64 -> 64 channels, K = 576: 139 -> 131 and 257 -> 241 us)
    else if (free_choice && (IC & 31) == 0 && FH <= 32 && FW <= 32 && OC <= 64 && OC > 32 && GK >= 576 &&
             (GM + 255) / 256 >= num_cu && (GM + 255) / 256 <= 65536)
        tile = TILE_SK_256x64;
    return gemm_launch_conv(p, tile, (hipStream_t)(intptr_t)streams[0]);
}

}  // namespace

extern "C" {

int dragon_Cuda_conv3D_conv3D(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW, int64_t dW,
                              int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC,
                              int32_t OC, int32_t sh, int32_t sw, int32_t ph, int32_t pw) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int dragon_Cuda_conv3D_conv3D_texture(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                      int64_t dW, int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW,
                                      int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw, int32_t ph,
                                      int32_t pw) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int dragon_Cuda_conv3D_conv3D_np(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW, int64_t dW,
                                 int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW, int32_t N,
                                 int32_t IC, int32_t OC, int32_t sh, int32_t sw) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, 0, 0);
}
int dragon_Cuda_conv3D_conv3D_W1(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW, int64_t dW,
                                 int64_t dY, int32_t N, int32_t IC, int32_t OC) {
    return conv_forward(s, n, dX, IH, IW, dW, 1, 1, dY, IH, IW, N, IC, OC, 1, 1, 0, 0);
}
int dragon_Cuda_conv3D_conv3DV2(int32_t, const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                int64_t dW, int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW,
                                int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw, int32_t ph,
                                int32_t pw) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int dragon_Cuda_conv3D_kernel_remode(int64_t stream, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
                                     int32_t OC, int32_t IC) {
    if (FH <= 0 || FW <= 0 || OC <= 0 || IC <= 0 || (IC & 3) || (OC & 3)) return hipErrorInvalidValue;
    const long long GK = (long long)FH * FW * IC;
    if (GK * OC > 0x7fffffffLL) return hipErrorInvalidValue;
    // W[OC][GK] -> CW[GK][OC]: a 2-D transpose, both row lengths multiples of 4
    return dragon_Cuda_expk2_transpose2D(stream, dW, dCW, (int32_t)GK, OC, (int32_t)GK, OC, (int32_t)(GK * OC));
}
int dragon_Cuda_conv3D_conv3D_GemmR(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW, int64_t dW,
                                    int64_t, int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW,
                                    int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw, int32_t ph,
                                    int32_t pw) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int dragon_Cuda_conv3D_conv3D_GemmR_SGM(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                        int64_t dW, int64_t, int32_t FH, int32_t FW, int64_t dY, int32_t OH,
                                        int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw,
                                        int32_t ph, int32_t pw, int32_t) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int dragon_Cuda_conv3D_conv3D_GemmR_texture(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                            int64_t dW, int64_t, int32_t FH, int32_t FW, int64_t dY, int32_t OH,
                                            int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh,
                                            int32_t sw, int32_t ph, int32_t pw) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int dragon_Cuda_conv3D_conv3D_GemmR_texture_SGM(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                                int64_t dW, int64_t, int32_t FH, int32_t FW, int64_t dY,
                                                int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC,
                                                int32_t sh, int32_t sw, int32_t ph, int32_t pw, int32_t) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int dragon_Cuda_conv3D_conv3D_GemmR_W1(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                       int64_t dW, int64_t, int64_t dY, int32_t N, int32_t IC, int32_t OC) {
    return conv_forward(s, n, dX, IH, IW, dW, 1, 1, dY, IH, IW, N, IC, OC, 1, 1, 0, 0);
}
int dragon_Cuda_conv3D_conv3D_GemmR_W1_SGM(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                           int64_t dW, int64_t, int64_t dY, int32_t N, int32_t IC, int32_t OC,
                                           int32_t) {
    return conv_forward(s, n, dX, IH, IW, dW, 1, 1, dY, IH, IW, N, IC, OC, 1, 1, 0, 0);
}
int dragon_Cuda_conv3D_conv3D_GemmV2R(int32_t, const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW,
                                      int64_t dW, int64_t, int32_t FH, int32_t FW, int64_t dY, int32_t OH,
                                      int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw,
                                      int32_t ph, int32_t pw) {
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
#define DRAGON_WINOGRAD(name, extra_decl)                                                                     \
    int name(int32_t, const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW, int64_t dW, int64_t,    \
             int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC,     \
             int32_t ph, int32_t pw extra_decl) {                                                              \
        const int e = conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, 1, 1, ph, pw);          \
        return e ? -e : 1;                                                                                     \
    }
#define DRAGON_COMMA_INT , int32_t
DRAGON_WINOGRAD(dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s8_R_texture, )
DRAGON_WINOGRAD(dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s8_texture_SGM, DRAGON_COMMA_INT)
DRAGON_WINOGRAD(dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s16_R_texture, )
DRAGON_WINOGRAD(dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s16_texture_SGM, DRAGON_COMMA_INT)
#undef DRAGON_WINOGRAD
#undef DRAGON_COMMA_INT

int dragon_Cuda_conv3D_conv3D_biased(const int64_t* s, int32_t n, int64_t dX, int32_t IH, int32_t IW, int64_t dW,
                                     int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW, int32_t N,
                                     int32_t IC, int32_t OC, int32_t sh, int32_t sw, int32_t ph, int32_t pw,
                                     int64_t dBias, int32_t lengthv, int32_t width) {
    if (dBias == 0) return hipErrorInvalidValue;
    return conv_forward(s, n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw, dBias, lengthv, width);
}

}  // extern "C"
