/*
 * dragon_hip_conv.h -- C ABI of the forward convolution Y = conv3D(X, W) on gfx950, computed as an
 * implicit GEMM on the FP32 matrix cores: Y[N*OH*OW, OC] = A[N*OH*OW, FH*FW*IC] * W[OC, FH*FW*IC]^T
 * where row (n, oh, ow), column (fh, fw, ic) of A is X[n, oh*sh - ph + fh, ow*sw - pw + fw, ic] (zero in
 * the padding) and is gathered on the fly, never stored.
 *
 * Each entry point takes the argument list of one `static native` method of the reference's
 * z.dragon.engine.cuda.impl.math.Cuda_conv3D class (alpha-Dragon-v1.2/src/z/dragon/engine/cuda/impl/math/
 * Cuda_conv3D.java; native side engine-cuda-base/Cuda_conv3D/Cuda_conv3D/A.cu), minus (JNIEnv*, jclass):
 * jlong -> int64_t, jint -> int32_t, jboolean -> int32_t, jlongArray -> const int64_t*.  They return the
 * hipError_t value as int (0 = success; 1 = invalid argument), the boolean natives 1 = "done" or a
 * negative hipError_t.
 *
 * Layout (the reference's): X[N, IH, IW, IC], W[OC, FH, FW, IC], Y[N, OH, OW, OC], row-major FP32, IC and
 * OC multiples of 4 (caller-padded with zeros), N as allocated (a multiple of 4; the images beyond the
 * logical batch are zeros and produce zeros).  Limits: FH*FW*IC < 2^24, X below 2^29 floats.  Work is
 * issued on streams[0]; the other handles stay idle (1 <= length <= 10).  Y is overwritten.
 *
 * The reference picks among a dozen kernels families by shape (plain / texture / no-padding / 1x1 /
 * "V2" / re-ordered filter "GemmR" / im2col-Winograd); all of them compute the same function, and all of
 * these entries run the same kernel.  The re-ordered filter CW that the GemmR and Winograd natives also
 * receive is not read (W is used as it is stored), but kernel_remode still produces it.
 */
#ifndef DRAGON_HIP_CONV_H
#define DRAGON_HIP_CONV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Cuda_conv3D.java:441 conv3D, :519 conv3D_texture */
int dragon_Cuda_conv3D_conv3D(const int64_t* streams, int32_t length, int64_t dX, int32_t IH, int32_t IW,
                              int64_t dW, int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW,
                              int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw, int32_t ph, int32_t pw);
int dragon_Cuda_conv3D_conv3D_texture(const int64_t* streams, int32_t length, int64_t dX, int32_t IH,
                                      int32_t IW, int64_t dW, int32_t FH, int32_t FW, int64_t dY, int32_t OH,
                                      int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw,
                                      int32_t ph, int32_t pw);
/* :566 conv3D_np -- no padding */
int dragon_Cuda_conv3D_conv3D_np(const int64_t* streams, int32_t length, int64_t dX, int32_t IH, int32_t IW,
                                 int64_t dW, int32_t FH, int32_t FW, int64_t dY, int32_t OH, int32_t OW,
                                 int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw);
/* :616 conv3D_W1 -- 1x1 filter, stride 1, no padding: OH = IH, OW = IW */
int dragon_Cuda_conv3D_conv3D_W1(const int64_t* streams, int32_t length, int64_t dX, int32_t IH, int32_t IW,
                                 int64_t dW, int64_t dY, int32_t N, int32_t IC, int32_t OC);
/* :685 conv3DV2 */
int dragon_Cuda_conv3D_conv3DV2(int32_t useTexture, const int64_t* streams, int32_t length, int64_t dX,
                                int32_t IH, int32_t IW, int64_t dW, int32_t FH, int32_t FW, int64_t dY,
                                int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh,
                                int32_t sw, int32_t ph, int32_t pw);
/* :707 kernel_remode -- CW[FH, FW, IC, OC] = W[OC, FH, FW, IC] re-ordered, on `stream` */
int dragon_Cuda_conv3D_kernel_remode(int64_t stream, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
                                     int32_t OC, int32_t IC);
/* :773 conv3D_GemmR, :813 _SGM, :918 _texture, :958 _texture_SGM */
int dragon_Cuda_conv3D_conv3D_GemmR(const int64_t* streams, int32_t length, int64_t dX, int32_t IH, int32_t IW,
                                    int64_t dW, int64_t dCW, int32_t FH, int32_t FW, int64_t dY, int32_t OH,
                                    int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw,
                                    int32_t ph, int32_t pw);
int dragon_Cuda_conv3D_conv3D_GemmR_SGM(const int64_t* streams, int32_t length, int64_t dX, int32_t IH,
                                        int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW, int64_t dY,
                                        int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh,
                                        int32_t sw, int32_t ph, int32_t pw, int32_t GM_slice);
int dragon_Cuda_conv3D_conv3D_GemmR_texture(const int64_t* streams, int32_t length, int64_t dX, int32_t IH,
                                            int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
                                            int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC,
                                            int32_t OC, int32_t sh, int32_t sw, int32_t ph, int32_t pw);
int dragon_Cuda_conv3D_conv3D_GemmR_texture_SGM(const int64_t* streams, int32_t length, int64_t dX, int32_t IH,
                                                int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
                                                int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC,
                                                int32_t OC, int32_t sh, int32_t sw, int32_t ph, int32_t pw,
                                                int32_t GM_slice);
/* :1036 conv3D_GemmR_W1, :1068 _SGM */
int dragon_Cuda_conv3D_conv3D_GemmR_W1(const int64_t* streams, int32_t length, int64_t dX, int32_t IH,
                                       int32_t IW, int64_t dW, int64_t dCW, int64_t dY, int32_t N, int32_t IC,
                                       int32_t OC);
int dragon_Cuda_conv3D_conv3D_GemmR_W1_SGM(const int64_t* streams, int32_t length, int64_t dX, int32_t IH,
                                           int32_t IW, int64_t dW, int64_t dCW, int64_t dY, int32_t N,
                                           int32_t IC, int32_t OC, int32_t GM_slice);
/* :1175 conv3D_GemmV2R */
int dragon_Cuda_conv3D_conv3D_GemmV2R(int32_t useTexture, const int64_t* streams, int32_t length, int64_t dX,
                                      int32_t IH, int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
                                      int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC,
                                      int32_t sh, int32_t sw, int32_t ph, int32_t pw);
/* :1211, :1251, :1316, :1351 the im2col-Winograd natives (stride 1): boolean "this native handled
 * it".  Always handled here: 1 on success, -(hipError_t) on failure. */
int dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s8_R_texture(int32_t useTexture, const int64_t* streams,
        int32_t length, int64_t dX, int32_t IH, int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
        int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t ph, int32_t pw);
int dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s8_texture_SGM(int32_t useTexture, const int64_t* streams,
        int32_t length, int64_t dX, int32_t IH, int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
        int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t ph, int32_t pw,
        int32_t GM_slice);
int dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s16_R_texture(int32_t useTexture, const int64_t* streams,
        int32_t length, int64_t dX, int32_t IH, int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
        int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t ph, int32_t pw);
int dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s16_texture_SGM(int32_t useTexture, const int64_t* streams,
        int32_t length, int64_t dX, int32_t IH, int32_t IW, int64_t dW, int64_t dCW, int32_t FH, int32_t FW,
        int64_t dY, int32_t OH, int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t ph, int32_t pw,
        int32_t GM_slice);

/* Convolution with the bias row added in the same launch: Y[m][oc] += Bias[oc] for the first
 * lengthv/OC rows m and oc < width (the logical channel count).  Every bit equals conv3D followed by
 * dragon_Cuda_function_linear_dual2D_row(streams[0], Y, Bias, OC, 1, 1, 0, Y, lengthv, width, OC).
 * No native counterpart: the reference's conv3D_biased issues those two launches from Java
 * (alpha-Dragon-v1.2/src/z/dragon/engine/cuda/CudaFloat32EngineBase.java, conv3D_biased). */
int dragon_Cuda_conv3D_conv3D_biased(const int64_t* streams, int32_t length, int64_t dX, int32_t IH,
                                     int32_t IW, int64_t dW, int32_t FH, int32_t FW, int64_t dY, int32_t OH,
                                     int32_t OW, int32_t N, int32_t IC, int32_t OC, int32_t sh, int32_t sw,
                                     int32_t ph, int32_t pw, int64_t dBias, int32_t lengthv, int32_t width);

#ifdef __cplusplus
}
#endif
#endif /* DRAGON_HIP_CONV_H */
