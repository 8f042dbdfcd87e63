// JNI shim: the exact symbols the reference's Java classes bind
//   z.dragon.engine.cuda.impl.math.Cuda_matMul        (reference: Cuda_matMul/Cuda_matMul/A.cu:20-178)
//   z.dragon.engine.cuda.impl.math.Cuda_batchMatMul   (reference: Cuda_batchMatMul/Cuda_batchMatMul/A.cu:20-143)
//   z.dragon.engine.cuda.impl.math.Cuda_conv3D        (reference: Cuda_conv3D/Cuda_conv3D/A.cu:18-600)
//   z.dragon.engine.cuda.impl.Cuda (the subset this path uses; reference: Cuda/Cuda/Cuda_memory.cuh,
//   Cuda_Stream.cuh, Cuda_Event.cuh, Cuda_Device.cuh, Cuda_float.cuh)
// each forwarding to the C ABI of include/dragon_hip_gemm.h / dragon_hip_runtime.h and turning a
// non-zero status into z.dragon.engine.cuda.impl.CudaException(int), as the reference's
// handleError / throwCudaException do (Cuda_matMul/Cuda_matMul/JNITool.cuh:9-25).
//
// Built where a JDK provides <jni.h> (build_jni.sh next to this file); the rest of the library does not
// depend on it.  Without a JDK the CPU tests still compile it, against a minimal stand-in header, and
// compare its exports with the reference's names.
#if __has_include(<jni.h>)
#include <jni.h>
#include <stddef.h>
#include <stdint.h>

#include <vector>

#include "../../../include/dragon_hip_conv.h"
#include "../../../include/dragon_hip_gemm.h"
#include "../../../include/dragon_hip_runtime.h"

namespace {

JavaVM* g_jvm = nullptr;

void throwCudaException(JNIEnv* env, int code) {
    jclass cls = env->FindClass("z/dragon/engine/cuda/impl/CudaException");
    if (cls == nullptr) return;                       // NoClassDefFoundError is already pending
    jmethodID ctor = env->GetMethodID(cls, "<init>", "(I)V");
    if (ctor == nullptr) return;
    jobject ex = env->NewObject(cls, ctor, (jint)code);
    if (ex != nullptr) env->Throw((jthrowable)ex);
}
inline void handle(JNIEnv* env, int code) {
    if (code != 0) throwCudaException(env, code);
}
inline jlong handle_addr(JNIEnv* env, int64_t v) {
    if (v == 0) {
        int code = dragon_Cuda_getLastExceptionType();
        throwCudaException(env, code ? code : 2);
    }
    return (jlong)v;
}

// The reference copies the handles into a fixed jlong streams[10]; a longer array is an
// error here instead of a buffer overrun.
struct Streams {
    int64_t s[10];
    int n;
    bool ok;
    Streams(JNIEnv* env, jlongArray arr, jint length) : n(length), ok(false) {
        if (arr == nullptr || length < 1 || length > 10 || env->GetArrayLength(arr) < length) {
            throwCudaException(env, 1);
            return;
        }
        jlong tmp[10];
        env->GetLongArrayRegion(arr, 0, length, tmp);
        for (int i = 0; i < length; i++) s[i] = (int64_t)tmp[i];
        ok = true;
    }
};

std::vector<int64_t> long_array(JNIEnv* env, jlongArray arr, jint length) {
    std::vector<int64_t> v;
    if (arr == nullptr || length <= 0) return v;
    std::vector<jlong> tmp((size_t)length);
    env->GetLongArrayRegion(arr, 0, length, tmp.data());
    v.assign(tmp.begin(), tmp.end());
    return v;
}

}  // namespace

#define MM(name) Java_z_dragon_engine_cuda_impl_math_Cuda_1matMul_##name
#define BMM(name) Java_z_dragon_engine_cuda_impl_math_Cuda_1batchMatMul_##name
#define RT(name) Java_z_dragon_engine_cuda_impl_Cuda_##name
#define FN(name) Java_z_dragon_engine_cuda_impl_math_Cuda_1function_##name
#define EK(name) Java_z_dragon_engine_cuda_impl_Cuda_1expk2_##name
#define CV(name) Java_z_dragon_engine_cuda_impl_math_Cuda_1conv3D_##name

extern "C" {

JNIEXPORT jint JNICALL JNI_OnLoad(JavaVM* vm, void*) {   // reference: Cuda/Cuda/JNIConfig.cuh:12-20
    g_jvm = vm;
    return JNI_VERSION_1_8;
}

// ---- Cuda_matMul -------------------------------------------------------------------------
JNIEXPORT void JNICALL MM(SKbuf_1summary)(JNIEnv* env, jclass, jlong stream, jlong dCbuf, jlong dC,
                                          jint part, jint sizeC) {
    handle(env, dragon_Cuda_matMul_SKbuf_summary(stream, dCbuf, dC, part, sizeC));
}

#define DEF_MM2D(jname, cname)                                                                   \
    JNIEXPORT void JNICALL MM(jname)(JNIEnv* env, jclass, jlongArray streamArray, jint length,   \
                                     jlong dA, jlong dB, jlong dC, jint N, jint M, jint K) {     \
        Streams st(env, streamArray, length);                                                    \
        if (!st.ok) return;                                                                      \
        handle(env, cname(st.s, st.n, dA, dB, dC, N, M, K));                                     \
    }
DEF_MM2D(matMul, dragon_Cuda_matMul_matMul)
DEF_MM2D(matMulT1, dragon_Cuda_matMul_matMulT1)
DEF_MM2D(matMulT2, dragon_Cuda_matMul_matMulT2)
DEF_MM2D(matMul_1mma, dragon_Cuda_matMul_matMul_mma)
DEF_MM2D(matMulT1_1mma, dragon_Cuda_matMul_matMulT1_mma)
DEF_MM2D(matMulT2_1mma, dragon_Cuda_matMul_matMulT2_mma)

#define DEF_MMSK(jname, cname)                                                                   \
    JNIEXPORT void JNICALL MM(jname)(JNIEnv* env, jclass, jlongArray streamArray, jint length,   \
                                     jint GridZ, jlong dA, jlong dB, jlong dC, jlong dCbuf,      \
                                     jint N, jint M, jint K) {                                   \
        Streams st(env, streamArray, length);                                                    \
        if (!st.ok) return;                                                                      \
        handle(env, cname(st.s, st.n, GridZ, dA, dB, dC, dCbuf, N, M, K));                       \
    }
DEF_MMSK(matMulSK, dragon_Cuda_matMul_matMulSK)
DEF_MMSK(matMulT1SK, dragon_Cuda_matMul_matMulT1SK)
DEF_MMSK(matMulT2SK, dragon_Cuda_matMul_matMulT2SK)

// Both split-K stages without any allocation (the partials stay in the library's static device workspace).
// The reference has no such native: a maintainer who wants it declares `public static native void
// matMulSK_static(long[] streamArray, int length, int variant, int GridZ, long dA_address, long dB_address,
// long dC_address, int N, int M, int K)` in Cuda_matMul.java.
JNIEXPORT void JNICALL MM(matMulSK_1static)(JNIEnv* env, jclass, jlongArray streamArray, jint length,
                                            jint variant, jint GridZ, jlong dA, jlong dB, jlong dC, jint N,
                                            jint M, jint K) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_matMul_matMulSK_static(st.s, st.n, variant, GridZ, dA, dB, dC, N, M, K));
}

// One launch for matMul + bias row.  The reference has no such native: a maintainer who wants it
// declares `public static native void matMul_biased(long[] streamArray, int length, long dA_address,
// long dB_address, long dC_address, long dBias_address, int N, int M, int K, int lengthv, int width)`
// in Cuda_matMul.java and calls it from the unsplit branch of CudaFloat32EngineBase.matMul_biased.
JNIEXPORT void JNICALL MM(matMul_1biased)(JNIEnv* env, jclass, jlongArray streamArray, jint length,
                                          jlong dA, jlong dB, jlong dC, jlong dBias, jint N, jint M,
                                          jint K, jint lengthv, jint width) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_matMul_matMul_biased(st.s, st.n, dA, dB, dC, dBias, N, M, K, lengthv, width));
}

// ---- Cuda_function: the bias row (reference: Cuda_function/Cuda_function/A.cu:287-303) ---------
JNIEXPORT void JNICALL FN(linear_1dual2D_1row)(JNIEnv* env, jclass, jlong stream, jlong dX1, jlong dX2,
                                               jint row_lengthv, jfloat alpha, jfloat beta,
                                               jfloat gamma, jlong dY, jint lengthv, jint width,
                                               jint stride) {
    handle(env, dragon_Cuda_function_linear_dual2D_row(stream, dX1, dX2, row_lengthv, alpha, beta, gamma,
                                                       dY, lengthv, width, stride));
}

// Y = alpha*X + beta (reference: Cuda_function/Cuda_function/A.cu:170-185)
JNIEXPORT void JNICALL FN(linear2D)(JNIEnv* env, jclass, jlong stream, jfloat alpha, jlong dX, jfloat beta,
                                    jlong dY, jint lengthv, jint width, jint stride) {
    handle(env, dragon_Cuda_function_linear2D(stream, alpha, dX, beta, dY, lengthv, width, stride));
}

// ---- Cuda_conv3D: forward convolution (reference: Cuda_conv3D/Cuda_conv3D/A.cu:18-600) ----------
JNIEXPORT void JNICALL CV(kernel_1remode)(JNIEnv* env, jclass, jlong stream, jlong dW, jlong dCW, jint FH,
                                          jint FW, jint OC, jint IC) {
    handle(env, dragon_Cuda_conv3D_kernel_remode(stream, dW, dCW, FH, FW, OC, IC));
}
#define DEF_CV(jname, cname)                                                                            \
    JNIEXPORT void JNICALL CV(jname)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dX, \
                                     jint IH, jint IW, jlong dW, jint FH, jint FW, jlong dY, jint OH,    \
                                     jint OW, jint N, jint IC, jint OC, jint sh, jint sw, jint ph,       \
                                     jint pw) {                                                          \
        Streams st(env, streamArray, length);                                                            \
        if (!st.ok) return;                                                                              \
        handle(env, cname(st.s, st.n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw));   \
    }
DEF_CV(conv3D, dragon_Cuda_conv3D_conv3D)
DEF_CV(conv3D_1texture, dragon_Cuda_conv3D_conv3D_texture)
JNIEXPORT void JNICALL CV(conv3DV2)(JNIEnv* env, jclass, jboolean useTexture, jlongArray streamArray,
                                    jint length, jlong dX, jint IH, jint IW, jlong dW, jint FH, jint FW,
                                    jlong dY, jint OH, jint OW, jint N, jint IC, jint OC, jint sh, jint sw,
                                    jint ph, jint pw) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_conv3D_conv3DV2(useTexture, st.s, st.n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC,
                                            OC, sh, sw, ph, pw));
}
JNIEXPORT void JNICALL CV(conv3D_1np)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dX,
                                      jint IH, jint IW, jlong dW, jint FH, jint FW, jlong dY, jint OH, jint OW,
                                      jint N, jint IC, jint OC, jint sh, jint sw) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_conv3D_conv3D_np(st.s, st.n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw));
}
JNIEXPORT void JNICALL CV(conv3D_1W1)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dX,
                                      jint IH, jint IW, jlong dW, jlong dY, jint N, jint IC, jint OC) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_conv3D_conv3D_W1(st.s, st.n, dX, IH, IW, dW, dY, N, IC, OC));
}
#define DEF_CVR(jname, cname)                                                                           \
    JNIEXPORT void JNICALL CV(jname)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dX, \
                                     jint IH, jint IW, jlong dW, jlong dCW, jint FH, jint FW, jlong dY,  \
                                     jint OH, jint OW, jint N, jint IC, jint OC, jint sh, jint sw,       \
                                     jint ph, jint pw) {                                                 \
        Streams st(env, streamArray, length);                                                            \
        if (!st.ok) return;                                                                              \
        handle(env, cname(st.s, st.n, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph,    \
                          pw));                                                                          \
    }
DEF_CVR(conv3D_1GemmR, dragon_Cuda_conv3D_conv3D_GemmR)
DEF_CVR(conv3D_1GemmR_1texture, dragon_Cuda_conv3D_conv3D_GemmR_texture)
#define DEF_CVR_SGM(jname, cname)                                                                       \
    JNIEXPORT void JNICALL CV(jname)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dX, \
                                     jint IH, jint IW, jlong dW, jlong dCW, jint FH, jint FW, jlong dY,  \
                                     jint OH, jint OW, jint N, jint IC, jint OC, jint sh, jint sw,       \
                                     jint ph, jint pw, jint GM_slice) {                                  \
        Streams st(env, streamArray, length);                                                            \
        if (!st.ok) return;                                                                              \
        handle(env, cname(st.s, st.n, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph,    \
                          pw, GM_slice));                                                                \
    }
DEF_CVR_SGM(conv3D_1GemmR_1SGM, dragon_Cuda_conv3D_conv3D_GemmR_SGM)
DEF_CVR_SGM(conv3D_1GemmR_1texture_1SGM, dragon_Cuda_conv3D_conv3D_GemmR_texture_SGM)
JNIEXPORT void JNICALL CV(conv3D_1GemmR_1W1)(JNIEnv* env, jclass, jlongArray streamArray, jint length,
                                             jlong dX, jint IH, jint IW, jlong dW, jlong dCW, jlong dY, jint N,
                                             jint IC, jint OC) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_conv3D_conv3D_GemmR_W1(st.s, st.n, dX, IH, IW, dW, dCW, dY, N, IC, OC));
}
JNIEXPORT void JNICALL CV(conv3D_1GemmR_1W1_1SGM)(JNIEnv* env, jclass, jlongArray streamArray, jint length,
                                                  jlong dX, jint IH, jint IW, jlong dW, jlong dCW, jlong dY,
                                                  jint N, jint IC, jint OC, jint GM_slice) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_conv3D_conv3D_GemmR_W1_SGM(st.s, st.n, dX, IH, IW, dW, dCW, dY, N, IC, OC, GM_slice));
}
JNIEXPORT void JNICALL CV(conv3D_1GemmV2R)(JNIEnv* env, jclass, jboolean useTexture, jlongArray streamArray,
                                           jint length, jlong dX, jint IH, jint IW, jlong dW, jlong dCW,
                                           jint FH, jint FW, jlong dY, jint OH, jint OW, jint N, jint IC,
                                           jint OC, jint sh, jint sw, jint ph, jint pw) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_conv3D_conv3D_GemmV2R(useTexture, st.s, st.n, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW,
                                                  N, IC, OC, sh, sw, ph, pw));
}
// the im2col-Winograd natives answer "handled" (true) or leave the work to the caller's next branch
#define DEF_CVW(jname, cname)                                                                           \
    JNIEXPORT jboolean JNICALL CV(jname)(JNIEnv* env, jclass, jboolean useTexture,                       \
                                         jlongArray streamArray, jint length, jlong dX, jint IH,         \
                                         jint IW, jlong dW, jlong dCW, jint FH, jint FW, jlong dY,       \
                                         jint OH, jint OW, jint N, jint IC, jint OC, jint ph, jint pw) { \
        Streams st(env, streamArray, length);                                                            \
        if (!st.ok) return JNI_FALSE;                                                                    \
        const int rc = cname(useTexture, st.s, st.n, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW, N, IC, OC, \
                             ph, pw);                                                                    \
        if (rc < 0) { throwCudaException(env, -rc); return JNI_FALSE; }                                  \
        return rc ? JNI_TRUE : JNI_FALSE;                                                                \
    }
DEF_CVW(conv3D_1Im2col_1Winograd_1s8_1R_1texture, dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s8_R_texture)
DEF_CVW(conv3D_1Im2col_1Winograd_1s16_1R_1texture, dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s16_R_texture)
#define DEF_CVW_SGM(jname, cname)                                                                       \
    JNIEXPORT jboolean JNICALL CV(jname)(JNIEnv* env, jclass, jboolean useTexture,                       \
                                         jlongArray streamArray, jint length, jlong dX, jint IH,         \
                                         jint IW, jlong dW, jlong dCW, jint FH, jint FW, jlong dY,       \
                                         jint OH, jint OW, jint N, jint IC, jint OC, jint ph, jint pw,   \
                                         jint GM_slice) {                                                \
        Streams st(env, streamArray, length);                                                            \
        if (!st.ok) return JNI_FALSE;                                                                    \
        const int rc = cname(useTexture, st.s, st.n, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW, N, IC, OC, \
                             ph, pw, GM_slice);                                                          \
        if (rc < 0) { throwCudaException(env, -rc); return JNI_FALSE; }                                  \
        return rc ? JNI_TRUE : JNI_FALSE;                                                                \
    }
DEF_CVW_SGM(conv3D_1Im2col_1WinogradR_1s8_1texture_1SGM, dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s8_texture_SGM)
DEF_CVW_SGM(conv3D_1Im2col_1WinogradR_1s16_1texture_1SGM, dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s16_texture_SGM)

// One launch for the convolution + bias row.  The reference has no such native: a maintainer who wants it
// declares `public static native void conv3D_biased(long[] streamArray, int length, long dX_address, int IH,
// int IW, long dW_address, int FH, int FW, long dY_address, int OH, int OW, int N, int IC, int OC, int sh,
// int sw, int ph, int pw, long dBias_address, int lengthv, int width)` in Cuda_conv3D.java and calls it from
// CudaFloat32EngineBase.conv3D_biased in place of the convolution native and linear_dual2D_row.
JNIEXPORT void JNICALL CV(conv3D_1biased)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dX,
                                          jint IH, jint IW, jlong dW, jint FH, jint FW, jlong dY, jint OH,
                                          jint OW, jint N, jint IC, jint OC, jint sh, jint sw, jint ph, jint pw,
                                          jlong dBias, jint lengthv, jint width) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_conv3D_conv3D_biased(st.s, st.n, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw,
                                                 ph, pw, dBias, lengthv, width));
}

// ---- Cuda_expk2: dimension swap (reference: Cuda_expk2/Cuda_expk2/Cuda_transpose.cuh:13-75) ----
JNIEXPORT void JNICALL EK(transpose2D)(JNIEnv* env, jclass, jlong stream, jlong dX, jlong dY, jint Xdim1,
                                       jint Ydim1, jint strideX, jint strideY, jint length) {
    handle(env, dragon_Cuda_expk2_transpose2D(stream, dX, dY, Xdim1, Ydim1, strideX, strideY, length));
}
JNIEXPORT void JNICALL EK(transpose3D)(JNIEnv* env, jclass, jlong stream, jlong dX, jlong dY, jint Xdim1,
                                       jint Xdim2, jint Ydim1, jint Ydim2, jint dimIndex1, jint dimIndex2,
                                       jint strideX, jint strideY, jint length) {
    handle(env, dragon_Cuda_expk2_transpose3D(stream, dX, dY, Xdim1, Xdim2, Ydim1, Ydim2, dimIndex1,
                                              dimIndex2, strideX, strideY, length));
}
JNIEXPORT void JNICALL EK(transpose4D)(JNIEnv* env, jclass, jlong stream, jlong dX, jlong dY, jint Xdim1,
                                       jint Xdim2, jint Xdim3, jint Ydim1, jint Ydim2, jint Ydim3,
                                       jint dimIndex1, jint dimIndex2, jint strideX, jint strideY,
                                       jint length) {
    handle(env, dragon_Cuda_expk2_transpose4D(stream, dX, dY, Xdim1, Xdim2, Xdim3, Ydim1, Ydim2, Ydim3,
                                              dimIndex1, dimIndex2, strideX, strideY, length));
}

// ---- Cuda_batchMatMul -------------------------------------------------------------------------
#define DEF_BMM(jname, cname)                                                                    \
    JNIEXPORT void JNICALL BMM(jname)(JNIEnv* env, jclass, jlongArray streamArray, jint length,  \
                                      jlong dA, jlong dB, jlong dC, jint Batch, jint d0,         \
                                      jint d1, jint d2, jint d3) {                               \
        Streams st(env, streamArray, length);                                                    \
        if (!st.ok) return;                                                                      \
        handle(env, cname(st.s, st.n, dA, dB, dC, Batch, d0, d1, d2, d3));                       \
    }
DEF_BMM(batchMatMul, dragon_Cuda_batchMatMul_batchMatMul)
DEF_BMM(batchMatMul_1texture, dragon_Cuda_batchMatMul_batchMatMul_texture)
DEF_BMM(batchMatMulT1, dragon_Cuda_batchMatMul_batchMatMulT1)
DEF_BMM(batchMatMulT1_1mma, dragon_Cuda_batchMatMul_batchMatMulT1_mma)
DEF_BMM(batchMatMulT2, dragon_Cuda_batchMatMul_batchMatMulT2)
DEF_BMM(batchMatMulT2_1texture, dragon_Cuda_batchMatMul_batchMatMulT2_texture)

// The attention block in one launch.  The reference has no such native: a maintainer who wants it declares
// `public static native void attention(long[] streamArray, int length, long dQ_address, long dK_address,
// long dV_address, long dY_address, int N, int head, int QL, int VL, int dK4, int dV4, boolean head_inner,
// float scale)` in Cuda_batchMatMul.java and calls it from ChannelMHA.__forward__ when mask == null.
JNIEXPORT void JNICALL BMM(attention)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dQ,
                                      jlong dK, jlong dV, jlong dY, jint N, jint head, jint QL, jint VL,
                                      jint dK4, jint dV4, jboolean head_inner, jfloat scale) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_attention_forward(st.s, st.n, dQ, dK, dV, dY, N, head, QL, VL, dK4, dV4,
                                              head_inner ? 1 : 0, scale));
}

// ... and `attention_masked(long[] streamArray, int length, long dQ_address, long dK_address, long dV_address,
// long dMask_address, long dY_address, int N, int head, int QL, int VL, int dK4, int dV4, boolean head_inner,
// float scale, int mask_pitch, boolean mask_per_head)` for a mask unit that multiplies element by element.
JNIEXPORT void JNICALL BMM(attention_1masked)(JNIEnv* env, jclass, jlongArray streamArray, jint length, jlong dQ,
                                              jlong dK, jlong dV, jlong dMask, jlong dY, jint N, jint head, jint QL,
                                              jint VL, jint dK4, jint dV4, jboolean head_inner, jfloat scale,
                                              jint mask_pitch, jboolean mask_per_head) {
    Streams st(env, streamArray, length);
    if (!st.ok) return;
    handle(env, dragon_Cuda_attention_forward_masked(st.s, st.n, dQ, dK, dV, dMask, dY, N, head, QL, VL, dK4, dV4,
                                                     head_inner ? 1 : 0, scale, mask_pitch, mask_per_head ? 1 : 0));
}

#define DEF_BMM_MMA(jname, cname)                                                                \
    JNIEXPORT void JNICALL BMM(jname)(JNIEnv* env, jclass, jboolean useTexture,                  \
                                      jlongArray streamArray, jint length, jlong dA, jlong dB,   \
                                      jlong dC, jint Batch, jint d0, jint d1, jint d2, jint d3) {\
        Streams st(env, streamArray, length);                                                    \
        if (!st.ok) return;                                                                      \
        handle(env, cname(useTexture ? 1 : 0, st.s, st.n, dA, dB, dC, Batch, d0, d1, d2, d3));   \
    }
DEF_BMM_MMA(batchMatMul_1mma, dragon_Cuda_batchMatMul_batchMatMul_mma)
DEF_BMM_MMA(batchMatMulT2_1mma, dragon_Cuda_batchMatMul_batchMatMulT2_mma)

// ---- Cuda: memory ---------------------------------------------------------------------------------
JNIEXPORT jlong JNICALL RT(malloc)(JNIEnv* env, jclass, jlong size) {
    return handle_addr(env, dragon_Cuda_malloc(size));
}
JNIEXPORT void JNICALL RT(free)(JNIEnv* env, jclass, jlong address) { handle(env, dragon_Cuda_free(address)); }
JNIEXPORT jlong JNICALL RT(mallocHost)(JNIEnv* env, jclass, jlong size) {
    return handle_addr(env, dragon_Cuda_mallocHost(size));
}
JNIEXPORT void JNICALL RT(freeHost)(JNIEnv* env, jclass, jlong address) { handle(env, dragon_Cuda_freeHost(address)); }
JNIEXPORT void JNICALL RT(memsetAsync)(JNIEnv* env, jclass, jlong stream, jlong address, jint value, jlong size) {
    handle(env, dragon_Cuda_memsetAsync(stream, address, value, size));
}
JNIEXPORT void JNICALL RT(memcpyAsyncHostToDevice)(JNIEnv* env, jclass, jlong s, jlong dst, jlong src, jlong n) {
    handle(env, dragon_Cuda_memcpyAsyncHostToDevice(s, dst, src, n));
}
JNIEXPORT void JNICALL RT(memcpyAsyncDeviceToHost)(JNIEnv* env, jclass, jlong s, jlong dst, jlong src, jlong n) {
    handle(env, dragon_Cuda_memcpyAsyncDeviceToHost(s, dst, src, n));
}
JNIEXPORT void JNICALL RT(memcpyAsyncDeviceToDevice)(JNIEnv* env, jclass, jlong s, jlong dst, jlong src, jlong n) {
    handle(env, dragon_Cuda_memcpyAsyncDeviceToDevice(s, dst, src, n));
}
JNIEXPORT void JNICALL RT(memcpyAsyncHostToHost)(JNIEnv* env, jclass, jlong s, jlong dst, jlong src, jlong n) {
    handle(env, dragon_Cuda_memcpyAsyncHostToHost(s, dst, src, n));
}
JNIEXPORT void JNICALL RT(memcpyAsyncDefault)(JNIEnv* env, jclass, jlong s, jlong dst, jlong src, jlong n) {
    handle(env, dragon_Cuda_memcpyAsyncDefault(s, dst, src, n));
}

// ---- Cuda: device ----------------------------------------------------------------------------------
JNIEXPORT jint JNICALL RT(getDeviceId)(JNIEnv*, jclass) { return dragon_Cuda_getDeviceId(); }
JNIEXPORT jint JNICALL RT(getDeviceCount)(JNIEnv*, jclass) { return dragon_Cuda_getDeviceCount(); }
JNIEXPORT void JNICALL RT(setDevice)(JNIEnv* env, jclass, jint id) { handle(env, dragon_Cuda_setDevice(id)); }
JNIEXPORT void JNICALL RT(deviceSynchronize)(JNIEnv* env, jclass) { handle(env, dragon_Cuda_deviceSynchronize()); }

// ---- Cuda: streams (overloads carry the JNI signature suffix) -------------------------------------------
JNIEXPORT jlong JNICALL RT(newStream_1Blocking__)(JNIEnv* env, jclass) {
    return handle_addr(env, dragon_Cuda_newStream_Blocking());
}
JNIEXPORT jlong JNICALL RT(newStream_1Blocking__I)(JNIEnv* env, jclass, jint) {   // priority ignored
    return handle_addr(env, dragon_Cuda_newStream_Blocking());
}
JNIEXPORT jlong JNICALL RT(newStream_1NonBlocking__)(JNIEnv* env, jclass) {
    return handle_addr(env, dragon_Cuda_newStream_NonBlocking());
}
JNIEXPORT jlong JNICALL RT(newStream_1NonBlocking__I)(JNIEnv* env, jclass, jint) {
    return handle_addr(env, dragon_Cuda_newStream_NonBlocking());
}
JNIEXPORT void JNICALL RT(deleteStream__J)(JNIEnv* env, jclass, jlong stream) {
    handle(env, dragon_Cuda_deleteStream(stream));
}
JNIEXPORT void JNICALL RT(deleteStream___3JI)(JNIEnv* env, jclass, jlongArray arr, jint length) {
    std::vector<int64_t> v = long_array(env, arr, length);
    handle(env, dragon_Cuda_deleteStreams(v.data(), (int)v.size()));
}
JNIEXPORT jboolean JNICALL RT(streamQuery)(JNIEnv* env, jclass, jlong stream) {
    int r = dragon_Cuda_streamQuery(stream);
    if (r < 0) { throwCudaException(env, dragon_Cuda_getLastExceptionType()); return JNI_FALSE; }
    return r ? JNI_TRUE : JNI_FALSE;
}
JNIEXPORT void JNICALL RT(streamSynchronize__J)(JNIEnv* env, jclass, jlong stream) {
    handle(env, dragon_Cuda_streamSynchronize(stream));
}
JNIEXPORT void JNICALL RT(streamSynchronize___3JI)(JNIEnv* env, jclass, jlongArray arr, jint length) {
    std::vector<int64_t> v = long_array(env, arr, length);
    handle(env, dragon_Cuda_streamsSynchronize(v.data(), (int)v.size()));
}

// ---- Cuda: events -------------------------------------------------------------------------------------------
JNIEXPORT jlong JNICALL RT(newEvent_1Default)(JNIEnv* env, jclass) { return handle_addr(env, dragon_Cuda_newEvent_Default()); }
JNIEXPORT jlong JNICALL RT(newEvent_1BlockingSync)(JNIEnv* env, jclass) { return handle_addr(env, dragon_Cuda_newEvent_BlockingSync()); }
JNIEXPORT jlong JNICALL RT(newEvent_1DisableTiming)(JNIEnv* env, jclass) { return handle_addr(env, dragon_Cuda_newEvent_DisableTiming()); }
JNIEXPORT void JNICALL RT(deleteEvent)(JNIEnv* env, jclass, jlong event) { handle(env, dragon_Cuda_deleteEvent(event)); }
JNIEXPORT void JNICALL RT(eventRecord__JJ)(JNIEnv* env, jclass, jlong event, jlong stream) {
    handle(env, dragon_Cuda_eventRecord(event, stream));
}
JNIEXPORT void JNICALL RT(eventRecord__J_3JI)(JNIEnv* env, jclass, jlong event, jlongArray arr, jint length) {
    std::vector<int64_t> v = long_array(env, arr, length);
    handle(env, dragon_Cuda_eventRecord_streams(event, v.data(), (int)v.size()));
}
JNIEXPORT void JNICALL RT(eventSynchronize)(JNIEnv* env, jclass, jlong event) { handle(env, dragon_Cuda_eventSynchronize(event)); }
JNIEXPORT void JNICALL RT(eventSync_1Del)(JNIEnv* env, jclass, jlong event) { handle(env, dragon_Cuda_eventSync_Del(event)); }
JNIEXPORT void JNICALL RT(eventSynchronize_1delete)(JNIEnv* env, jclass, jlong event) { handle(env, dragon_Cuda_eventSync_Del(event)); }
JNIEXPORT jfloat JNICALL RT(eventElapsedTime)(JNIEnv* env, jclass, jlong e0, jlong e1) {
    float ms = dragon_Cuda_eventElapsedTime(e0, e1);
    if (ms < 0) throwCudaException(env, dragon_Cuda_getLastExceptionType());
    return ms;
}
JNIEXPORT void JNICALL RT(streamWaitEvent_1default)(JNIEnv* env, jclass, jlong stream, jlong event) {
    handle(env, dragon_Cuda_streamWaitEvent_default(stream, event));
}
JNIEXPORT void JNICALL RT(streamsWaitEvent_1default)(JNIEnv* env, jclass, jlongArray arr, jint length, jlong event) {
    std::vector<int64_t> v = long_array(env, arr, length);
    handle(env, dragon_Cuda_streamsWaitEvent_default(v.data(), (int)v.size(), event));
}

// ---- Cuda: errors -----------------------------------------------------------------------------------------------
JNIEXPORT jstring JNICALL RT(getExceptionName)(JNIEnv* env, jclass, jint type) {
    return env->NewStringUTF(dragon_Cuda_getExceptionName(type));
}
JNIEXPORT jstring JNICALL RT(getExceptionInfo)(JNIEnv* env, jclass, jint type) {
    return env->NewStringUTF(dragon_Cuda_getExceptionInfo(type));
}
JNIEXPORT jint JNICALL RT(getLastExceptionType)(JNIEnv*, jclass) { return dragon_Cuda_getLastExceptionType(); }

// ---- Cuda: float fill / transfer -------------------------------------------------------------------------------------
JNIEXPORT void JNICALL RT(set1D__JJFI)(JNIEnv* env, jclass, jlong stream, jlong address, jfloat value, jint length) {
    handle(env, dragon_Cuda_set1D_value(stream, address, value, length));
}
JNIEXPORT void JNICALL RT(set2D__JJFIII)(JNIEnv* env, jclass, jlong stream, jlong address, jfloat value,
                                         jint height, jint width, jint stride) {
    handle(env, dragon_Cuda_set2D_value(stream, address, value, height, width, stride));
}
JNIEXPORT void JNICALL RT(get1D)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value, jint length) {
    std::vector<float> x((size_t)(length > 0 ? length : 0));
    int rc = dragon_Cuda_get1D(stream, address, x.data(), length);
    if (rc) { throwCudaException(env, rc); return; }
    env->SetFloatArrayRegion(value, 0, length, x.data());
}
JNIEXPORT void JNICALL RT(get2D)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value,
                                 jint height, jint width, jint stride) {
    std::vector<float> x((size_t)height * (size_t)width);
    int rc = dragon_Cuda_get2D(stream, address, x.data(), height, width, stride);
    if (rc) { throwCudaException(env, rc); return; }
    env->SetFloatArrayRegion(value, 0, height * width, x.data());
}
JNIEXPORT void JNICALL RT(get1D_1v2)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value,
                                     jlong buf, jint length) {
    std::vector<float> x((size_t)(length > 0 ? length : 0));
    int rc = dragon_Cuda_get1D_v2(stream, address, x.data(), buf, length);
    if (rc) { throwCudaException(env, rc); return; }
    env->SetFloatArrayRegion(value, 0, length, x.data());
}
JNIEXPORT void JNICALL RT(get2D_1v2)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value,
                                     jlong buf, jint height, jint width, jint stride) {
    std::vector<float> x((size_t)height * (size_t)width);
    int rc = dragon_Cuda_get2D_v2(stream, address, x.data(), buf, height, width, stride);
    if (rc) { throwCudaException(env, rc); return; }
    env->SetFloatArrayRegion(value, 0, height * width, x.data());
}
JNIEXPORT void JNICALL RT(set1D__JJ_3FI)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value, jint length) {
    jfloat* x = env->GetFloatArrayElements(value, nullptr);
    int rc = dragon_Cuda_set1D(stream, address, x, length);
    env->ReleaseFloatArrayElements(value, x, JNI_ABORT);
    handle(env, rc);
}
JNIEXPORT void JNICALL RT(set2D__JJ_3FIII)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value,
                                           jint height, jint width, jint stride) {
    jfloat* x = env->GetFloatArrayElements(value, nullptr);
    int rc = dragon_Cuda_set2D(stream, address, x, height, width, stride);
    env->ReleaseFloatArrayElements(value, x, JNI_ABORT);
    handle(env, rc);
}
JNIEXPORT void JNICALL RT(set1D_1v2__JJ_3FJI)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value,
                                              jlong buf, jint length) {
    jfloat* x = env->GetFloatArrayElements(value, nullptr);
    int rc = dragon_Cuda_set1D_v2(stream, address, x, buf, length);
    env->ReleaseFloatArrayElements(value, x, JNI_ABORT);
    handle(env, rc);
}
JNIEXPORT void JNICALL RT(set2D_1v2__JJ_3FJIII)(JNIEnv* env, jclass, jlong stream, jlong address, jfloatArray value,
                                                jlong buf, jint height, jint width, jint stride) {
    jfloat* x = env->GetFloatArrayElements(value, nullptr);
    int rc = dragon_Cuda_set2D_v2(stream, address, x, buf, height, width, stride);
    env->ReleaseFloatArrayElements(value, x, JNI_ABORT);
    handle(env, rc);
}

}  // extern "C"
#endif  // __has_include(<jni.h>)
