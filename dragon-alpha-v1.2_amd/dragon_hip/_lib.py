"""ctypes binding of libdragon_hip.so: the C ABI declared in include/dragon_hip_gemm.h
and include/dragon_hip_runtime.h, the host-side engine of include/dragon_hip_engine.h and the
test hooks of include/dragon_hip_testing.h.

The library is loaded from the package directory.  There is no fallback: if the shared
object is missing or a symbol cannot be resolved the import fails, and every compute
entry point needs a GPU.
"""
import ctypes
import os
from ctypes import c_int32, c_int64, c_float, c_void_p, c_char_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libdragon_hip.so")

i32, i64, f32 = c_int32, c_int64, c_float
p_i64 = POINTER(c_int64)
p_f32 = POINTER(c_float)
p_i32 = POINTER(c_int32)

# name -> (restype, argtypes); mirrors the two public headers one to one
_MM2D = [p_i64, i32, i64, i64, i64, i32, i32, i32]
_MMSK = [p_i64, i32, i32, i64, i64, i64, i64, i32, i32, i32]
_BMM = [p_i64, i32, i64, i64, i64, i32, i32, i32, i32, i32]
# streams, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw  (and with CW after W)
_CONV = [p_i64, i32, i64, i32, i32, i64, i32, i32, i64, i32, i32, i32, i32, i32, i32, i32, i32, i32]
_CONVR = [p_i64, i32, i64, i32, i32, i64, i64, i32, i32, i64, i32, i32, i32, i32, i32, i32, i32, i32, i32]
SIGNATURES = {
    # include/dragon_hip_gemm.h
    "dragon_Cuda_matMul_matMul": (i32, _MM2D),
    "dragon_Cuda_matMul_matMulT1": (i32, _MM2D),
    "dragon_Cuda_matMul_matMulT2": (i32, _MM2D),
    "dragon_Cuda_matMul_matMulSK": (i32, _MMSK),
    "dragon_Cuda_matMul_matMulT1SK": (i32, _MMSK),
    "dragon_Cuda_matMul_matMulT2SK": (i32, _MMSK),
    "dragon_Cuda_matMul_SKbuf_summary": (i32, [i64, i64, i64, i32, i32]),
    "dragon_Cuda_matMul_matMulSK_static": (i32, [p_i64, i32, i32, i32, i64, i64, i64, i32, i32, i32]),
    "dragon_Cuda_function_linear_dual2D_row": (i32, [i64, i64, i64, i32, f32, f32, f32, i64, i32, i32, i32]),
    "dragon_Cuda_matMul_matMul_biased": (i32, [p_i64, i32, i64, i64, i64, i64, i32, i32, i32, i32, i32]),
    "dragon_Cuda_function_linear2D": (i32, [i64, f32, i64, f32, i64, i32, i32, i32]),
    "dragon_Cuda_reduce_softmax2D": (i32, [i64, i64, i64, i32, i32, i32, i32, f32]),
    "dragon_Cuda_attention_forward": (i32, [p_i64, i32, i64, i64, i64, i64, i32, i32, i32, i32, i32, i32, i32, f32]),
    "dragon_Cuda_attention_forward_masked": (i32, [p_i64, i32, i64, i64, i64, i64, i64, i32, i32, i32, i32, i32, i32, i32,
                                                   f32, i32, i32]),
    "dragon_Cuda_expk2_transpose2D": (i32, [i64, i64, i64, i32, i32, i32, i32, i32]),
    "dragon_Cuda_expk2_transpose3D": (i32, [i64, i64, i64] + [i32] * 9),
    "dragon_Cuda_expk2_transpose4D": (i32, [i64, i64, i64] + [i32] * 11),
    # include/dragon_hip_conv.h
    "dragon_Cuda_conv3D_conv3D": (i32, _CONV),
    "dragon_Cuda_conv3D_conv3D_texture": (i32, _CONV),
    "dragon_Cuda_conv3D_conv3D_np": (i32, _CONV[:-2]),
    "dragon_Cuda_conv3D_conv3D_W1": (i32, [p_i64, i32, i64, i32, i32, i64, i64, i32, i32, i32]),
    "dragon_Cuda_conv3D_conv3DV2": (i32, [i32] + _CONV),
    "dragon_Cuda_conv3D_kernel_remode": (i32, [i64, i64, i64, i32, i32, i32, i32]),
    "dragon_Cuda_conv3D_conv3D_GemmR": (i32, _CONVR),
    "dragon_Cuda_conv3D_conv3D_GemmR_SGM": (i32, _CONVR + [i32]),
    "dragon_Cuda_conv3D_conv3D_GemmR_texture": (i32, _CONVR),
    "dragon_Cuda_conv3D_conv3D_GemmR_texture_SGM": (i32, _CONVR + [i32]),
    "dragon_Cuda_conv3D_conv3D_GemmR_W1": (i32, [p_i64, i32, i64, i32, i32, i64, i64, i64, i32, i32, i32]),
    "dragon_Cuda_conv3D_conv3D_GemmR_W1_SGM": (i32, [p_i64, i32, i64, i32, i32, i64, i64, i64, i32, i32, i32, i32]),
    "dragon_Cuda_conv3D_conv3D_GemmV2R": (i32, [i32] + _CONVR),
    "dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s8_R_texture": (i32, [i32] + _CONVR[:-4] + [i32, i32]),
    "dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s8_texture_SGM": (i32, [i32] + _CONVR[:-4] + [i32, i32, i32]),
    "dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s16_R_texture": (i32, [i32] + _CONVR[:-4] + [i32, i32]),
    "dragon_Cuda_conv3D_conv3D_Im2col_WinogradR_s16_texture_SGM": (i32, [i32] + _CONVR[:-4] + [i32, i32, i32]),
    "dragon_Cuda_conv3D_conv3D_biased": (i32, _CONV + [i64, i32, i32]),
    "dragon_Cuda_batchMatMul_batchMatMul": (i32, _BMM),
    "dragon_Cuda_batchMatMul_batchMatMul_texture": (i32, _BMM),
    "dragon_Cuda_batchMatMul_batchMatMulT1": (i32, _BMM),
    "dragon_Cuda_batchMatMul_batchMatMulT2": (i32, _BMM),
    "dragon_Cuda_batchMatMul_batchMatMulT2_texture": (i32, _BMM),
    "dragon_Cuda_matMul_matMul_mma": (i32, _MM2D),
    "dragon_Cuda_matMul_matMulT1_mma": (i32, _MM2D),
    "dragon_Cuda_matMul_matMulT2_mma": (i32, _MM2D),
    "dragon_Cuda_batchMatMul_batchMatMul_mma": (i32, [i32] + _BMM),
    "dragon_Cuda_batchMatMul_batchMatMulT1_mma": (i32, _BMM),
    "dragon_Cuda_batchMatMul_batchMatMulT2_mma": (i32, [i32] + _BMM),
    "dragon_Cuda_matMul_blockNum": (i32, [i32, i32]),
    "dragon_Cuda_matMul_nstream": (i32, [i32, i32]),
    "dragon_Cuda_batchMatMul_streamSize": (i32, [i32, i32]),
    "dragon_gemm_force_tile": (None, [i32]),
    "dragon_gemm_skinny_form": (None, [i32]),
    "dragon_test_mem_get_info": (i32, [POINTER(i64), POINTER(i64)]),
    "dragon_gemm_split_policy": (None, [i32]),
    "dragon_gemm_fold_skip": (None, [i32]),
    "dragon_gemm_folds_skipped": (i64, []),
    "dragon_gemm_declined_splits": (i64, []),
    "dragon_gemm_split_loses": (i32, [i32, i32, i32, i32, i32, i32]),
    "dragon_gemm_estimate_us": (ctypes.c_double, [i32, i32, i32, i32, i32, i32]),
    "dragon_gemm_workspace_count": (i32, []),
    "dragon_gemm_workspaces_refused": (i64, []),
    "dragon_gemm_release_workspaces": (i32, []),
    "dragon_gemm_choose_tile": (i32, [i32, i32, i32, i32, i32, i32]),
    "dragon_gemm_paired_form_fits": (i32, [i32, i32, i32, i32, i32]),
    "dragon_gemm_tile_divisor": (None, [ctypes.c_uint32, POINTER(ctypes.c_uint32), POINTER(ctypes.c_uint32)]),
    # include/dragon_hip_runtime.h
    "dragon_Cuda_malloc": (i64, [i64]),
    "dragon_Cuda_free": (i32, [i64]),
    "dragon_Cuda_mallocHost": (i64, [i64]),
    "dragon_Cuda_freeHost": (i32, [i64]),
    "dragon_Cuda_memsetAsync": (i32, [i64, i64, i32, i64]),
    "dragon_Cuda_memcpyAsyncHostToDevice": (i32, [i64, i64, i64, i64]),
    "dragon_Cuda_memcpyAsyncHostToHost": (i32, [i64, i64, i64, i64]),
    "dragon_Cuda_memcpyAsyncDeviceToHost": (i32, [i64, i64, i64, i64]),
    "dragon_Cuda_memcpyAsyncDeviceToDevice": (i32, [i64, i64, i64, i64]),
    "dragon_Cuda_memcpyAsyncDefault": (i32, [i64, i64, i64, i64]),
    "dragon_Cuda_getDeviceId": (i32, []),
    "dragon_Cuda_getDeviceCount": (i32, []),
    "dragon_Cuda_setDevice": (i32, [i32]),
    "dragon_Cuda_deviceSynchronize": (i32, []),
    "dragon_CudaDevice_multiProcessorCount": (i32, [i32]),
    "dragon_Cuda_newStream_Blocking": (i64, []),
    "dragon_Cuda_newStream_NonBlocking": (i64, []),
    "dragon_Cuda_deleteStream": (i32, [i64]),
    "dragon_Cuda_deleteStreams": (i32, [p_i64, i32]),
    "dragon_Cuda_streamQuery": (i32, [i64]),
    "dragon_Cuda_streamSynchronize": (i32, [i64]),
    "dragon_Cuda_streamsSynchronize": (i32, [p_i64, i32]),
    "dragon_Cuda_newEvent_Default": (i64, []),
    "dragon_Cuda_newEvent_BlockingSync": (i64, []),
    "dragon_Cuda_newEvent_DisableTiming": (i64, []),
    "dragon_Cuda_deleteEvent": (i32, [i64]),
    "dragon_Cuda_eventRecord": (i32, [i64, i64]),
    "dragon_Cuda_eventRecord_streams": (i32, [i64, p_i64, i32]),
    "dragon_Cuda_eventSynchronize": (i32, [i64]),
    "dragon_Cuda_eventSync_Del": (i32, [i64]),
    "dragon_Cuda_eventElapsedTime": (f32, [i64, i64]),
    "dragon_Cuda_streamWaitEvent_default": (i32, [i64, i64]),
    "dragon_Cuda_streamsWaitEvent_default": (i32, [p_i64, i32, i64]),
    "dragon_Cuda_getExceptionName": (c_char_p, [i32]),
    "dragon_Cuda_getExceptionInfo": (c_char_p, [i32]),
    "dragon_Cuda_getLastExceptionType": (i32, []),
    "dragon_Cuda_set1D_value": (i32, [i64, i64, f32, i32]),
    "dragon_Cuda_set2D_value": (i32, [i64, i64, f32, i32, i32, i32]),
    "dragon_Cuda_get1D": (i32, [i64, i64, c_void_p, i32]),
    "dragon_Cuda_get2D": (i32, [i64, i64, c_void_p, i32, i32, i32]),
    "dragon_Cuda_set1D": (i32, [i64, i64, c_void_p, i32]),
    "dragon_Cuda_set2D": (i32, [i64, i64, c_void_p, i32, i32, i32]),
    "dragon_Cuda_get1D_v2": (i32, [i64, i64, c_void_p, i64, i32]),
    "dragon_Cuda_get2D_v2": (i32, [i64, i64, c_void_p, i64, i32, i32, i32]),
    "dragon_Cuda_set1D_v2": (i32, [i64, i64, c_void_p, i64, i32]),
    "dragon_Cuda_set2D_v2": (i32, [i64, i64, c_void_p, i64, i32, i32, i32]),
    "dragon_test_copy1D_kernel": (i32, [i64, i64, i64, i64]),
    # include/dragon_hip_engine.h
    "dragon_engine_last_error": (c_char_p, []),
    "dragon_engine_last_cuda_code": (i32, []),
    "dragon_engine_last_status": (i32, []),
    "dragon_engine_cuda_float32": (c_void_p, [i32, i32]),
    "dragon_engine_cuda_float32_buffered": (c_void_p, [i32, i32, i64]),
    "dragon_engine_cuda_float32_pooled": (c_void_p, [i32, i32, i64, i64]),
    "dragon_engine_delete": (None, [c_void_p]),
    "dragon_engine_check": (i32, [c_void_p, i32]),
    "dragon_engine_sync": (i32, [c_void_p, i32]),
    "dragon_engine_set_param": (i32, [c_void_p, c_char_p, i32]),
    "dragon_engine_get_param": (i32, [c_void_p, c_char_p]),
    "dragon_engine_gridZ": (i32, [c_void_p, i32, i32, i32, i32]),
    "dragon_policy_gridZ": (i32, [i32, i32, i32, i32, i32]),
    "dragon_policy_smooth_maxPart": (i32, [i32]),
    "dragon_engine_empty": (c_void_p, [c_void_p, p_i32, i32]),
    "dragon_engine_zeros": (c_void_p, [c_void_p, p_i32, i32]),
    "dragon_engine_tensor": (c_void_p, [c_void_p, c_void_p, i32, p_i32, i32]),
    "dragon_engine_set": (i32, [c_void_p, c_void_p, c_void_p, i32]),
    "dragon_engine_valueOf": (i32, [c_void_p, c_void_p, c_void_p, i32]),
    "dragon_engine_delete_tensor": (i32, [c_void_p, c_void_p]),
    "dragon_tensor_c": (i32, [c_void_p]),
    "dragon_tensor_ndim": (i32, [c_void_p]),
    "dragon_tensor_dim": (i32, [c_void_p, i32]),
    "dragon_tensor_length": (i32, [c_void_p]),
    "dragon_tensor_lengthv": (i32, [c_void_p]),
    "dragon_tensor_length_4x": (i32, [c_void_p]),
    "dragon_tensor_address": (i64, [c_void_p]),
    "dragon_engine_product": (c_void_p, [c_void_p, i32, i32, c_void_p, c_void_p]),
    "dragon_engine_product_into": (i32, [c_void_p, i32, c_void_p, c_void_p, c_void_p]),
    "dragon_engine_fullconnect": (c_void_p, [c_void_p, i32, c_void_p, c_void_p, c_void_p]),
    "dragon_engine_fullconnect_into": (i32, [c_void_p, i32, c_void_p, c_void_p, c_void_p, c_void_p]),
    "dragon_engine_conv3D": (c_void_p, [c_void_p, c_void_p, c_void_p, i32, i32, i32, i32, i32, i32, c_void_p]),
    "dragon_engine_conv3D_into": (i32, [c_void_p, c_void_p, c_void_p, c_void_p, i32, i32, i32, i32, c_void_p]),
    "dragon_policy_conv3D_GEMM_nstream": (i32, [i32, i32]),
    "dragon_engine_attention": (c_void_p, [c_void_p, c_void_p, c_void_p, c_void_p, i32, f32]),
    "dragon_engine_attention_masked": (c_void_p, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, i32, f32]),
    "dragon_engine_linear": (c_void_p, [c_void_p, i32, f32, c_void_p, f32]),
    "dragon_engine_softmax": (c_void_p, [c_void_p, i32, c_void_p, i32, f32]),
    "dragon_engine_transpose": (c_void_p, [c_void_p, i32, c_void_p, i32, i32]),
    "dragon_engine_linear2_row": (c_void_p, [c_void_p, i32, c_void_p, c_void_p, f32, f32, f32]),
}


def load(path=None):
    """Loads the library from the package directory, or from $DRAGON_HIP_LIBRARY when set
    (for trying out another build of the same ABI)."""
    path = path or os.environ.get("DRAGON_HIP_LIBRARY") or LIB_PATH
    if not os.path.exists(path):
        raise ImportError(
            "libdragon_hip.so is not built (%s); run dragon-alpha-v1.2_amd/csrc/build.sh" % path)
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing: fail loudly
        fn.restype = restype
        fn.argtypes = argtypes
    return lib
