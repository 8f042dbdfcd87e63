/*
 * dragon_hip_runtime.h -- C ABI of the runtime bridge the matrix-multiplication path
 * needs: device memory, streams, events and float tensor transfer.
 *
 * Each entry point mirrors one `static native` method of the reference's
 * z.dragon.engine.cuda.impl.Cuda class (source/alpha-Dragon-v1.2/src/z/dragon/engine/
 * cuda/impl/Cuda.java) as implemented by Cuda.dll (RT = source/engine-cuda-base/Cuda/Cuda).
 * Handles (streams, events) and addresses are pointers carried in int64_t, exactly as
 * the reference carries them in jlong.  Where the native returns void and throws
 * CudaException(int), the C function returns the hipError_t value as int (0 = success);
 * functions that return a handle or address report failure as 0 and leave the code in
 * dragon_Cuda_getLastExceptionType().  Java arrays become (pointer, length) pairs.
 */
#ifndef DRAGON_HIP_RUNTIME_H
#define DRAGON_HIP_RUNTIME_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- memory (Cuda.java:66-85; RT/Cuda_memory.cuh:7-110) ------------------------- */
int64_t dragon_Cuda_malloc(int64_t size);                 /* RT/Cuda_memory.cuh:7  */
int dragon_Cuda_free(int64_t address);                    /* RT/Cuda_memory.cuh:16 */
int64_t dragon_Cuda_mallocHost(int64_t size);             /* pinned; RT/Cuda_memory.cuh:24 */
int dragon_Cuda_freeHost(int64_t address);                /* RT/Cuda_memory.cuh:33 */
int dragon_Cuda_memsetAsync(int64_t stream, int64_t address, int32_t value, int64_t size); /* :41 */
int dragon_Cuda_memcpyAsyncHostToDevice(int64_t stream, int64_t dst, int64_t src, int64_t size);   /* :51 */
int dragon_Cuda_memcpyAsyncHostToHost(int64_t stream, int64_t dst, int64_t src, int64_t size);     /* :63 */
int dragon_Cuda_memcpyAsyncDeviceToHost(int64_t stream, int64_t dst, int64_t src, int64_t size);   /* :75 */
int dragon_Cuda_memcpyAsyncDeviceToDevice(int64_t stream, int64_t dst, int64_t src, int64_t size); /* :87 */
int dragon_Cuda_memcpyAsyncDefault(int64_t stream, int64_t dst, int64_t src, int64_t size);        /* :99 */

/* ---- device (Cuda.java:98-105; RT/Cuda_Device.cuh:7-68) -------------------------- */
int32_t dragon_Cuda_getDeviceId(void);
int32_t dragon_Cuda_getDeviceCount(void);
int dragon_Cuda_setDevice(int32_t dev_id);
int dragon_Cuda_deviceSynchronize(void);
/* What CudaDevice.multiProcessorCount() must return (CudaDevice.java:116,245): the
 * number of compute units; it drives the split-K decision and maxPart. */
int32_t dragon_CudaDevice_multiProcessorCount(int32_t dev_id);

/* ---- streams (Cuda.java:120-144; RT/Cuda_Stream.cuh:18-107).  Every stream is
 * created at the default priority; the priority overloads of the reference are not
 * offered. ----------------------------------------------------------------------- */
int64_t dragon_Cuda_newStream_Blocking(void);             /* RT/Cuda_Stream.cuh:18 */
int64_t dragon_Cuda_newStream_NonBlocking(void);          /* RT/Cuda_Stream.cuh:36 */
int dragon_Cuda_deleteStream(int64_t stream);             /* RT/Cuda_Stream.cuh:55 */
int dragon_Cuda_deleteStreams(const int64_t* streams, int32_t length); /* :64, skips 0 handles */
int32_t dragon_Cuda_streamQuery(int64_t stream);          /* 1 done, 0 not ready, -1 error; :78 */
int dragon_Cuda_streamSynchronize(int64_t stream);        /* RT/Cuda_Stream.cuh:90 */
int dragon_Cuda_streamsSynchronize(const int64_t* streams, int32_t length); /* :98 */

/* ---- events (Cuda.java:150-168; RT/Cuda_Event.cuh:7-149) ------------------------- */
int64_t dragon_Cuda_newEvent_Default(void);               /* RT/Cuda_Event.cuh:7  */
int64_t dragon_Cuda_newEvent_BlockingSync(void);          /* :15 */
int64_t dragon_Cuda_newEvent_DisableTiming(void);         /* :23 */
int dragon_Cuda_deleteEvent(int64_t event);               /* :39 */
int dragon_Cuda_eventRecord(int64_t event, int64_t stream); /* :47 */
/* The reference's array overload (RT/Cuda_Event.cuh:56-65) blocks the host on every
 * stream and never touches the event.  Here each stream i >= 1 records a private event
 * that streams[0] waits on, then `event` is recorded on streams[0]: the same ordering
 * guarantee (the event completes after all work on all streams) without stalling the
 * host thread. */
int dragon_Cuda_eventRecord_streams(int64_t event, const int64_t* streams, int32_t length);
int dragon_Cuda_eventSynchronize(int64_t event);          /* :68 */
int dragon_Cuda_eventSync_Del(int64_t event);             /* :75 */
float dragon_Cuda_eventElapsedTime(int64_t start_event, int64_t stop_event); /* :95, ms; <0 on error */
int dragon_Cuda_streamWaitEvent_default(int64_t stream, int64_t event);      /* :106 */
int dragon_Cuda_streamsWaitEvent_default(const int64_t* streams, int32_t length, int64_t event); /* :124 */

/* ---- errors (Cuda.java:172-174; RT/Cuda_Exception.cuh:7-27) ---------------------- */
const char* dragon_Cuda_getExceptionName(int32_t type);
const char* dragon_Cuda_getExceptionInfo(int32_t type);
int32_t dragon_Cuda_getLastExceptionType(void);

/* ---- float tensor fill / transfer (Cuda.java:178-194; RT/Cuda_float.cuh:16-368).
 * The set and get forms that move host data are stream-synchronous like the reference's.  The 2-D forms
 * move `height` rows of `width` floats to or from device rows of `stride` floats
 * (stride = width rounded up to 4); uploading writes zeros into the pad. ------------ */
int dragon_Cuda_set1D_value(int64_t stream, int64_t address, float value, int32_t length);   /* :16 */
int dragon_Cuda_set2D_value(int64_t stream, int64_t address, float value,
                            int32_t height, int32_t width, int32_t stride);                  /* :26 */
int dragon_Cuda_get1D(int64_t stream, int64_t address, float* value, int32_t length);        /* :45 */
int dragon_Cuda_get2D(int64_t stream, int64_t address, float* value,
                      int32_t height, int32_t width, int32_t stride);                        /* :83 */
int dragon_Cuda_set1D(int64_t stream, int64_t address, const float* value, int32_t length);  /* :214 */
int dragon_Cuda_set2D(int64_t stream, int64_t address, const float* value,
                      int32_t height, int32_t width, int32_t stride);                        /* :311 */
/* _v2: the caller provides a pinned staging buffer of height*stride (or length) floats. */
int dragon_Cuda_get1D_v2(int64_t stream, int64_t address, float* value, int64_t buf, int32_t length);
int dragon_Cuda_get2D_v2(int64_t stream, int64_t address, float* value, int64_t buf,
                         int32_t height, int32_t width, int32_t stride);
int dragon_Cuda_set1D_v2(int64_t stream, int64_t address, const float* value, int64_t buf, int32_t length);
int dragon_Cuda_set2D_v2(int64_t stream, int64_t address, const float* value, int64_t buf,
                         int32_t height, int32_t width, int32_t stride);

#ifdef __cplusplus
}
#endif
#endif /* DRAGON_HIP_RUNTIME_H */
