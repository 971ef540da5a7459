/*
 * Device utilities of the drop-in boundary, on the HIP runtime.
 *
 * Same eleven exports, names, argument order and "no error channel" convention as the
 * reference's src/cuda/device_utils.h:12-22 (bodies src/cuda/device_utils.cu:4-99):
 * a failure prints the HIP error with file/line and exits, as CUDA_ASSERT /
 * CURESULT_ASSERT do (src/cuda/kernel_header.h:64-98).
 */
#ifndef MP_DEVICE_UTILS_H
#define MP_DEVICE_UTILS_H

#include "tensor_types.h"

#if defined(__cplusplus)
  #define EXTERN_C extern "C"
#else
  #define EXTERN_C extern
#endif

/* device_utils.cu:32-51 — select the device; exits when the ordinal does not exist. */
EXTERN_C void mpInitDevice(uint32_t device_number);
/* device_utils.cu:4-9 — stream-ordered allocation of N bytes (hipMallocAsync). */
EXTERN_C void* mpMemAlloc(len_t N, StreamContext);
/* device_utils.cu:10-14 — asynchronous host-to-device copy on the stream. */
EXTERN_C void mpMemcpyHtoD(void* dptr, void const* hptr, len_t N, StreamContext);
/* device_utils.cu:15-19 — device-to-host copy; returns after the bytes have landed,
 * because the reference's callers read the host buffer immediately
 * (src/core/graph.zig:153-182, src/examples/experimental.zig:40-43). */
EXTERN_C void mpMemcpyDtoH(void* hptr, void const* dptr, len_t N, StreamContext);
/* device_utils.cu:20-24 — stream-ordered free (hipFreeAsync). */
EXTERN_C void mpMemFree(void* dptr, StreamContext);
/* device_utils.cu:29-31 */
EXTERN_C void mpDeviceSynchronize();
/* device_utils.cu:25-28 */
EXTERN_C void mpStreamSynchronize(StreamContext);
/* device_utils.cu:70-88 — create a stream (default priority) and a rocBLAS handle bound to it. */
EXTERN_C StreamContext mpInitStream();
/* device_utils.cu:90-99 */
EXTERN_C void mpDeinitStream(StreamContext);
/* No counterpart in the reference: for callers that bring their own stream (a framework's).
 * Returns a context for `hip_stream` (NULL = the default stream) with a new rocBLAS handle bound
 * to it, which the matrix-product launchers need; mpReleaseStream destroys that handle and
 * leaves the stream alone. */
EXTERN_C StreamContext mpAdoptStream(void* hip_stream);
EXTERN_C void mpReleaseStream(StreamContext);
/* device_utils.cu:55-62 — device sync, then print (not exit on) the last error. */
EXTERN_C void mpCheckLastError();
/* device_utils.cu:64-68 */
EXTERN_C len_t mpDeviceTotalMemory(uint32_t device);

#endif
