/*
 * Device utilities on the HIP runtime: the mp* exports of the boundary
 * (include/device_utils.h), replacing the CUDA driver-API bodies of the reference's
 * src/cuda/device_utils.cu:4-99. Built as libdev_utils.so, as the reference does
 * (build.zig:23-45).
 */
#include "gemm_dispatch.h"
#include "device_utils.h"

extern "C" void* mpMemAlloc(len_t N, StreamContext stream) {
  void* dptr = nullptr;
  HIP_ASSERT(hipMallocAsync(&dptr, N, get_stream(stream)));
  return dptr;
}

extern "C" void mpMemcpyHtoD(void* dev_ptr, const void* cpu_ptr, len_t N, StreamContext stream) {
  HIP_ASSERT(hipMemcpyAsync(dev_ptr, cpu_ptr, N, hipMemcpyHostToDevice, get_stream(stream)));
}

extern "C" void mpMemcpyDtoH(void* cpu_ptr, void const* dev_ptr, len_t N, StreamContext stream) {
  HIP_ASSERT(hipMemcpyAsync(cpu_ptr, dev_ptr, N, hipMemcpyDeviceToHost, get_stream(stream)));
  HIP_ASSERT(hipStreamSynchronize(get_stream(stream)));
}

extern "C" void mpMemFree(void* dev_ptr, StreamContext stream) {
  HIP_ASSERT(hipFreeAsync(dev_ptr, get_stream(stream)));
}

extern "C" void mpStreamSynchronize(StreamContext stream) {
  HIP_ASSERT(hipStreamSynchronize(get_stream(stream)));
}

extern "C" void mpDeviceSynchronize() {
  HIP_ASSERT(hipDeviceSynchronize());
}

extern "C" void mpInitDevice(uint32_t device_number) {
  int device_count = 0;
  HIP_ASSERT(hipGetDeviceCount(&device_count));
  if (device_count <= (int)device_number) {
    fprintf(stderr, "Error: no devices supporting HIP\n");
    exit(-1);
  }
  HIP_ASSERT(hipSetDevice((int)device_number));
}

extern "C" void mpCheckLastError() {
  HIP_ASSERT(hipDeviceSynchronize());
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    fprintf(stderr, "Error %s: %s", hipGetErrorName(err), hipGetErrorString(err));
  }
}

extern "C" len_t mpDeviceTotalMemory(uint32_t device) {
  hipDeviceProp_t prop;
  HIP_ASSERT(hipGetDeviceProperties(&prop, (int)device));
  return (len_t)prop.totalGlobalMem;
}

extern "C" StreamContext mpInitStream() {
  hipStream_t hip_stream = nullptr;
  HIP_ASSERT(hipStreamCreate(&hip_stream));
  StreamContext context;
  context.hip_stream.ptr = reinterpret_cast<void*>(hip_stream);
  /* the matrix-product launchers find their library handle here, bound to this stream
   * (device_utils.cu:72-86 does the same with cuBLAS) */
  context.blas_handle.ptr = mpCreateBlasContext(hip_stream);
  return context;
}

extern "C" StreamContext mpAdoptStream(void* hip_stream) {
  StreamContext context;
  context.hip_stream.ptr = hip_stream;
  context.blas_handle.ptr = mpCreateBlasContext(static_cast<hipStream_t>(hip_stream));
  return context;
}

extern "C" void mpReleaseStream(StreamContext stream) {
  mpDestroyBlasContext(get_blas(stream));
}

extern "C" void mpDeinitStream(StreamContext stream) {
  mpDestroyBlasContext(get_blas(stream));
  HIP_ASSERT(hipStreamDestroy(get_stream(stream)));
}
