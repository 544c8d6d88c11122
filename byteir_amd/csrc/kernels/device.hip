// Device plumbing of the ROCm provider behind a C ABI: memory, copies, streams, events.
// The provider's host C++ (allocator, work queue, device API) is compiled without HIP
// headers and reaches the runtime only through these calls.
#include <hip/hip_runtime.h>

#include "brt_rocm_kernels.h"

extern "C" {

const char *brt_rocm_version(void) { return "byteir-amd 0.1 (gfx950)"; }
const char *brt_rocm_error_string(int err) { return hipGetErrorString(static_cast<hipError_t>(err)); }

int brt_rocm_device_count(int *count) { return hipGetDeviceCount(count); }
int brt_rocm_set_device(int device_id) { return hipSetDevice(device_id); }
int brt_rocm_malloc(void **ptr, size_t bytes) { return hipMalloc(ptr, bytes); }
int brt_rocm_free(void *ptr) { return hipFree(ptr); }
int brt_rocm_host_malloc(void **ptr, size_t bytes) { return hipHostMalloc(ptr, bytes, hipHostMallocDefault); }
int brt_rocm_host_free(void *ptr) { return hipHostFree(ptr); }

int brt_rocm_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
  return hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream));
}
int brt_rocm_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
  return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream));
}
int brt_rocm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream));
}
int brt_rocm_memset(void *dst, int value, size_t bytes, void *stream) {
  return hipMemsetAsync(dst, value, bytes, static_cast<hipStream_t>(stream));
}

int brt_rocm_stream_create(void **stream) {
  hipStream_t s = nullptr;
  const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);  // default priority
  *stream = s;
  return e;
}
int brt_rocm_stream_destroy(void *stream) { return hipStreamDestroy(static_cast<hipStream_t>(stream)); }
int brt_rocm_stream_synchronize(void *stream) { return hipStreamSynchronize(static_cast<hipStream_t>(stream)); }
int brt_rocm_device_synchronize(void) { return hipDeviceSynchronize(); }

int brt_rocm_event_create(void **event) {
  hipEvent_t e = nullptr;
  const hipError_t r = hipEventCreate(&e);
  *event = e;
  return r;
}
int brt_rocm_event_destroy(void *event) { return hipEventDestroy(static_cast<hipEvent_t>(event)); }
int brt_rocm_event_record(void *event, void *stream) {
  return hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream));
}
int brt_rocm_event_synchronize(void *event) { return hipEventSynchronize(static_cast<hipEvent_t>(event)); }
int brt_rocm_event_elapsed_ms(float *ms, void *start, void *stop) {
  return hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop));
}

}  // extern "C"
