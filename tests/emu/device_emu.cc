// Host stand-in for the device layer of libbrt_rocm_kernels.so (byteir_amd/csrc/kernels/device.hip)
// in the emulated build: "device" memory is host memory that ends at a protected page, a stream
// is a token and everything enqueued on it has already happened when the call returns.  Test
// infrastructure: together with reduce.hip / softmax.hip / fill.hip compiled against wave_emu.h
// it exports every symbol of include/brt_rocm_kernels.h and include/brt_rocm_bench.h, so the
// runtime (libbrt) and the Python mirror run unchanged on a machine without a GPU.
#include <chrono>
#include <cstdint>
#include <cstring>

#include "brt_rocm_bench.h"
#include "brt_rocm_kernels.h"
#include "wave_emu.h"

namespace {
constexpr int kErrUnsupported = 801;  // hipErrorNotSupported
struct Event { std::chrono::steady_clock::time_point t; };
int g_stream_token;
}  // namespace

extern "C" {

const char *brt_rocm_version(void) { return "byteir-amd 0.1 (host emulation)"; }
const char *brt_rocm_error_string(int err) {
  if (err == 0) return "no error";
  if (err == BRT_ROCM_ERROR_STATIC_SCRATCH_TOO_SMALL)
    return "brt_rocm_reduce_static: the split partials of this fold exceed the 8 MiB static scratch "
           "(BRT_ROCM_REDUCE_STATIC_SCRATCH_BYTES); use brt_rocm_reduce with a caller workspace";
  if (err == kErrUnsupported) return "not available in the host emulation";
  if (err == 719) return fa_emu::last_error();
  return fa_emu::hipGetErrorString(err);
}

int brt_rocm_device_count(int *count) { *count = 1; return 0; }
int brt_rocm_set_device(int device_id) { return device_id == 0 ? 0 : 101; }
int brt_rocm_malloc(void **ptr, size_t bytes) { *ptr = fa_emu::guarded_alloc(bytes, true); return *ptr ? 0 : 2; }
int brt_rocm_free(void *ptr) { fa_emu::guarded_free(ptr); return 0; }
int brt_rocm_host_malloc(void **ptr, size_t bytes) { *ptr = fa_emu::guarded_alloc(bytes, true); return *ptr ? 0 : 2; }
int brt_rocm_host_free(void *ptr) { fa_emu::guarded_free(ptr); return 0; }
int brt_rocm_memcpy_h2d(void *dst, const void *src, size_t bytes, void *) { std::memmove(dst, src, bytes); return 0; }
int brt_rocm_memcpy_d2h(void *dst, const void *src, size_t bytes, void *) { std::memmove(dst, src, bytes); return 0; }
int brt_rocm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *) { std::memmove(dst, src, bytes); return 0; }
int brt_rocm_memset(void *dst, int value, size_t bytes, void *) { std::memset(dst, value, bytes); return 0; }
int brt_rocm_copy_kernel(void *dst, const void *src, size_t bytes, void *) {
  if (bytes % 16 != 0 || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u)) return 1;
  std::memmove(dst, src, bytes);
  return 0;
}
// a __global__ function of an external library cannot be run here: it was compiled for the GPU
int brt_rocm_launch_kernel(const void *, const unsigned *, const unsigned *, void **, size_t, void *) { return kErrUnsupported; }
int brt_rocm_launch_host_func(void *, void (*fn)(void *), void *arg) {
  if (!fn) return 1;
  fn(arg);  // everything enqueued before has already run
  return 0;
}
int brt_rocm_stream_create(void **stream) { *stream = &g_stream_token; return 0; }
int brt_rocm_stream_destroy(void *) { return 0; }
int brt_rocm_stream_synchronize(void *) { return 0; }
int brt_rocm_device_synchronize(void) { return 0; }

int brt_rocm_event_create(void **event) { *event = new Event{}; return 0; }
int brt_rocm_event_destroy(void *event) { delete static_cast<Event *>(event); return 0; }
int brt_rocm_event_record(void *event, void *) { static_cast<Event *>(event)->t = std::chrono::steady_clock::now(); return 0; }
int brt_rocm_event_synchronize(void *) { return 0; }
int brt_rocm_event_elapsed_ms(float *ms, void *start, void *stop) {
  *ms = std::chrono::duration<float, std::milli>(static_cast<Event *>(stop)->t - static_cast<Event *>(start)->t).count();
  return 0;
}
int brt_rocm_mfma_rate_probe(int, const void *, size_t, float *, size_t, int, int, void *) { return kErrUnsupported; }

}  // extern "C"
