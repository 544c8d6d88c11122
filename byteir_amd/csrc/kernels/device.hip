// Device plumbing of the ROCm provider behind a C ABI: memory, copies, streams, events.
// The provider's host C++ (allocator, work queue, device API) is compiled without HIP
// headers and reaches the runtime only through these calls.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "brt_rocm_kernels.h"
#include "brt_rocm_bench.h"

namespace {
// 128-bit copy, one word per lane (n16 = number of 16-byte words), non-temporal load and ordinary
// store: the fastest of the copy kernels probed on MI355X (256 MiB -> 256 MiB: 7.06 TB/s of
// reads plus writes; non-temporal stores as well 6.50, ordinary loads 6.06-6.30, two or four
// words per lane and resident grid-stride workgroups 5.8-6.3).
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) copy16_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n16) return;
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src) + i);
  dst[i] = uint4{t.x, t.y, t.z, t.w};
}

// Nothing but matrix instructions: each wave keeps eight A and eight B operands (read once from
// `operands`, 256 bytes per lane) and four accumulator tiles in registers and issues 16 independent
// v_mfma_f32_32x32x16 per iteration.  What limits it is the clock the chip holds under that load,
// which depends on how many operand bits toggle: the rate on zeros is the instruction-issue peak,
// the rate on normally distributed operands is the ceiling that any kernel fed such data can reach.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
template <bool Bf16>
__global__ void __launch_bounds__(512, 2) mfma_rate_kernel(const u32x4 *__restrict__ operands, float *__restrict__ sink, int iters) {
  const size_t t = (size_t)blockIdx.x * 512 + threadIdx.x;
  u32x4 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) { a[i] = operands[t * 16 + i]; b[i] = operands[t * 16 + 8 + i]; }
  f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = f32x16{0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int ia = m & 7, ib = (m * 3 + (m >> 3)) & 7;
      if (Bf16) acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[ia]), __builtin_bit_cast(bf16x8, b[ib]), acc[m & 3], 0, 0, 0);
      else acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[ia]), __builtin_bit_cast(f16x8, b[ib]), acc[m & 3], 0, 0, 0);
    }
    if ((it & 63) == 63) {  // keeps the sums finite; 64 multiplies per 1024 matrix instructions
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] *= 1e-3f;
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[i][j];
  sink[t] = s;
}
}  // namespace

extern "C" {

int brt_rocm_mfma_rate_probe(int dtype, const void *operands, size_t operand_bytes, float *sink, size_t sink_bytes,
                             int blocks, int iters, void *stream) {
  if (blocks <= 0 || iters < 0 || (dtype != BRT_ROCM_F16 && dtype != BRT_ROCM_BF16)) return hipErrorInvalidValue;
  if (operand_bytes < (size_t)blocks * 512 * 256 || sink_bytes < (size_t)blocks * 512 * 4) return hipErrorInvalidValue;
  if (reinterpret_cast<uintptr_t>(operands) & 15u) return hipErrorInvalidValue;
  if (dtype == BRT_ROCM_BF16)
    mfma_rate_kernel<true><<<dim3(blocks), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(static_cast<const u32x4 *>(operands), sink, iters);
  else
    mfma_rate_kernel<false><<<dim3(blocks), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(static_cast<const u32x4 *>(operands), sink, iters);
  return hipGetLastError();
}

int brt_rocm_copy_kernel(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes % 16 != 0 || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u))
    return hipErrorInvalidValue;
  const size_t n16 = bytes / 16;
  if (n16 == 0) return hipSuccess;
  const size_t blocks = (n16 + 255) / 256;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  copy16_kernel<<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<uint4 *>(dst), static_cast<const uint4 *>(src), n16);
  return hipGetLastError();
}

const char *brt_rocm_version(void) { return "byteir-amd 0.1 (gfx950)"; }
const char *brt_rocm_error_string(int err) {
  if (err == BRT_ROCM_ERROR_STATIC_SCRATCH_TOO_SMALL)
    return "brt_rocm_reduce_static: the split partials of this fold exceed the 8 MiB static scratch "
           "(BRT_ROCM_REDUCE_STATIC_SCRATCH_BYTES); use brt_rocm_reduce with a caller workspace";
  return hipGetErrorString(static_cast<hipError_t>(err));
}

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
// A fill kernel instead of hipMemsetAsync: a caller may capture the call in a HIP graph, and
// memset nodes have given wrong results on replays after the first on these machines.  Bytes
// before the first and after the last 16-byte boundary are written one by one.
__global__ void __launch_bounds__(256) fill_bytes_kernel(unsigned char *dst, unsigned value, size_t bytes) {
  size_t head = (16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15;
  if (head > bytes) head = bytes;
  const size_t body = (bytes - head) / 16, tail = bytes - head - body * 16;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
  const unsigned w = value * 0x01010101u;
  for (size_t i = idx; i < head; i += stride) dst[i] = (unsigned char)value;
  uint4 *mid = reinterpret_cast<uint4 *>(dst + head);
  for (size_t i = idx; i < body; i += stride) mid[i] = uint4{w, w, w, w};
  for (size_t i = idx; i < tail; i += stride) dst[head + body * 16 + i] = (unsigned char)value;
}

int brt_rocm_memset(void *dst, int value, size_t bytes, void *stream) {
  if (bytes == 0) return hipSuccess;
  if (!dst) return hipErrorInvalidValue;
  size_t blocks = (bytes / 16 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 8192) blocks = 8192;
  fill_bytes_kernel<<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<unsigned char *>(dst), (unsigned)value & 0xffu, bytes);
  return hipGetLastError();
}

int brt_rocm_launch_kernel(const void *func, const unsigned grid[3], const unsigned block[3],
                           void **kernel_args, size_t shared_bytes, void *stream) {
  if (!func || !grid || !block) return hipErrorInvalidValue;
  if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return hipSuccess;  // nothing to do
  return hipLaunchKernel(func, dim3(grid[0], grid[1], grid[2]), dim3(block[0], block[1], block[2]), kernel_args,
                         shared_bytes, static_cast<hipStream_t>(stream));
}

int brt_rocm_launch_host_func(void *stream, void (*fn)(void *), void *arg) {
  if (!fn) return hipErrorInvalidValue;
  return hipLaunchHostFunc(static_cast<hipStream_t>(stream), fn, arg);
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
