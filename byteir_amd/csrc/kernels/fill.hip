// Counter-based synthetic data for benchmarks and tests: element i of a buffer is a pure
// function of (seed, i), computed in integer arithmetic plus exact float operations only, so a
// host implementation of the same few lines yields the same bits without copying the buffer.
//
//   z_i  = splitmix64 output number i of the stream seeded with `seed`
//          (state seed + (i + 1) * 0x9E3779B97F4A7C15, then the two xor-shift-multiply rounds)
//   uniform [lo, hi):  u = (z >> 40) * 2^-24,  x = fma(u, hi - lo, lo)   (a fused multiply-add: one rounding)
//   normal (0, sigma): the twelve 16-bit fields of z_{3i}, z_{3i+1}, z_{3i+2} are added; the sum
//          of twelve uniform 16-bit integers has mean 393210 and variance 2^32 - 1, so
//          x = (sum - 393210) * 2^-16 * sigma is N(0, sigma) to the accuracy of the twelve-term
//          central limit (support +-6 sigma), and every step is exact in float.
// Stored as f32, f16 or bf16 with round-to-nearest-even.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

#include "brt_rocm_kernels.h"
#include "launch.h"
#include "brt_rocm_bench.h"

namespace {

__device__ __forceinline__ uint64_t splitmix64_at(uint64_t seed, uint64_t i) {
  uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float sample(int dist, uint64_t seed, uint64_t i, float a, float b) {
  if (dist == BRT_ROCM_FILL_UNIFORM) {
    const float u = (float)(uint32_t)(splitmix64_at(seed, i) >> 40) * 0x1p-24f;
    return __builtin_fmaf(u, b - a, a);  // one rounding, the same on the host (fmaf)
  }
  uint32_t sum = 0;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const uint64_t z = splitmix64_at(seed, 3 * i + k);
    sum += (uint32_t)(z & 0xffff) + (uint32_t)((z >> 16) & 0xffff) + (uint32_t)((z >> 32) & 0xffff) + (uint32_t)(z >> 48);
  }
  return __fmul_rn((float)((int32_t)sum - 393210) * 0x1p-16f, b);
}

template <typename T> __device__ __forceinline__ T to_storage(float v);
template <> __device__ __forceinline__ float to_storage<float>(float v) { return v; }
template <> __device__ __forceinline__ __half to_storage<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __bf16 to_storage<__bf16>(float v) { return (__bf16)v; }

template <typename T>
__global__ void __launch_bounds__(256) fill_kernel(T *__restrict__ out, uint64_t n, int dist, uint64_t seed, float a, float b) {
  uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  const uint64_t stride = (uint64_t)gridDim.x * 256;
  for (; i < n; i += stride) out[i] = to_storage<T>(sample(dist, seed, i, a, b));
}

}  // namespace

extern "C" int brt_rocm_fill(int dtype, int dist, uint64_t seed, void *ptr, size_t n, float a, float b, void *stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (dist != BRT_ROCM_FILL_UNIFORM && dist != BRT_ROCM_FILL_NORMAL) return hipErrorInvalidValue;
  if (n == 0) return hipSuccess;
  if (!ptr) return hipErrorInvalidValue;
  size_t blocks = (n + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  const dim3 grid((unsigned)blocks), block(256);
  switch (dtype) {
  case BRT_ROCM_F32: BRT_ROCM_LAUNCH((fill_kernel<float>), grid, block, stream, static_cast<float *>(ptr), n, dist, seed, a, b); break;
  case BRT_ROCM_F16: BRT_ROCM_LAUNCH((fill_kernel<__half>), grid, block, stream, static_cast<__half *>(ptr), n, dist, seed, a, b); break;
  case BRT_ROCM_BF16: BRT_ROCM_LAUNCH((fill_kernel<__bf16>), grid, block, stream, static_cast<__bf16 *>(ptr), n, dist, seed, a, b); break;
  default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}
