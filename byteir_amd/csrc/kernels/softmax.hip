// Fused row softmax for gfx950: y = exp(x - max(x)) / sum(exp(x - max(x))) over the last
// axis of a dense [rows, cols] tensor, float internals, one rounding at the store.
//
// (A softmax over an inner axis, [A, B, C] over B with C > 1, takes softmax_inner_kernel: lanes
// along the contiguous C axis, one online max/sum pass over B and a second pass that re-reads
// the tile -- mostly from L2 -- and writes.)
//
// softmax_wave_kernel keeps a whole row in the registers of one wave (NV 128-bit vectors per
// lane), so a row is read from HBM once and written once; max and sum are wave64 shuffle
// trees.  Rows too long for registers, or not 16-byte aligned, take softmax_block_kernel,
// which streams the row three times (the re-reads hit L2).
//
// Arithmetic contract: the compiler's linalg_ext.softmax lowering
// (compiler/lib/Conversion/ToLinalg/LinalgExtToLinalg.cpp:286-410): max from -inf with
// maxnum semantics, exp(x - m), sum from 0, divide.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

#include "brt_rocm_kernels.h"

namespace {

constexpr int kBlock = 256;
constexpr float kLog2e = 1.4426950408889634f;

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int EPV = 4;  // elements per 128-bit vector
  static __device__ __forceinline__ float get(const float &v) { return v; }
  static __device__ __forceinline__ float make(float v) { return v; }
};
template <> struct Elem<__half> {
  static constexpr int EPV = 8;
  static __device__ __forceinline__ float get(const __half &v) { return __half2float(v); }
  static __device__ __forceinline__ __half make(float v) { return __float2half_rn(v); }
};
template <> struct Elem<__bf16> {
  static constexpr int EPV = 8;
  static __device__ __forceinline__ float get(const __bf16 &v) { return (float)v; }
  static __device__ __forceinline__ __bf16 make(float v) { return (__bf16)v; }  // RNE
};

// the tensor is read once and written once: non-temporal accesses keep it out of the caches
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream(const uint4 *p) {
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return uint4{t.x, t.y, t.z, t.w};
}
__device__ __forceinline__ void store_stream(uint4 *p, const uint4 &v) {
  __builtin_nontemporal_store(u32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4 *>(p));
}

__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// one wave per row; lane l owns vectors l, l+64, ... (coalesced 1 KiB per wave load)
template <typename T, int NV>
__global__ void __launch_bounds__(kBlock)
softmax_wave_kernel(const T *__restrict__ in, T *__restrict__ out, uint64_t rows, uint32_t nvec) {
  constexpr int EPV = Elem<T>::EPV;
  const int lane = threadIdx.x & 63;
  const uint64_t row = (uint64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;  // whole waves leave together
  const uint4 *src = reinterpret_cast<const uint4 *>(in) + row * nvec;
  uint4 *dst = reinterpret_cast<uint4 *>(out) + row * nvec;

  uint4 raw[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t v = lane + 64u * i;
    if (v < nvec) raw[i] = load_stream(src + v);
  }
  float x[NV][EPV];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const bool ok = lane + 64u * i < nvec;
    const T *e = reinterpret_cast<const T *>(&raw[i]);
#pragma unroll
    for (int k = 0; k < EPV; ++k) {
      x[i][k] = ok ? Elem<T>::get(e[k]) : -INFINITY;
      m = fmaxf(m, x[i][k]);
    }
  }
  m = wave_max(m);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int k = 0; k < EPV; ++k) {
      x[i][k] = fast_exp(x[i][k] - m);  // exp(-inf) = 0 for the padding
      s += x[i][k];
    }
  s = wave_sum(s);
  const float inv = 1.0f / s;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t v = lane + 64u * i;
    if (v < nvec) {
      uint4 o;
      T *e = reinterpret_cast<T *>(&o);
#pragma unroll
      for (int k = 0; k < EPV; ++k) e[k] = Elem<T>::make(x[i][k] * inv);
      store_stream(dst + v, o);
    }
  }
}

__device__ __forceinline__ float block_combine(float v, float *sm, bool is_max) {
  v = is_max ? wave_max(v) : wave_sum(v);
  __syncthreads();  // protects sm against the previous combine's readers
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
  __syncthreads();
  return is_max ? fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3])) : (sm[0] + sm[1]) + (sm[2] + sm[3]);
}

// one block per row, any length and alignment
template <typename T>
__global__ void __launch_bounds__(kBlock)
softmax_block_kernel(const T *in, T *out, uint64_t cols) {
  __shared__ float sm[kBlock / 64];
  const T *x = in + (uint64_t)blockIdx.x * cols;
  T *y = out + (uint64_t)blockIdx.x * cols;
  float m = -INFINITY;
  for (uint64_t j = threadIdx.x; j < cols; j += kBlock) m = fmaxf(m, Elem<T>::get(x[j]));
  m = block_combine(m, sm, true);
  float s = 0.f;
  for (uint64_t j = threadIdx.x; j < cols; j += kBlock) s += fast_exp(Elem<T>::get(x[j]) - m);
  s = block_combine(s, sm, false);
  const float inv = 1.0f / s;
  for (uint64_t j = threadIdx.x; j < cols; j += kBlock)
    y[j] = Elem<T>::make(fast_exp(Elem<T>::get(x[j]) - m) * inv);
}

// Softmax over the middle axis of a dense [A, B, C] tensor: one thread per (a, c) column, lanes
// along c.  Pass 1 keeps a running maximum and a sum rescaled on the fly (so the column is read
// once for both), pass 2 re-reads and writes.
template <typename T>
__global__ void __launch_bounds__(kBlock)
softmax_inner_kernel(const T *__restrict__ in, T *__restrict__ out, uint64_t B, uint64_t C) {
  const uint64_t c = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (c >= C) return;
  const T *x = in + (uint64_t)blockIdx.y * B * C + c;
  T *y = out + (uint64_t)blockIdx.y * B * C + c;
  float m = -INFINITY, s = 0.f;
  for (uint64_t b = 0; b < B; ++b) {
    const float v = Elem<T>::get(x[b * C]);
    const float m_new = fmaxf(m, v);
    // exp(-inf - -inf) would be NaN: a column that is -inf so far keeps s = 0 (if it stays
    // -inf to the end, pass 2 produces the NaN the two-pass definition gives)
    s = m_new == -INFINITY ? 0.f : s * fast_exp(m - m_new) + fast_exp(v - m_new);
    m = m_new;
  }
  const float inv = 1.0f / s;
  for (uint64_t b = 0; b < B; ++b) y[b * C] = Elem<T>::make(fast_exp(Elem<T>::get(x[b * C]) - m) * inv);
}

template <typename T>
hipError_t run_inner(const T *in, T *out, uint64_t A, uint64_t B, uint64_t C, hipStream_t stream) {
  const uint64_t bx = (C + kBlock - 1) / kBlock;
  if (bx > 0x7fffffffull || A > 65535) {
    // the grid's y extent is 16 bits: fold batches into several launches
    for (uint64_t a0 = 0; a0 < A; a0 += 65535) {
      const uint64_t na = A - a0 < 65535 ? A - a0 : 65535;
      if (bx > 0x7fffffffull) return hipErrorInvalidValue;
      softmax_inner_kernel<T><<<dim3((unsigned)bx, (unsigned)na), dim3(kBlock), 0, stream>>>(in + a0 * B * C, out + a0 * B * C, B, C);
    }
    return hipGetLastError();
  }
  softmax_inner_kernel<T><<<dim3((unsigned)bx, (unsigned)A), dim3(kBlock), 0, stream>>>(in, out, B, C);
  return hipGetLastError();
}

template <typename T>
hipError_t run(const T *in, T *out, uint64_t rows, uint64_t cols, hipStream_t stream) {
  constexpr int EPV = Elem<T>::EPV;
  const bool vec_ok = cols % EPV == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const uint64_t nvec = cols / EPV;
  if (vec_ok && nvec <= 64 * 16) {
    const uint64_t blocks = (rows + kBlock / 64 - 1) / (kBlock / 64);
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks), block(kBlock);
    const uint32_t nv = (uint32_t)nvec;
    if (nvec <= 64) softmax_wave_kernel<T, 1><<<grid, block, 0, stream>>>(in, out, rows, nv);
    else if (nvec <= 128) softmax_wave_kernel<T, 2><<<grid, block, 0, stream>>>(in, out, rows, nv);
    else if (nvec <= 256) softmax_wave_kernel<T, 4><<<grid, block, 0, stream>>>(in, out, rows, nv);
    else if (nvec <= 512) softmax_wave_kernel<T, 8><<<grid, block, 0, stream>>>(in, out, rows, nv);
    else softmax_wave_kernel<T, 16><<<grid, block, 0, stream>>>(in, out, rows, nv);
    return hipGetLastError();
  }
  if (rows > 0x7fffffffull) return hipErrorInvalidValue;
  softmax_block_kernel<T><<<dim3((unsigned)rows), dim3(kBlock), 0, stream>>>(in, out, cols);
  return hipGetLastError();
}

}  // namespace

extern "C" int brt_rocm_softmax_axis(int dtype, const void *input, void *output, size_t A, size_t B,
                                     size_t C, void *stream_) {
  if (C == 1) return brt_rocm_softmax(dtype, input, output, A, B, stream_);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (A == 0 || B == 0 || C == 0) return hipSuccess;
  if (!input || !output) return hipErrorInvalidValue;
  switch (dtype) {
  case BRT_ROCM_F32:
    return run_inner(static_cast<const float *>(input), static_cast<float *>(output), A, B, C, stream);
  case BRT_ROCM_F16:
    return run_inner(static_cast<const __half *>(input), static_cast<__half *>(output), A, B, C, stream);
  case BRT_ROCM_BF16:
    return run_inner(static_cast<const __bf16 *>(input), static_cast<__bf16 *>(output), A, B, C, stream);
  default:
    return hipErrorInvalidValue;
  }
}

extern "C" int brt_rocm_softmax(int dtype, const void *input, void *output, size_t rows,
                                size_t cols, void *stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (rows == 0 || cols == 0) return hipSuccess;
  if (!input || !output) return hipErrorInvalidValue;
  switch (dtype) {
  case BRT_ROCM_F32:
    return run(static_cast<const float *>(input), static_cast<float *>(output), rows, cols, stream);
  case BRT_ROCM_F16:
    return run(static_cast<const __half *>(input), static_cast<__half *>(output), rows, cols, stream);
  case BRT_ROCM_BF16:
    return run(static_cast<const __bf16 *>(input), static_cast<__bf16 *>(output), rows, cols, stream);
  default:
    return hipErrorInvalidValue;
  }
}
