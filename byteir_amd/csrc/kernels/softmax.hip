// Fused row softmax for gfx950: y = exp(x - max(x)) / sum(exp(x - max(x))) over the last
// axis of a dense [rows, cols] tensor, float internals, one rounding at the store.
//
// (A softmax over an inner axis, [A, B, C] over B with C > 1, takes softmax_inner_kernel: a
// workgroup per column tile, lanes along the contiguous C axis with 128-bit accesses, row lanes
// along B; one online max/sum pass and a second pass that re-reads the tile and writes.)
//
// softmax_wave_kernel keeps a whole row of up to 128 vectors in the registers of one wave (one
// or two 128-bit vectors per lane), softmax_split_kernel a row of up to 1024 vectors in those of
// 2, 4 or 8 waves, so a row is read from HBM once and written once; max and sum are wave64
// shuffle trees (plus one LDS hop between the waves of a row).  Longer rows, and rows that are
// not 16-byte aligned, take one workgroup each:
// softmax_regs_kernel holds the row in the workgroup's registers (up to 65536 elements: one HBM
// read, one write), softmax_stream_kernel reads longer ones twice (online maximum and sum, then
// the output pass); both use 128-bit accesses on the aligned span that covers the row.  softmax_block_kernel
// (scalar accesses, three passes) is left for input and output pointers that are misaligned
// differently.
//
// Arithmetic contract: the compiler's linalg_ext.softmax lowering
// (compiler/lib/Conversion/ToLinalg/LinalgExtToLinalg.cpp:286-410): max from -inf with
// maxnum semantics, exp(x - m), sum from 0, divide.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

#include "brt_rocm_kernels.h"
#include "launch.h"

namespace {

constexpr int kBlock = 256;
constexpr float kLog2e = 1.4426950408889634f;

// get / make convert one element; unpack / pack convert a whole 128-bit vector held as four
// 32-bit words (the form in which a vector stays between its load and its use).
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int EPV = 4;  // elements per 128-bit vector
  static __device__ __forceinline__ float get(const float &v) { return v; }
  static __device__ __forceinline__ float make(float v) { return v; }
  static __device__ __forceinline__ void unpack(const uint4 &r, float *x) {
    x[0] = __uint_as_float(r.x); x[1] = __uint_as_float(r.y); x[2] = __uint_as_float(r.z); x[3] = __uint_as_float(r.w);
  }
  static __device__ __forceinline__ uint4 pack(const float *x) {
    return uint4{__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3])};
  }
};
template <> struct Elem<__half> {
  static constexpr int EPV = 8;
  static __device__ __forceinline__ float get(const __half &v) { return __half2float(v); }
  static __device__ __forceinline__ __half make(float v) { return __float2half_rn(v); }
  static __device__ __forceinline__ void unpack(const uint4 &r, float *x) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f16x2 h = __builtin_bit_cast(f16x2, w[j]);
      x[2 * j] = (float)h.x;
      x[2 * j + 1] = (float)h.y;
    }
  }
  static __device__ __forceinline__ uint4 pack(const float *x) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = __builtin_bit_cast(uint32_t, f16x2{(_Float16)x[2 * j], (_Float16)x[2 * j + 1]});  // RNE
    return uint4{w[0], w[1], w[2], w[3]};
  }
};
template <> struct Elem<__bf16> {
  static constexpr int EPV = 8;
  static __device__ __forceinline__ float get(const __bf16 &v) { return (float)v; }
  static __device__ __forceinline__ __bf16 make(float v) { return (__bf16)v; }  // RNE
  static __device__ __forceinline__ void unpack(const uint4 &r, float *x) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      x[2 * j] = __uint_as_float(w[j] << 16);  // a bf16 is the upper half of a float
      x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ uint4 pack(const float *x) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = __builtin_bit_cast(uint32_t, bf16x2{(__bf16)x[2 * j], (__bf16)x[2 * j + 1]});  // RNE
    return uint4{w[0], w[1], w[2], w[3]};
  }
};

// the tensor is read once and written once: non-temporal accesses keep it out of the caches
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream(const uint4 *p) {
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return uint4{t.x, t.y, t.z, t.w};
}
// Stores are ordinary (cached) stores on purpose: with non-temporal loads and ordinary stores a
// 256 MiB -> 256 MiB copy runs at 7.06 TB/s on MI355X, with non-temporal stores as well at 6.50,
// with ordinary loads at 6.06-6.30 (probe over block sizes, vectors per lane and block orders).
#ifndef SOFTMAX_NT_STORE
#define SOFTMAX_NT_STORE 0
#endif
__device__ __forceinline__ void store_stream(uint4 *p, const uint4 &v) {
#if SOFTMAX_NT_STORE
  __builtin_nontemporal_store(u32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4 *>(p));
#else
  *p = v;
#endif
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

  // Every load is issued unconditionally (a lane beyond the row re-reads the row's last vector
  // and ignores it): a load under a branch would be waited for before the next one is issued.
  uint4 raw[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t v = lane + 64u * i;
    raw[i] = load_stream(src + (v < nvec ? v : nvec - 1));
  }
  float x[NV][EPV];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const bool ok = lane + 64u * i < nvec;
    Elem<T>::unpack(raw[i], x[i]);
#pragma unroll
    for (int k = 0; k < EPV; ++k) {
      x[i][k] = ok ? x[i][k] : -INFINITY;
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
#pragma unroll
      for (int k = 0; k < EPV; ++k) x[i][k] *= inv;
      store_stream(dst + v, Elem<T>::pack(x[i]));
    }
  }
}

// A row shared by RW waves of a 512-thread workgroup, two vectors per lane: the same single
// read and single write per element as the wave kernel, but in 2 KiB pieces per wave with twice
// the waves per SIMD.  On MI355X this moves a [32768, 4096] bf16 tensor as fast as a plain copy
// kernel does (6.4-6.5 TB/s); one wave per 8 KiB row, 8 vectors per lane, reaches 6.1 TB/s, and
// resident waves that walk the rows with the next row's loads in flight 5.8-6.0 TB/s.
// FULL: every row is exactly RW * 128 vectors.  Workgroups hold 8 / RW rows; a workgroup's
// rows beyond the tensor are computed on the last row and not stored (all waves meet the barriers).
constexpr int kSplitWaves = 8;
template <typename T, int RW, bool FULL>
__global__ void __launch_bounds__(kSplitWaves * 64)
softmax_split_kernel(const T *__restrict__ in, T *__restrict__ out, uint64_t rows, uint32_t nvec) {
  constexpr int EPV = Elem<T>::EPV;
  constexpr int NV = 2;
  __shared__ float red[2][kSplitWaves];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int first = wave / RW * RW;  // first wave of this row
  // Workgroup ids go round-robin over the 8 XCDs; giving each XCD a contiguous eighth of the rows
  // (instead of every eighth workgroup's rows) measured 2.5 % faster on a plain copy of this size
  // (7.28 against 7.09 TB/s) and the same here.
  uint32_t blk = blockIdx.x;
  if ((gridDim.x & 7u) == 0) blk = (blk & 7u) * (gridDim.x >> 3) + (blk >> 3);
  uint64_t row = (uint64_t)blk * (kSplitWaves / RW) + wave / RW;
  const bool row_ok = row < rows;
  if (!row_ok) row = rows - 1;
  const uint32_t base = (uint32_t)(wave % RW) * (NV * 64) + lane;
  const uint4 *src = reinterpret_cast<const uint4 *>(in) + row * nvec;
  uint4 *dst = reinterpret_cast<uint4 *>(out) + row * nvec;

  uint4 raw[NV];
  bool ok[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t v = base + 64u * i;
    ok[i] = FULL || v < nvec;
    raw[i] = load_stream(src + (ok[i] ? v : nvec - 1));  // never a load under a branch
  }
  float x[NV][EPV];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    Elem<T>::unpack(raw[i], x[i]);
#pragma unroll
    for (int k = 0; k < EPV; ++k) {
      if (!FULL) x[i][k] = ok[i] ? x[i][k] : -INFINITY;
      m = fmaxf(m, x[i][k]);
    }
  }
  m = wave_max(m);
  if (lane == 0) red[0][wave] = m;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < RW; ++r) m = fmaxf(m, red[0][first + r]);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int k = 0; k < EPV; ++k) {
      x[i][k] = fast_exp(x[i][k] - m);  // exp(-inf) = 0 for the padding
      s += x[i][k];
    }
  s = wave_sum(s);
  if (lane == 0) red[1][wave] = s;
  __syncthreads();
  s = 0.f;
#pragma unroll
  for (int r = 0; r < RW; ++r) s += red[1][first + r];
  const float inv = 1.0f / s;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
#pragma unroll
    for (int k = 0; k < EPV; ++k) x[i][k] *= inv;
    if (row_ok && ok[i]) store_stream(dst + base + 64u * i, Elem<T>::pack(x[i]));
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

// ---- rows longer than a wave's registers: one workgroup per row, 128-bit accesses ----------
// A row may start anywhere (odd lengths shift every row), so it is addressed as the span of
// 16-byte vectors that covers it: vector j of the span holds span elements j*EPV .. j*EPV+EPV-1,
// the row is the span elements [lo, hi).  Elements outside belong to the neighbouring rows (or
// to the same 16-byte granule beyond the tensor, which lies in the same page): they are read,
// ignored, and never written.
template <typename T> struct Span {
  static constexpr int EPV = Elem<T>::EPV;
  const uint4 *src;
  uint4 *dst;
  uint64_t lo, hi, nvec;
  __device__ __forceinline__ Span(const T *x, T *y, uint64_t cols) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(x);
    src = reinterpret_cast<const uint4 *>(a & ~(uintptr_t)15);
    dst = reinterpret_cast<uint4 *>(reinterpret_cast<uintptr_t>(y) & ~(uintptr_t)15);  // same offset as x
    lo = (a & 15) / sizeof(T);
    hi = lo + cols;
    nvec = (hi + EPV - 1) / EPV;
  }
  __device__ __forceinline__ bool whole(uint64_t j) const { return j * EPV >= lo && (j + 1) * EPV <= hi; }
  template <typename F> __device__ __forceinline__ void each(const uint4 &raw, uint64_t j, F f) const {
    const T *e = reinterpret_cast<const T *>(&raw);
    if (whole(j)) {
#pragma unroll
      for (int k = 0; k < EPV; ++k) f(Elem<T>::get(e[k]));
    } else {
#pragma unroll
      for (int k = 0; k < EPV; ++k)
        if (j * EPV + k >= lo && j * EPV + k < hi) f(Elem<T>::get(e[k]));
    }
  }
  // y = exp(x - m) * inv for the row's elements of vector j
  __device__ __forceinline__ void finish(const uint4 &raw, uint64_t j, float m, float inv) const {
    const T *e = reinterpret_cast<const T *>(&raw);
    uint4 o;
    T *oe = reinterpret_cast<T *>(&o);
#pragma unroll
    for (int k = 0; k < EPV; ++k) oe[k] = Elem<T>::make(fast_exp(Elem<T>::get(e[k]) - m) * inv);
    if (whole(j)) {
      store_stream(dst + j, o);
    } else {
      T *d = reinterpret_cast<T *>(dst + j);
#pragma unroll
      for (int k = 0; k < EPV; ++k)
        if (j * EPV + k >= lo && j * EPV + k < hi) d[k] = oe[k];
    }
  }
};

template <int THREADS> __device__ __forceinline__ float block_all(float v, float *sm, bool is_max) {
  v = is_max ? wave_max(v) : wave_sum(v);
  __syncthreads();  // protects sm against the previous call's readers
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = sm[0];
#pragma unroll
  for (int w = 1; w < THREADS / 64; ++w) r = is_max ? fmaxf(r, sm[w]) : r + sm[w];
  return r;
}

// The row lives in the registers of one workgroup as floats (thread t owns vectors t,
// t + THREADS, ...; XR floats per thread), so it is read from HBM once and written once and every
// exponential is taken once: softmax_wave_kernel with a workgroup in place of a wave.
template <typename T, int THREADS, int XR>
__global__ void __launch_bounds__(THREADS)
softmax_regs_kernel(const T *in, T *out, uint64_t cols) {
  constexpr int EPV = Elem<T>::EPV, NV = XR / EPV;
  __shared__ float sm[THREADS / 64];
  const Span<T> sp(in + (uint64_t)blockIdx.x * cols, out + (uint64_t)blockIdx.x * cols, cols);
  const uint32_t nvec = (uint32_t)sp.nvec;
  // vectors beyond the row's span (j >= nvec) are skipped as a whole: for a given i they are
  // the last threads of the workgroup, so whole waves skip together
  // Four-byte elements: all loads are issued in a loop of their own before the first value is
  // used (measured 5.3 against 4.8 TB/s on [4096, 32000] f32).  Two-byte elements: the load
  // sits in the loop that unpacks it, which keeps the kernel within 64 registers, i.e. two
  // 1024-thread workgroups per CU (5.4 against 3.5 TB/s on [8192, 16384] bf16).
  constexpr bool kLoadsFirst = sizeof(T) == 4;
  uint4 raw[NV];
  if constexpr (kLoadsFirst) {
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (threadIdx.x + (uint32_t)THREADS * i < nvec) raw[i] = load_stream(sp.src + threadIdx.x + (uint32_t)THREADS * i);
  }
  float x[NV][EPV];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t j = threadIdx.x + (uint32_t)THREADS * i;
    if (j < nvec) {
      if constexpr (!kLoadsFirst) raw[i] = load_stream(sp.src + j);
      const T *e = reinterpret_cast<const T *>(&raw[i]);
      const bool whole = sp.whole(j);
#pragma unroll
      for (int k = 0; k < EPV; ++k) {
        const uint64_t idx = (uint64_t)j * EPV + k;
        x[i][k] = (whole || (idx >= sp.lo && idx < sp.hi)) ? Elem<T>::get(e[k]) : -INFINITY;
        m = fmaxf(m, x[i][k]);
      }
    }
  }
  m = block_all<THREADS>(m, sm, true);
  const float ms = m * kLog2e;
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (threadIdx.x + (uint32_t)THREADS * i < nvec) {
#pragma unroll
      for (int k = 0; k < EPV; ++k) {
        x[i][k] = __builtin_amdgcn_exp2f(fmaf(x[i][k], kLog2e, -ms));  // 0 for elements outside the row
        s += x[i][k];
      }
    }
  }
  s = block_all<THREADS>(s, sm, false);
  const float inv = 1.0f / s;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t j = threadIdx.x + (uint32_t)THREADS * i;
    if (j < nvec) {
      uint4 o;
      T *oe = reinterpret_cast<T *>(&o);
#pragma unroll
      for (int k = 0; k < EPV; ++k) oe[k] = Elem<T>::make(x[i][k] * inv);
      if (sp.whole(j)) {
        store_stream(sp.dst + j, o);
      } else {
        T *d = reinterpret_cast<T *>(sp.dst + j);
#pragma unroll
        for (int k = 0; k < EPV; ++k)
          if ((uint64_t)j * EPV + k >= sp.lo && (uint64_t)j * EPV + k < sp.hi) d[k] = oe[k];
      }
    }
  }
}

// Rows beyond a workgroup's registers: pass 1 keeps a running maximum and a sum rescaled on the fly (one read
// for both), pass 2 reads the row again (from the caches when they hold it) and writes.
template <typename T, int THREADS>
__global__ void __launch_bounds__(THREADS)
softmax_stream_kernel(const T *in, T *out, uint64_t cols) {
  __shared__ float sm[THREADS / 64];
  const Span<T> sp(in + (uint64_t)blockIdx.x * cols, out + (uint64_t)blockIdx.x * cols, cols);
  float m = -INFINITY, s = 0.f;
#pragma unroll 4
  for (uint64_t j = threadIdx.x; j < sp.nvec; j += THREADS) {
    const uint4 raw = sp.src[j];
    float vm = -INFINITY;
    sp.each(raw, j, [&](float v) { vm = fmaxf(vm, v); });
    if (vm > m) { s *= fast_exp(m - vm); m = vm; }  // exp(-inf - vm) = 0 for the first finite value
    if (m != -INFINITY) sp.each(raw, j, [&](float v) { s += fast_exp(v - m); });
    else sp.each(raw, j, [&](float v) { if (v != v) s = v; });  // only -inf so far: s stays 0, or NaN after a NaN
  }
  const float m_all = block_all<THREADS>(m, sm, true);
  s = (m == -INFINITY) ? s : s * fast_exp(m - m_all);  // a lane that saw only -inf (and NaN) adds 0 (NaN)
  s = block_all<THREADS>(s, sm, false);
  const float inv = 1.0f / s;
#pragma unroll 4
  for (uint64_t j = threadIdx.x; j < sp.nvec; j += THREADS) sp.finish(load_stream(sp.src + j), j, m_all, inv);
}

// Softmax over the middle axis of a dense [A, B, C] tensor.  A workgroup owns TX * VEC adjacent
// columns of one a: lane (tx, ty) owns VEC columns (one 128-bit load per row when VEC > 1) and
// walks rows ty, ty + TY, ...  Pass 1 keeps a running maximum and a sum rescaled on the fly per
// column (one read for both); the TY partials of a column meet in LDS; pass 2 reads the tile
// again (from the caches when they hold it) and writes.
// Few columns and a long B would leave most of the chip idle, so B can be cut into S segments
// over workgroups: MODE 1 runs pass 1 on a segment and writes the column's (maximum, sum) to
// part[a][segment][c][2]; MODE 2 folds the S partials of its columns and runs pass 2 on its
// segment.  MODE 0 is both passes in one workgroup (S = 1).
template <typename T, int VEC, int TX, int MODE>
__global__ void __launch_bounds__(kBlock)
softmax_inner_kernel(const T *__restrict__ in, T *__restrict__ out, uint64_t B, uint64_t C, uint32_t col_tiles,
                     uint32_t S, uint64_t seg_rows, float *__restrict__ part) {
  constexpr int TY = kBlock / TX;
  __shared__ float pm[TY][TX * VEC + 1], ps[TY][TX * VEC + 1];
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const uint32_t tile = blockIdx.x % col_tiles;
  const uint32_t seg = (blockIdx.x / col_tiles) % S;
  const uint64_t a = blockIdx.x / ((uint64_t)col_tiles * S);
  const uint64_t b0 = (uint64_t)seg * seg_rows, b1 = b0 + seg_rows < B ? b0 + seg_rows : B;
  const uint64_t c = ((uint64_t)tile * TX + tx) * VEC;
  const bool ok = c < C;  // C is a multiple of VEC
  const T *x = in + a * B * C + c;
  T *y = out + a * B * C + c;
  auto load = [&](uint64_t b, float (&v)[VEC]) {
    if constexpr (VEC > 1) {
      const uint4 raw = *reinterpret_cast<const uint4 *>(x + b * C);
      const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
      for (int k = 0; k < VEC; ++k) v[k] = Elem<T>::get(e[k]);
    } else {
      v[0] = Elem<T>::get(x[b * C]);
    }
  };
  float m[VEC], s[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) { m[k] = -INFINITY; s[k] = 0.f; }
  if (MODE != 2 && ok) {
#pragma unroll 8
    for (uint64_t b = b0 + ty; b < b1; b += TY) {
      float v[VEC];
      load(b, v);
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const float m_new = fmaxf(m[k], v[k]);
        // exp(-inf - -inf) would be NaN: a column that is -inf so far keeps its s, which is 0,
        // or NaN once a NaN has been seen (the maximum skips NaN, the sum must not); if the
        // column stays -inf to the end, pass 2 produces the NaN the two-pass definition gives
        // One exponential serves both cases: a new maximum rescales the sum by exp(m - v) and adds
        // 1, otherwise exp(v - m) is added.  (m = -inf: e = 0, s becomes 1; v = -inf: e = 0.)
        const float d = v[k] - m[k];
        const float e = fast_exp(-fabsf(d));
        s[k] = m_new == -INFINITY ? (v[k] != v[k] ? v[k] : s[k]) : (d > 0.f ? fmaf(s[k], e, 1.f) : s[k] + e);
        m[k] = m_new;
      }
    }
  }
  if (MODE == 2 && ok) {  // the segments' partials of this lane's columns, shared out over the row lanes
    const float *pp = part + (a * S * C + c) * 2;
    for (uint32_t r = ty; r < S; r += TY)
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const float mr = pp[((uint64_t)r * C + k) * 2], sr = pp[((uint64_t)r * C + k) * 2 + 1];
        const float m_new = fmaxf(m[k], mr);
        // a side that saw only -inf (and NaN) adds its s as it is: 0, or NaN
        s[k] = (m[k] == -INFINITY ? s[k] : s[k] * fast_exp(m[k] - m_new)) + (mr == -INFINITY ? sr : sr * fast_exp(mr - m_new));
        m[k] = m_new;
      }
  }
  // the TY partials of every column meet in LDS
#pragma unroll
  for (int k = 0; k < VEC; ++k) { pm[ty][tx * VEC + k] = m[k]; ps[ty][tx * VEC + k] = s[k]; }
  __syncthreads();
  float inv[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    float mm = -INFINITY, ss = 0.f;
#pragma unroll 4
    for (int r = 0; r < TY; ++r) mm = fmaxf(mm, pm[r][tx * VEC + k]);
#pragma unroll 4
    for (int r = 0; r < TY; ++r) {
      const float mr = pm[r][tx * VEC + k];
      ss += mr == -INFINITY ? ps[r][tx * VEC + k] : ps[r][tx * VEC + k] * fast_exp(mr - mm);
    }
    m[k] = mm;
    inv[k] = 1.0f / ss;
    s[k] = ss;
  }
  if constexpr (MODE == 1) {
    if (ok && ty == 0) {
      float *o = part + ((a * S + seg) * C + c) * 2;
#pragma unroll
      for (int k = 0; k < VEC; ++k) { o[2 * k] = m[k]; o[2 * k + 1] = s[k]; }
    }
    return;
  }
  if (!ok) return;
#pragma unroll 8
  for (uint64_t b = b0 + ty; b < b1; b += TY) {
    float v[VEC];
    load(b, v);
    if constexpr (VEC > 1) {
      uint4 o;
      T *oe = reinterpret_cast<T *>(&o);
#pragma unroll
      for (int k = 0; k < VEC; ++k) oe[k] = Elem<T>::make(fast_exp(v[k] - m[k]) * inv[k]);
      store_stream(reinterpret_cast<uint4 *>(y + b * C), o);
    } else {
      y[b * C] = Elem<T>::make(fast_exp(v[0] - m[0]) * inv[0]);
    }
  }
}

// ws / ws_bytes: the caller's scratch for the segment partials (may be null); query: when not
// null nothing is launched and the scratch size for 16-byte aligned tensors is written there.
template <typename T>
hipError_t run_inner(const T *in, T *out, uint64_t A, uint64_t B, uint64_t C, void *ws, size_t ws_bytes, size_t *query,
                     hipStream_t stream) {
  constexpr int EPV = Elem<T>::EPV;
  const bool vec = C % EPV == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const uint64_t ncolv = vec ? C / EPV : C;
  // narrower tiles (more row lanes) while the grid would not fill the chip: measured faster than
  // wide tiles with the axis cut into segments ([4096, 65536] f32 over axis 0: 3.4 against 2.6 TB/s)
  int tx = 256;
  while (tx > 16 && (ncolv < (uint64_t)tx || A * ((ncolv + tx - 1) / tx) < 512)) tx /= 4;
  const uint64_t col_tiles = (ncolv + tx - 1) / tx;
  const int ty = kBlock / tx;
  // segments of B over workgroups when the column tiles alone leave the chip idle (at least
  // eight rows per lane and segment); the partials live in a stream-ordered allocation
  uint64_t S = 1;
  if (A * col_tiles < 512 && B >= (uint64_t)ty * 16) {
    S = (512 + A * col_tiles - 1) / (A * col_tiles);
    const uint64_t room = B / ((uint64_t)ty * 8);
    if (S > room) S = room;
    if (S > 1024) S = 1024;
  }
  uint64_t seg_rows = ((B + S - 1) / S + ty - 1) / ty * ty;
  S = (B + seg_rows - 1) / seg_rows;
  float *part = nullptr;
  bool owned = false;
  const size_t need = S > 1 ? (size_t)(A * S * C * 2) * sizeof(float) : 0;
  if (query) { *query = need; return hipSuccess; }
  if (need) {
    if (ws && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0 && ws_bytes >= need) part = static_cast<float *>(ws);
    else if (hipMallocAsync(reinterpret_cast<void **>(&part), need, stream) == hipSuccess) owned = true;
    else {
      (void)hipGetLastError();  // no scratch: one workgroup per column tile
      part = nullptr;
      S = 1;
      seg_rows = B;
    }
  }
  if (col_tiles > 0xffffffffull || A * col_tiles * S > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid((unsigned)(A * col_tiles * S)), block(kBlock);
#define INNER(V, X, M) BRT_ROCM_LAUNCH((softmax_inner_kernel<T, V, X, M>), grid, block, stream, in, out, B, C, (uint32_t)col_tiles, (uint32_t)S, seg_rows, part)
#define INNER_TX(V, M) do { if (tx == 256) INNER(V, 256, M); else if (tx == 64) INNER(V, 64, M); else INNER(V, 16, M); } while (0)
  hipError_t e = hipSuccess;
  if (S == 1) {
    if (vec) INNER_TX(EPV, 0); else INNER_TX(1, 0);
    e = hipGetLastError();
  } else {
    if (vec) INNER_TX(EPV, 1); else INNER_TX(1, 1);
    e = hipGetLastError();
    if (e == hipSuccess) {
      if (vec) INNER_TX(EPV, 2); else INNER_TX(1, 2);
      e = hipGetLastError();
    }
    if (owned) {
      const hipError_t f = hipFreeAsync(part, stream);
      if (e == hipSuccess) e = f;
    }
  }
#undef INNER_TX
#undef INNER
  return e;
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
    if (nvec <= 64) BRT_ROCM_LAUNCH((softmax_wave_kernel<T, 1>), grid, block, stream, in, out, rows, nv);
    else if (nvec <= 128) BRT_ROCM_LAUNCH((softmax_wave_kernel<T, 2>), grid, block, stream, in, out, rows, nv);
    else {
      // longer rows: RW waves per row, two vectors per lane
      const int rw = nvec <= 256 ? 2 : nvec <= 512 ? 4 : 8;
      const bool full = nvec == (uint64_t)rw * 128;
      const uint64_t rpb = kSplitWaves / rw, sblocks = (rows + rpb - 1) / rpb;
      if (sblocks > 0x7fffffffull) return hipErrorInvalidValue;
      const dim3 sgrid((unsigned)sblocks), sblock(kSplitWaves * 64);
#define SPLIT(RW)                                                                                \
  if (full) BRT_ROCM_LAUNCH((softmax_split_kernel<T, RW, true>), sgrid, sblock, stream, in, out, rows, nv);  \
  else BRT_ROCM_LAUNCH((softmax_split_kernel<T, RW, false>), sgrid, sblock, stream, in, out, rows, nv)
      if (rw == 2) { SPLIT(2); } else if (rw == 4) { SPLIT(4); } else { SPLIT(8); }
#undef SPLIT
    }
    return hipGetLastError();
  }
  if (rows > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid((unsigned)rows);
  // rows of input and output start at the same offset inside a 16-byte granule: vector accesses
  if (((reinterpret_cast<uintptr_t>(in) ^ reinterpret_cast<uintptr_t>(out)) & 15u) == 0 &&
      (reinterpret_cast<uintptr_t>(in) & (sizeof(T) - 1)) == 0) {
    const uint64_t span = (cols + 2 * (EPV - 1)) / EPV;  // vectors that cover a row wherever it starts
    const uint64_t xr = span * EPV;                      // floats a workgroup must hold
    // registers per thread and threads per workgroup are sized so that several workgroups share
    // a CU while the row is short enough, and one row's loads overlap another's stores
    if (xr <= 256 * 32) BRT_ROCM_LAUNCH((softmax_regs_kernel<T, 256, 32>), grid, dim3(256), stream, in, out, cols);
    else if (xr <= 256 * 64) BRT_ROCM_LAUNCH((softmax_regs_kernel<T, 256, 64>), grid, dim3(256), stream, in, out, cols);
    else if (xr <= 1024 * 32) BRT_ROCM_LAUNCH((softmax_regs_kernel<T, 1024, 32>), grid, dim3(1024), stream, in, out, cols);
    else BRT_ROCM_LAUNCH((softmax_stream_kernel<T, 1024>), grid, dim3(1024), stream, in, out, cols);
    return hipGetLastError();
  }
  BRT_ROCM_LAUNCH((softmax_block_kernel<T>), grid, dim3(kBlock), stream, in, out, cols);
  return hipGetLastError();
}

}  // namespace

namespace {
int softmax_axis_impl(int dtype, const void *input, void *output, size_t A, size_t B, size_t C, void *ws, size_t ws_bytes,
                      size_t *query, void *stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (query) *query = 0;
  if (C == 1) return query ? hipSuccess : brt_rocm_softmax(dtype, input, output, A, B, stream_);
  if (A == 0 || B == 0 || C == 0) return hipSuccess;
  if (!query && (!input || !output)) return hipErrorInvalidValue;
  switch (dtype) {
  case BRT_ROCM_F32:
    return run_inner(static_cast<const float *>(input), static_cast<float *>(output), A, B, C, ws, ws_bytes, query, stream);
  case BRT_ROCM_F16:
    return run_inner(static_cast<const __half *>(input), static_cast<__half *>(output), A, B, C, ws, ws_bytes, query, stream);
  case BRT_ROCM_BF16:
    return run_inner(static_cast<const __bf16 *>(input), static_cast<__bf16 *>(output), A, B, C, ws, ws_bytes, query, stream);
  default:
    return hipErrorInvalidValue;
  }
}
}  // namespace

extern "C" int brt_rocm_softmax_axis(int dtype, const void *input, void *output, size_t A, size_t B,
                                     size_t C, void *stream) {
  return softmax_axis_impl(dtype, input, output, A, B, C, nullptr, 0, nullptr, stream);
}
extern "C" int brt_rocm_softmax_axis_ws(int dtype, const void *input, void *output, size_t A, size_t B, size_t C,
                                        void *workspace, size_t workspace_bytes, void *stream) {
  return softmax_axis_impl(dtype, input, output, A, B, C, workspace, workspace_bytes, nullptr, stream);
}
extern "C" size_t brt_rocm_softmax_workspace_bytes(int dtype, size_t A, size_t B, size_t C) {
  size_t n = 0;
  return softmax_axis_impl(dtype, nullptr, nullptr, A, B, C, nullptr, 0, &n, nullptr) == hipSuccess ? n : 0;
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
