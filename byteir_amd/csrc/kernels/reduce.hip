// Reduction kernels of the ROCm provider: out[a, c] = fold_b in[a, b, c] over a dense
// row-major [A, B, C] view, for gfx950 (wave64).
//
// Two kernels cover every shape:
//   * reduce_row_kernel  (C == 1): G lanes cooperate on one row segment with 128-bit loads,
//     several loads in flight per lane, then a wave shuffle tree (and one LDS hop when a
//     whole 256-thread block shares a row).
//   * reduce_col_kernel  (C > 1): each lane owns a 128-bit group of adjacent columns, a wave
//     spans 1 KiB of contiguous columns, the waves of a block interleave rows; partial
//     results meet in LDS.
// When one pass cannot fill the chip (few outputs, long fold axis) the fold axis is split in
// S segments whose float partials go to the caller's workspace, and the same kernels run a
// second, tiny pass over [A, S, C].  The split depends only on (dtype, A, B, C), so the
// workspace can be sized when an execution plan is built.
//
// Semantics follow the reference's operators
// (runtime/lib/backends/cuda/providers/default/reduction/kernels/reduction_helper.h:18-36,158-179):
// sum starts from 0, max from -inf and returns NaN when either operand is NaN; f16 folds in
// float (reduce_impl.h:64-69).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>

#include <cstdint>
#include <type_traits>

#include "brt_rocm_kernels.h"
#include "launch.h"
#include "brt_rocm_bench.h"

namespace {

// 128-bit loads in flight per lane.  Four measured fastest for both kernels on MI355X: with
// about 512 resident workgroups that is 8 MB in flight chip-wide, and deeper queues lose
// HBM efficiency (79 us against 82 us with eight for the [16384, 8192] column fold).
constexpr int kRowU = 4;
constexpr int kColU = 4;
constexpr int kColWideU = 2;  // rows in flight per lane and column group, wide kernel
constexpr int kBlock = 256;            // threads per workgroup (4 waves)
constexpr uint64_t kFillThreads = 256ull * 1024;  // threads wanted in flight chip-wide

// A fold operator: init, apply (associative up to rounding), map (applied to every element as
// it is read from the tensor, never to partials) and finish (applied once, to the final value,
// with the fold length as a float).
struct FoldPlain {
  static __device__ __forceinline__ float map(float x) { return x; }
  static __device__ __forceinline__ float finish(float r, float) { return r; }
};
template <int OP> struct Fold;
template <> struct Fold<BRT_ROCM_REDUCE_SUM> : FoldPlain {
  static __device__ __forceinline__ float init() { return 0.f; }
  static __device__ __forceinline__ float apply(float l, float r) { return l + r; }
};
template <> struct Fold<BRT_ROCM_REDUCE_MAX> : FoldPlain {
  static __device__ __forceinline__ float init() { return -INFINITY; }
  static __device__ __forceinline__ float apply(float l, float r) {
    return (l != l || l > r) ? l : r;  // NaN on either side wins
  }
};
template <> struct Fold<BRT_ROCM_REDUCE_MIN> : FoldPlain {
  static __device__ __forceinline__ float init() { return INFINITY; }
  static __device__ __forceinline__ float apply(float l, float r) {
    return (l != l || l < r) ? l : r;  // NaN on either side wins
  }
};
template <> struct Fold<BRT_ROCM_REDUCE_PROD> : FoldPlain {
  static __device__ __forceinline__ float init() { return 1.f; }
  static __device__ __forceinline__ float apply(float l, float r) { return l * r; }
};
template <> struct Fold<BRT_ROCM_REDUCE_MEAN> : Fold<BRT_ROCM_REDUCE_SUM> {
  static __device__ __forceinline__ float finish(float r, float len) { return r / len; }
};
template <> struct Fold<BRT_ROCM_REDUCE_SUMSQR> : Fold<BRT_ROCM_REDUCE_SUM> {
  static __device__ __forceinline__ float map(float x) { return x * x; }
};
// With partials in a workspace the first pass maps and the second one finishes.
template <int OP> struct Passes { static constexpr int first = OP, second = OP; };
template <> struct Passes<BRT_ROCM_REDUCE_MEAN> {
  static constexpr int first = BRT_ROCM_REDUCE_SUM, second = BRT_ROCM_REDUCE_MEAN;
};
template <> struct Passes<BRT_ROCM_REDUCE_SUMSQR> {
  static constexpr int first = BRT_ROCM_REDUCE_SUMSQR, second = BRT_ROCM_REDUCE_SUM;
};

// ---- typed loads into float -----------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
template <typename T, int VEC> struct Loader;
template <> struct Loader<float, 4> {
  static __device__ __forceinline__ void load(const float *p, float (&v)[4]) {
    // streamed once: a non-temporal load keeps the data from displacing cache lines
    const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
};
template <> struct Loader<float, 1> {
  static __device__ __forceinline__ void load(const float *p, float (&v)[1]) { v[0] = *p; }
  static __device__ __forceinline__ float get(const float *p) { return *p; }
};
template <> struct Loader<__half, 8> {
  static __device__ __forceinline__ void load(const __half *p, float (&v)[8]) {
    const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    const __half2 *h = reinterpret_cast<const __half2 *>(&t);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float2 f = __half22float2(h[i]);
      v[2 * i] = f.x; v[2 * i + 1] = f.y;
    }
  }
};
template <> struct Loader<__half, 1> {
  static __device__ __forceinline__ void load(const __half *p, float (&v)[1]) { v[0] = __half2float(*p); }
  static __device__ __forceinline__ float get(const __half *p) { return __half2float(*p); }
};

template <typename TO> __device__ __forceinline__ TO to_out(float v);
template <> __device__ __forceinline__ float to_out<float>(float v) { return v; }
template <> __device__ __forceinline__ __half to_out<__half>(float v) { return __float2half_rn(v); }

template <int OP> __device__ __forceinline__ float wave_fold(float r, int width) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
    if (off < width) r = Fold<OP>::apply(r, __shfl_xor(r, off, 64));
  return r;
}

// Workgroup ids go round-robin over the 8 XCDs of the chip; this gives each XCD a contiguous
// eighth of the launch instead of every eighth workgroup.
#ifndef REDUCE_XCD_CONTIG
#define REDUCE_XCD_CONTIG 1
#endif
__device__ __forceinline__ uint32_t xcd_contiguous(uint32_t b, uint32_t n) {
#if REDUCE_XCD_CONTIG
  return (n & 7u) == 0 ? (b & 7u) * (n >> 3) + (b >> 3) : b;
#else
  return b;
#endif
}

// ---- rows: C == 1 -----------------------------------------------------------------------
// unit = a * S + s; G lanes fold in[a, s*seg_len : min(B, (s+1)*seg_len)] into out[unit].
// PEEL: the segment may start and end anywhere (a row length that is no multiple of the vector,
// or an unaligned tensor): the elements before the first 16-byte boundary and after the last
// are folded one by one, the aligned body with the same 128-bit loads.
template <typename T, typename TO, int OP, int VEC, int G, bool PEEL>
__global__ void __launch_bounds__(kBlock)
reduce_row_kernel(const T *__restrict__ in, TO *__restrict__ out, uint64_t units, uint64_t B,
                  uint32_t S, uint64_t seg_len, float len) {
  constexpr int GPB = kBlock / G;
  constexpr int U = kRowU;
  const int lane = threadIdx.x % G;
  uint64_t unit = (uint64_t)xcd_contiguous(blockIdx.x, gridDim.x) * GPB + threadIdx.x / G;
  const bool valid = unit < units;
  if (!valid) unit = units - 1;  // surplus groups redo the last unit so shuffles stay whole
  const uint64_t a = unit / S, s = unit % S;
  uint64_t begin = s * seg_len;
  uint64_t end = begin + seg_len;
  if (end > B) end = B;
  const T *row = in + a * B;

  float acc[U];
#pragma unroll
  for (int u = 0; u < U; ++u) acc[u] = Fold<OP>::init();
  if constexpr (PEEL) {
    const uint64_t n = end - begin;
    uint64_t head = ((16 - (reinterpret_cast<uintptr_t>(row + begin) & 15)) & 15) / sizeof(T);
    if (head > n) head = n;
    const uint64_t tail = (n - head) % VEC;
    for (uint64_t e = lane; e < head; e += G) acc[0] = Fold<OP>::apply(acc[0], Fold<OP>::map(Loader<T, 1>::get(row + begin + e)));
    for (uint64_t e = lane; e < tail; e += G) acc[1] = Fold<OP>::apply(acc[1], Fold<OP>::map(Loader<T, 1>::get(row + end - tail + e)));
    begin += head;
    end -= tail;
  }
  const uint64_t step = (uint64_t)G * VEC;
  uint64_t i = begin + (uint64_t)lane * VEC;
  for (; i + (U - 1) * step < end; i += U * step) {
    float v[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) Loader<T, VEC>::load(row + i + u * step, v[u]);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[u] = Fold<OP>::apply(acc[u], Fold<OP>::map(v[u][k]));
  }
  for (; i < end; i += step) {
    float v[VEC];
    Loader<T, VEC>::load(row + i, v);
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[0] = Fold<OP>::apply(acc[0], Fold<OP>::map(v[k]));
  }
  float r = acc[0];
#pragma unroll
  for (int u = 1; u < U; ++u) r = Fold<OP>::apply(r, acc[u]);
  if constexpr (G <= 64) {
    r = wave_fold<OP>(r, G);
  } else {
    static_assert(G == kBlock, "a unit is shared by lanes of one wave or by the whole block");
    __shared__ float part[kBlock / 64];
    r = wave_fold<OP>(r, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = r;
    __syncthreads();
    r = Fold<OP>::apply(Fold<OP>::apply(part[0], part[1]), Fold<OP>::apply(part[2], part[3]));
  }
  if (valid && lane == 0) out[unit] = to_out<TO>(Fold<OP>::finish(r, len));
}

// ---- columns: C > 1 ---------------------------------------------------------------------
// block = (column tile, segment s, a); lane (tx, ty) folds rows ty, ty+TY, ... of its segment
// for VEC adjacent columns; out[(a*S + s)*C + c].
template <typename T, typename TO, int OP, int VEC, int TX>
__global__ void __launch_bounds__(kBlock)
reduce_col_kernel(const T *__restrict__ in, TO *__restrict__ out, uint64_t B, uint64_t C,
                  uint32_t S, uint64_t seg_rows, uint32_t col_tiles, float len) {
  constexpr int TY = kBlock / TX;
  constexpr int U = VEC == 1 ? 4 * kColU : kColU;  // scalar loads: as many bytes in flight as with vectors
  __shared__ float part[TY][TX * VEC + 1];
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  uint64_t bid = blockIdx.x;
  const uint32_t tile = bid % col_tiles; bid /= col_tiles;
  const uint32_t s = bid % S;
  const uint64_t a = bid / S;
  const uint64_t c = ((uint64_t)tile * TX + tx) * VEC;
  const bool col_ok = c < C;
  const uint64_t r0 = (uint64_t)s * seg_rows;
  uint64_t r1 = r0 + seg_rows;
  if (r1 > B) r1 = B;

  float acc[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) acc[k] = Fold<OP>::init();
  if (col_ok) {
    const T *p = in + a * B * C + c;
    uint64_t r = r0 + ty;
    for (; r + (uint64_t)(U - 1) * TY < r1; r += (uint64_t)U * TY) {
      float v[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) Loader<T, VEC>::load(p + (r + (uint64_t)u * TY) * C, v[u]);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] = Fold<OP>::apply(acc[k], Fold<OP>::map(v[u][k]));
    }
    for (; r < r1; r += TY) {
      float v[VEC];
      Loader<T, VEC>::load(p + r * C, v);
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[k] = Fold<OP>::apply(acc[k], Fold<OP>::map(v[k]));
    }
  }
#pragma unroll
  for (int k = 0; k < VEC; ++k) part[ty][tx * VEC + k] = acc[k];
  __syncthreads();
  // TX*VEC columns remain, TY partials each: lane j folds column j (coalesced store)
  for (int j = threadIdx.x; j < TX * VEC; j += kBlock) {
    float r = part[0][j];
#pragma unroll 4
    for (int y = 1; y < TY; ++y) r = Fold<OP>::apply(r, part[y][j]);
    const uint64_t cj = (uint64_t)tile * TX * VEC + j;
    if (cj < C) out[(a * S + s) * C + cj] = to_out<TO>(Fold<OP>::finish(r, len));
  }
}

// Wide tensors: a block of 256 lanes spans W * 4 KiB of a row, every lane owns W groups of
// VEC adjacent columns 256 * VEC apart and keeps U rows in flight (W * U 128-bit loads per
// lane).  No LDS: every lane stores its own columns.  Several groups with two rows in flight
// measured fastest for the [16384, 8192] fold: 77.3 us with two groups on 512 workgroups and
// 76.8 us with four groups on 256, against 79.6 us with one group and four rows.
template <typename T, typename TO, int OP, int VEC, int W, int U>
__global__ void __launch_bounds__(kBlock)
reduce_colwide_kernel(const T *__restrict__ in, TO *__restrict__ out, uint64_t B, uint64_t C,
                      uint32_t S, uint64_t seg_rows, uint32_t col_tiles, float len) {
  uint64_t bid = xcd_contiguous(blockIdx.x, gridDim.x);
  const uint32_t tile = bid % col_tiles; bid /= col_tiles;
  const uint32_t s = bid % S;
  const uint64_t a = bid / S;
  const uint64_t c0 = ((uint64_t)tile * W * kBlock + threadIdx.x) * VEC;  // first group of this lane
  constexpr uint64_t kGroupStep = (uint64_t)kBlock * VEC;
  const uint64_t r0 = (uint64_t)s * seg_rows;
  uint64_t r1 = r0 + seg_rows;
  if (r1 > B) r1 = B;
  const T *p = in + a * B * C + c0;
  TO *o = out + (a * S + s) * C + c0;
  // full: the whole tile lies inside the row (block-uniform), so the loads need no predicate
  auto fold = [&](auto full_tag) {
    constexpr bool kFull = decltype(full_tag)::value;
    bool ok[W];
#pragma unroll
    for (int w = 0; w < W; ++w) ok[w] = kFull || c0 + w * kGroupStep < C;
    float acc[W][VEC];
#pragma unroll
    for (int w = 0; w < W; ++w)
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[w][k] = Fold<OP>::init();
    uint64_t r = r0;
    for (; r + (U - 1) < r1; r += U) {
      float v[U][W][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int w = 0; w < W; ++w)
          if (kFull || ok[w]) Loader<T, VEC>::load(p + (r + u) * C + w * kGroupStep, v[u][w]);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int w = 0; w < W; ++w)
          if (kFull || ok[w]) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[w][k] = Fold<OP>::apply(acc[w][k], Fold<OP>::map(v[u][w][k]));
          }
    }
    for (; r < r1; ++r) {
#pragma unroll
      for (int w = 0; w < W; ++w)
        if (kFull || ok[w]) {
          float v[VEC];
          Loader<T, VEC>::load(p + r * C + w * kGroupStep, v);
#pragma unroll
          for (int k = 0; k < VEC; ++k) acc[w][k] = Fold<OP>::apply(acc[w][k], Fold<OP>::map(v[k]));
        }
    }
#pragma unroll
    for (int w = 0; w < W; ++w)
      if (kFull || ok[w]) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) o[w * kGroupStep + k] = to_out<TO>(Fold<OP>::finish(acc[w][k], len));
      }
  };
  if (((uint64_t)tile + 1) * W * kGroupStep <= C) fold(std::true_type{});
  else fold(std::false_type{});
}

// An empty fold axis: every output is the operator's identity run through finish().
template <typename TO>
__global__ void __launch_bounds__(kBlock) reduce_fill_kernel(TO *__restrict__ out, uint64_t n, float value) {
  const uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) out[i] = to_out<TO>(value);
}

// ---- host-side planning -------------------------------------------------------------------
struct Plan {
  int kind;       // 0 copy, 1 row, 2 col, 3 wide col (reduce_colwide_kernel)
  int vec;        // elements per load when pointers are 16-byte aligned
  int g;          // row: lanes per unit; col: TX
  uint32_t S;     // segments of the fold axis
  uint64_t seg;   // row: elements per segment; col: rows per segment
  uint32_t col_tiles;
};

inline uint64_t ceil_div(uint64_t a, uint64_t b) { return (a + b - 1) / b; }
inline uint64_t round_up(uint64_t a, uint64_t b) { return ceil_div(a, b) * b; }

Plan make_plan(int dtype, uint64_t A, uint64_t B, uint64_t C, bool allow_split) {
  Plan p{};
  if (!(A && B && C)) { p.kind = 0; p.S = 1; return p; }  // copy, fill or nothing: no workspace
  const int vec_full = dtype == BRT_ROCM_F32 ? 4 : 8;
  if (C == 1) {
    p.kind = 1;
    p.vec = (B % vec_full == 0) ? vec_full : 1;  // 1: rows start off the 16-byte grid, peeled kernel
    const uint64_t nvec = ceil_div(B, vec_full);
    p.g = nvec >= 2048 ? 256 : nvec >= 96 ? 64 : nvec >= 24 ? 16 : 4;
    uint64_t S = 1;
    if (allow_split && A * p.g < kFillThreads) {
      const uint64_t want = ceil_div(kFillThreads, A * p.g);
      const uint64_t room = nvec / ((uint64_t)p.g * 8);  // keep >= 8 loads per lane per segment
      S = want < room ? want : room;
      if (S < 1) S = 1;
      if (S > 1024) S = 1024;
    }
    p.seg = round_up(ceil_div(B, S), (uint64_t)p.g * vec_full);
    p.S = (uint32_t)ceil_div(B, p.seg);
    return p;
  }
  p.kind = 2;
  p.vec = (C % vec_full == 0) ? vec_full : 1;
  const uint64_t ncolv = ceil_div(C, p.vec);
  if (allow_split && p.vec > 1 && ncolv >= 2 * kBlock) {
    p.kind = 3;  // 8 or 16 KiB of a row per block (two or four column groups per lane)
    p.g = (ncolv >= 4 * kBlock ? 4 : 2) * kBlock;
  } else if (allow_split) {
    // first (or only) pass: a block spans up to 256 lanes x 128 bits = 4 KiB of one row
    p.g = ncolv >= 256 ? 256 : ncolv > 32 ? 64 : ncolv > 8 ? 32 : 8;
  } else {
    // second pass over few rows of partials: narrow tiles so that enough blocks exist
    p.g = 64;
    if (A * ceil_div(ncolv, 64) < 256) p.g = 32;
    if (A * ceil_div(ncolv, 32) < 256) p.g = 8;
  }
  const int ty = p.kind == 3 ? 1 : kBlock / p.g;
  p.col_tiles = (uint32_t)ceil_div(ncolv, p.g);
  const uint64_t blocks0 = A * p.col_tiles;
  uint64_t S = 1;
  // Long sequential streams from about two resident workgroups per CU measured fastest on
  // MI355X (more, shorter segments lose HBM efficiency), so the split aims at 512 workgroups;
  // with four column groups per lane a workgroup keeps as many loads in flight as two of the
  // others, and one per CU is enough.
  const uint64_t kWantBlocks = (p.kind == 3 && p.g == 4 * kBlock) ? 256 : 512;
  if (allow_split && blocks0 < kWantBlocks && B > (uint64_t)ty * 8) {
    const uint64_t want = ceil_div(kWantBlocks, blocks0);
    const uint64_t room = ceil_div(B, (uint64_t)ty * 8);
    S = want < room ? want : room;
    if (S > 1024) S = 1024;
  }
  p.seg = round_up(ceil_div(B, S), ty);
  p.S = (uint32_t)ceil_div(B, p.seg);
  return p;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T, typename TO, int OP>
hipError_t launch(const Plan &p, const T *in, TO *out, uint64_t A, uint64_t B, uint64_t C,
                  float len, hipStream_t stream) {
  constexpr int VF = sizeof(T) == 4 ? 4 : 8;
  const bool vec = p.vec > 1 && aligned16(in);
  if (p.kind == 1) {
    const uint64_t units = A * p.S;
    const uint64_t blocks = ceil_div(units, kBlock / p.g);
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks), block(kBlock);
#define ROW(G)                                                                                   \
  if (vec) BRT_ROCM_LAUNCH((reduce_row_kernel<T, TO, OP, VF, G, false>), grid, block, stream, in, out, units, B, p.S, p.seg, len); \
  else BRT_ROCM_LAUNCH((reduce_row_kernel<T, TO, OP, VF, G, true>), grid, block, stream, in, out, units, B, p.S, p.seg, len)
    switch (p.g) {
    case 4: ROW(4); break;
    case 16: ROW(16); break;
    case 64: ROW(64); break;
    default: ROW(256); break;
    }
#undef ROW
    return hipGetLastError();
  }
  // The plan counts column tiles in 128-bit groups; a pointer that is not 16-byte aligned
  // forces scalar loads at launch time, and the same segments are then covered by four (f32)
  // or eight (f16) times as many tiles of the 256-lane kernel.
  const int tx = (p.kind == 3 && !vec) ? kBlock : p.g;
  const uint32_t col_tiles = vec ? p.col_tiles : (uint32_t)ceil_div(C, (uint64_t)tx);
  const uint64_t blocks = A * p.S * col_tiles;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid((unsigned)blocks), block(kBlock);
  if (p.kind == 3 && vec) {
    if (p.g == 4 * kBlock) BRT_ROCM_LAUNCH((reduce_colwide_kernel<T, TO, OP, VF, 4, kColWideU>), grid, block, stream, in, out, B, C, p.S, p.seg, col_tiles, len);
    else BRT_ROCM_LAUNCH((reduce_colwide_kernel<T, TO, OP, VF, 2, kColWideU>), grid, block, stream, in, out, B, C, p.S, p.seg, col_tiles, len);
    return hipGetLastError();
  }
#define COL(TX)                                                                                  \
  if (vec) BRT_ROCM_LAUNCH((reduce_col_kernel<T, TO, OP, VF, TX>), grid, block, stream, in, out, B, C, p.S, p.seg, col_tiles, len); \
  else BRT_ROCM_LAUNCH((reduce_col_kernel<T, TO, OP, 1, TX>), grid, block, stream, in, out, B, C, p.S, p.seg, col_tiles, len)
  switch (tx) {
  case 8: COL(8); break;
  case 32: COL(32); break;
  case 256: COL(256); break;
  default: COL(64); break;
  }
#undef COL
  return hipGetLastError();
}

template <typename T, int OP>
hipError_t run(const T *in, T *out, uint64_t A, uint64_t B, uint64_t C, void *ws, size_t ws_bytes,
               int dtype, hipStream_t stream, hipEvent_t first_pass_done) {
  const Plan p = make_plan(dtype, A, B, C, true);
  const float len = static_cast<float>(B);  // MeanOp divides by static_cast<wtype>(B)
  if (p.S == 1) {
    const hipError_t e = launch<T, T, OP>(p, in, out, A, B, C, len, stream);
    if (e == hipSuccess && first_pass_done) return hipEventRecord(first_pass_done, stream);
    return e;
  }
  const size_t need = sizeof(float) * A * p.S * C;
  if (ws == nullptr || ws_bytes < need) return hipErrorInvalidValue;
  float *part = static_cast<float *>(ws);
  hipError_t e = launch<T, float, Passes<OP>::first>(p, in, part, A, B, C, len, stream);
  if (e != hipSuccess) return e;
  if (first_pass_done && (e = hipEventRecord(first_pass_done, stream)) != hipSuccess) return e;
  const Plan p2 = make_plan(BRT_ROCM_F32, A, p.S, C, false);
  return launch<float, T, Passes<OP>::second>(p2, part, out, A, p.S, C, len, stream);
}

}  // namespace

// The first-pass kernel a fold of 16-byte aligned tensors is planned with, spelled the way a
// profiler prints the instantiation (the operator as OP), and the split: what a stored counter
// profile must name to be valid for today's library.
extern "C" int brt_rocm_reduce_plan_describe(int dtype, size_t A, size_t B, size_t C, char *buf, size_t len) {
  if (!buf || len == 0 || (dtype != BRT_ROCM_F32 && dtype != BRT_ROCM_F16)) return hipErrorInvalidValue;
  const Plan p = make_plan(dtype, A, B, C, true);
  const char *t = dtype == BRT_ROCM_F32 ? "float" : "__half";
  const char *to = p.S > 1 ? "float" : t;
  const int vf = dtype == BRT_ROCM_F32 ? 4 : 8;
  int n = 0;
  if (p.kind == 1) n = snprintf(buf, len, "reduce_row_kernel<%s, %s, OP, %d, %d, %s> S=%u", t, to, vf, p.g, p.vec > 1 ? "false" : "true", p.S);
  else if (p.kind == 3) n = snprintf(buf, len, "reduce_colwide_kernel<%s, %s, OP, %d, %d, %d> S=%u col_tiles=%u", t, to, vf, p.g / kBlock, kColWideU, p.S, p.col_tiles);
  else if (p.kind == 2) n = snprintf(buf, len, "reduce_col_kernel<%s, %s, OP, %d, %d> S=%u col_tiles=%u", t, to, p.vec > 1 ? vf : 1, p.g, p.S, p.col_tiles);
  else n = snprintf(buf, len, "copy or fill");
  return n > 0 && (size_t)n < len ? 0 : hipErrorInvalidValue;
}

extern "C" size_t brt_rocm_reduce_workspace_bytes(int dtype, size_t A, size_t B, size_t C) {
  if (dtype != BRT_ROCM_F32 && dtype != BRT_ROCM_F16) return 0;
  const Plan p = make_plan(dtype, A, B, C, true);
  return p.S > 1 ? sizeof(float) * A * p.S * C : 0;
}

extern "C" int brt_rocm_reduce_ex(int op, int dtype, const void *input, void *output, size_t A,
                                  size_t B, size_t C, void *workspace, size_t workspace_bytes,
                                  void *stream_, void *first_pass_done_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  hipEvent_t first_pass_done = static_cast<hipEvent_t>(first_pass_done_);
  if (op < BRT_ROCM_REDUCE_SUM || op > BRT_ROCM_REDUCE_SUMSQR ||
      (dtype != BRT_ROCM_F32 && dtype != BRT_ROCM_F16))
    return hipErrorInvalidValue;
  const size_t es = dtype == BRT_ROCM_F32 ? 4 : 2;
  if (A == 0 && B == 0) {  // nothing to fold: copy C elements (reduce_impl.h:55-58,71-74)
    if (C == 0) return hipSuccess;
    if (!input || !output) return hipErrorInvalidValue;
    return hipMemcpyAsync(output, input, C * es, hipMemcpyDeviceToDevice, stream);
  }
  if (A == 0 || C == 0) return hipSuccess;  // no output element
  if (B == 0) {
    // An empty fold axis.  The reference sends this to its copy branch too, which reads C
    // elements of an input that has none; here every output gets the operator's identity.
    if (!output) return hipErrorInvalidValue;
    float value = 0.f;
    switch (op) {
    case BRT_ROCM_REDUCE_MAX: value = -INFINITY; break;
    case BRT_ROCM_REDUCE_MIN: value = INFINITY; break;
    case BRT_ROCM_REDUCE_PROD: value = 1.f; break;
    case BRT_ROCM_REDUCE_MEAN: value = NAN; break;  // 0 / float(0)
    default: break;
    }
    const uint64_t n = (uint64_t)A * C, blocks = (n + kBlock - 1) / kBlock;
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    if (dtype == BRT_ROCM_F32) BRT_ROCM_LAUNCH((reduce_fill_kernel<float>), dim3((unsigned)blocks), dim3(kBlock), stream, static_cast<float *>(output), n, value);
    else BRT_ROCM_LAUNCH((reduce_fill_kernel<__half>), dim3((unsigned)blocks), dim3(kBlock), stream, static_cast<__half *>(output), n, value);
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess && first_pass_done) return hipEventRecord(first_pass_done, stream);
    return e;
  }
  if (!input || !output) return hipErrorInvalidValue;
#define RUN(T, OP) \
  case OP: return run<T, OP>(in, out, A, B, C, workspace, workspace_bytes, dtype, stream, first_pass_done)
#define RUN_ALL(T)                                                                               \
  switch (op) {                                                                                  \
    RUN(T, BRT_ROCM_REDUCE_SUM); RUN(T, BRT_ROCM_REDUCE_MAX); RUN(T, BRT_ROCM_REDUCE_MIN);       \
    RUN(T, BRT_ROCM_REDUCE_PROD); RUN(T, BRT_ROCM_REDUCE_MEAN); RUN(T, BRT_ROCM_REDUCE_SUMSQR);  \
  }
  if (dtype == BRT_ROCM_F32) {
    const float *in = static_cast<const float *>(input);
    float *out = static_cast<float *>(output);
    RUN_ALL(float)
  } else {
    const __half *in = static_cast<const __half *>(input);
    __half *out = static_cast<__half *>(output);
    RUN_ALL(__half)
  }
#undef RUN_ALL
#undef RUN
  return hipErrorInvalidValue;
}

extern "C" int brt_rocm_reduce(int op, int dtype, const void *input, void *output, size_t A,
                               size_t B, size_t C, void *workspace, size_t workspace_bytes,
                               void *stream) {
  return brt_rocm_reduce_ex(op, dtype, input, output, A, B, C, workspace, workspace_bytes, stream, nullptr);
}

// ---- the call that allocates nothing ------------------------------------------------------
// Partials of the split first pass live in a device array that is part of the code object, so
// every GPU the library is loaded on holds its own copy for the life of the process.  In host
// code the array's name is only a handle for hipGetSymbolAddress; kernels get the address that
// call returns, looked up once per device and kept.
namespace {
static __device__ __align__(256) float scratch[BRT_ROCM_REDUCE_STATIC_SCRATCH_BYTES / sizeof(float)];
constexpr int kMaxDevices = 64;
std::atomic<float *> g_scratch_ptr[kMaxDevices];

hipError_t static_scratch(float **ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  float *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void *sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));  // address on the current device
    if (e != hipSuccess) return e;
    if (sym == nullptr) return hipErrorInvalidSymbol;
    p = static_cast<float *>(sym);
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing first calls store the same value
  }
  *ptr = p;
  return hipSuccess;
}
}  // namespace

extern "C" int brt_rocm_reduce_static(int op, int dtype, const void *input, void *output, size_t A,
                                      size_t B, size_t C, void *stream) {
  if (dtype != BRT_ROCM_F32 && dtype != BRT_ROCM_F16) return hipErrorInvalidValue;
  const size_t need = brt_rocm_reduce_workspace_bytes(dtype, A, B, C);
  if (need > BRT_ROCM_REDUCE_STATIC_SCRATCH_BYTES) return BRT_ROCM_ERROR_STATIC_SCRATCH_TOO_SMALL;
  float *ws = nullptr;
  if (need) {
    const hipError_t e = static_scratch(&ws);
    if (e != hipSuccess) return e;
  }
  // Every partial the second pass reads is written by the first pass of the same call, so
  // nothing in the array has to start at zero.
  return brt_rocm_reduce_ex(op, dtype, input, output, A, B, C, ws, need, stream, nullptr);
}
