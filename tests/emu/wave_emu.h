// Host execution of the wave64 HIP kernels in this directory, for tests that need no GPU.
//
// The .hip sources are compiled unchanged by a host C++ compiler with this header in place of
// <hip/hip_runtime.h>.  A kernel launch (FA_LAUNCH) runs the grid's workgroups one after the
// other; inside a workgroup every lane is a fiber (ucontext) with its own stack, so the kernel
// body runs as written, lane by lane.  The few operations that exchange data between lanes
// (MFMA, the transposing LDS read, ballot, lane permutes, barriers) are rendezvous points: a
// lane deposits its operands and yields; the last lane of the wave to arrive computes the
// result for all 64 from the documented register layouts and everybody resumes.  LDS arrays are
// function-local statics, shared by all fibers because they run on one thread.
//
// What this is for: (1) parity of the kernels' logic against the CPU oracle without a GPU;
// (2) bounds: tensors handed in through emu_guarded_alloc end at a protected page (or begin
// behind one), buffer loads apply the hardware's range check and then must hit a registered
// allocation, and a stray access is reported with the workgroup and thread that made it.
// What it is not: a timing model, or a model of anything the hardware does that the ISA
// documents leave open (it rounds an MFMA once from a double accumulation).
//
// One launch at a time, from one thread: the scheduler's state is global.  A stray access is
// caught by a SIGSEGV handler that leaves the faulting lane through setcontext (Linux).
//
// All lanes of a wave must reach the same cross-lane operations in the same order (true for
// these kernels: their divergent branches contain none); a mismatch or a deadlock is detected
// and reported, not silently mis-executed.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>

namespace fa_emu {

struct dim3 {
  unsigned x, y, z;
  constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

// ---- state of the lane that is running (set by the scheduler at every switch) -----------------
extern dim3 g_thread_idx, g_block_idx, g_block_dim, g_grid_dim;

// Runs `body` once per lane of every selected workgroup of the grid.  Returns 0, or -1 after a
// fault (stray memory access, deadlock, mismatched cross-lane operation): see last_error().
int launch(dim3 grid, dim3 block, const std::function<void()> &body);
const char *last_error();

// ---- rendezvous ------------------------------------------------------------------------------
// Every lane of the running wave calls this with the same `op`; `fn(in, out, n)` runs once, on
// the last arrival, with the operand and result pointers of all n lanes (index = lane id).
void wave_rendezvous(const char *op, const void *in, void *out,
                     void (*fn)(const void *const *in, void *const *out, int n_lanes, void *ctx), void *ctx = nullptr);
void block_barrier();
void wave_sync();  // all lanes of the running wave arrive before any goes on

// ---- global memory ---------------------------------------------------------------------------
// Memory that ends at a protected page (`at_end`) or starts right behind one, 16-byte aligned
// either way, and is entered in the table that buffer loads are checked against.
void *guarded_alloc(size_t bytes, bool at_end);
void guarded_free(void *p);
void register_range(const void *p, size_t bytes);   // memory the caller owns, e.g. a numpy array
void unregister_range(const void *p);
bool range_ok(const void *p, size_t bytes);          // inside one registered range (true when none is registered)
[[noreturn]] void fail(const char *what, const void *addr);

struct BufferRsrc {
  const char *base;
  uint32_t num_records;
};

typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

inline BufferRsrc make_buffer_rsrc(const void *p, int /*stride*/, uint32_t num_records, unsigned /*flags*/) {
  return BufferRsrc{static_cast<const char *>(p), num_records};
}
// Raw buffer load of 16 bytes: the vector offset is range-checked against the descriptor (an
// access that does not lie wholly inside [0, num_records) returns zeros), the scalar offset is
// added unchecked, as the hardware does.
inline u32x4_t raw_buffer_load_b128(const BufferRsrc &r, uint32_t voffset, uint32_t soffset, int /*aux*/) {
  if ((uint64_t)voffset + 16 > r.num_records) return u32x4_t{0, 0, 0, 0};
  const char *p = r.base + (uint64_t)voffset + soffset;
  if (!range_ok(p, 16)) fail("buffer load that passed the descriptor's range check lies outside every tensor", p);
  u32x4_t v;
  std::memcpy(&v, p, 16);
  return v;
}

f32x16_t mfma_32x32x16_f16(f16x8_t a, f16x8_t b, f32x16_t c, int cbsz = 0, int abid = 0, int blgp = 0);
f32x16_t mfma_32x32x16_bf16(bf16x8_t a, bf16x8_t b, f32x16_t c, int cbsz = 0, int abid = 0, int blgp = 0);
s16x4_t ds_read_tr16_b64(const void *lds_ptr);
uint64_t ballot_w64(bool pred);
unsigned readfirstlane(unsigned v);
u32x2_t permlane32_swap(unsigned a, unsigned b, bool fi = false, bool bound_ctrl = false);
template <typename T> inline T readfirstlane_any(T v) { return (T)readfirstlane((unsigned)v); }
inline float fdot2(f16x2_t a, f16x2_t b, float c, bool /*clamp*/) { return c + (float)a[0] * (float)b[0] + (float)a[1] * (float)b[1]; }
inline float fdot2(bf16x2_t a, bf16x2_t b, float c, bool /*clamp*/) { return c + (float)a[0] * (float)b[0] + (float)a[1] * (float)b[1]; }
int ds_bpermute(int byte_index, int v);
unsigned shfl_xor_u32(unsigned v, int mask, int width);

template <typename T> inline T shfl_xor(T v, int mask, int width = 64) {
  static_assert(sizeof(T) == 4, "32-bit values only");
  unsigned u;
  std::memcpy(&u, &v, 4);
  u = shfl_xor_u32(u, mask, width);
  std::memcpy(&v, &u, 4);
  return v;
}

// ---- HIP's short vector structs ---------------------------------------------------------------
struct alignas(8) uint2 { unsigned x, y; };
struct alignas(16) uint4 { unsigned x, y, z, w; };
struct alignas(8) float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
struct alignas(8) int2 { int x, y; };
struct alignas(16) int4 { int x, y, z, w; };

// ---- device math helpers ------------------------------------------------------------------------
inline float __uint_as_float(unsigned u) { float f; std::memcpy(&f, &u, 4); return f; }
inline unsigned __float_as_uint(float f) { unsigned u; std::memcpy(&u, &f, 4); return u; }
// single roundings, never contracted (the host build is compiled with -ffp-contract=off)
inline float __fmul_rn(float a, float b) { return a * b; }
inline float __fadd_rn(float a, float b) { return a + b; }
inline float __fmaf_rn(float a, float b, float c) { return std::fma(a, b, c); }

// ---- hip_fp16.h: the half type as the kernels use it ---------------------------------------------
struct __half {
  _Float16 v;
  __half() = default;
  __half(_Float16 x) : v(x) {}
  operator _Float16() const { return v; }
};
struct alignas(4) __half2 { __half x, y; };
inline float __half2float(__half h) { return (float)h.v; }
inline __half __float2half_rn(float f) { return __half((_Float16)f); }
inline __half __float2half(float f) { return __half((_Float16)f); }
inline float2 __half22float2(__half2 h) { return float2{(float)h.x.v, (float)h.y.v}; }

// ---- the HIP runtime calls the launchers make --------------------------------------------------
typedef int hipError_t;
typedef void *hipStream_t;
typedef void *hipEvent_t;
constexpr hipError_t hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2, hipErrorInvalidDevice = 101,
                     hipErrorInvalidSymbol = 13, hipErrorLaunchFailure = 719;
enum hipMemcpyKind { hipMemcpyHostToHost, hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice, hipMemcpyDefault };
inline hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind, hipStream_t) { std::memmove(dst, src, bytes); return hipSuccess; }
inline hipError_t hipMemsetAsync(void *dst, int value, size_t bytes, hipStream_t) { std::memset(dst, value, bytes); return hipSuccess; }
inline hipError_t hipGetDevice(int *dev) { *dev = 0; return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void **p, const void *symbol) { *p = const_cast<void *>(symbol); return hipSuccess; }
extern hipError_t g_last_error;
inline hipError_t hipGetLastError() { const hipError_t e = g_last_error; g_last_error = hipSuccess; return e; }
inline const char *hipGetErrorString(hipError_t e) {
  return e == hipSuccess ? "no error" : e == hipErrorInvalidValue ? "invalid argument" : e == hipErrorLaunchFailure ? "launch failure (host emulation: see fa_emu_last_error)" : "error";
}
hipError_t hipMallocAsync(void **p, size_t bytes, hipStream_t);
hipError_t hipFreeAsync(void *p, hipStream_t);

}  // namespace fa_emu

// ---- names the sources use ------------------------------------------------------------------
using fa_emu::dim3;
using fa_emu::uint2;
using fa_emu::uint4;
using fa_emu::float2;
using fa_emu::float4;
using fa_emu::int2;
using fa_emu::int4;
using fa_emu::hipError_t;
using fa_emu::hipStream_t;
using fa_emu::hipSuccess;
using fa_emu::hipErrorInvalidValue;
using fa_emu::hipGetLastError;
using fa_emu::hipEvent_t;
using fa_emu::hipErrorInvalidDevice;
using fa_emu::hipErrorInvalidSymbol;
using fa_emu::hipGetDevice;
using fa_emu::hipMemcpyKind;
using fa_emu::hipMemcpyDeviceToDevice;
using fa_emu::hipMemcpyAsync;
using fa_emu::hipMemsetAsync;
using fa_emu::__uint_as_float;
using fa_emu::__float_as_uint;
using fa_emu::__fmul_rn;
using fa_emu::__fadd_rn;
using fa_emu::__fmaf_rn;
using fa_emu::hipEventRecord;
using fa_emu::hipGetSymbolAddress;
using fa_emu::__half;
using fa_emu::__half2;
using fa_emu::__half2float;
using fa_emu::__float2half_rn;
using fa_emu::__float2half;
using fa_emu::__half22float2;
using fa_emu::hipGetErrorString;
using fa_emu::hipMallocAsync;
using fa_emu::hipFreeAsync;
using std::max;
using std::min;

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static
#define threadIdx (::fa_emu::g_thread_idx)
#define blockIdx (::fa_emu::g_block_idx)
#define blockDim (::fa_emu::g_block_dim)
#define gridDim (::fa_emu::g_grid_dim)
#define __syncthreads() ::fa_emu::block_barrier()
#define __shfl_xor(...) ::fa_emu::shfl_xor(__VA_ARGS__)

#define __amdgpu_buffer_rsrc_t ::fa_emu::BufferRsrc
// (variadic so that braces with commas in an argument pass through)
#define __builtin_amdgcn_make_buffer_rsrc(...) ::fa_emu::make_buffer_rsrc(__VA_ARGS__)
#define __builtin_amdgcn_raw_buffer_load_b128(...) ::fa_emu::raw_buffer_load_b128(__VA_ARGS__)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(...) ::fa_emu::mfma_32x32x16_f16(__VA_ARGS__)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(...) ::fa_emu::mfma_32x32x16_bf16(__VA_ARGS__)
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(...) ::fa_emu::ds_read_tr16_b64((const void *)(__VA_ARGS__))
#define __builtin_amdgcn_ballot_w64(...) ::fa_emu::ballot_w64(__VA_ARGS__)
#define __builtin_amdgcn_readfirstlane(...) ::fa_emu::readfirstlane_any(__VA_ARGS__)
#define __builtin_amdgcn_permlane32_swap(...) ::fa_emu::permlane32_swap(__VA_ARGS__)
#define __builtin_amdgcn_ds_bpermute(...) ::fa_emu::ds_bpermute(__VA_ARGS__)
#define __builtin_amdgcn_exp2f(...) ::exp2f(__VA_ARGS__)
#define __builtin_amdgcn_logf(...) ::log2f(__VA_ARGS__)
#define __builtin_amdgcn_fdot2(...) ::fa_emu::fdot2(__VA_ARGS__)
#define __builtin_amdgcn_fdot2_f32_bf16(...) ::fa_emu::fdot2(__VA_ARGS__)

#define HIP_SYMBOL(x) (&(x))
#define __align__(n) __attribute__((aligned(n)))
#define BRT_ROCM_LAUNCH(kernel, grid, block, stream, ...) FA_LAUNCH(kernel, grid, block, stream, __VA_ARGS__)
#define FA_LAUNCH(kernel, grid, block, stream, ...) \
  ((void)(stream), ::fa_emu::g_last_error = ::fa_emu::launch((grid), (block), [&]() { kernel(__VA_ARGS__); }) ? ::fa_emu::hipErrorLaunchFailure : ::fa_emu::g_last_error)
#define FA_WAVE_SYNC() ::fa_emu::wave_sync()
#define FA_PIN(x) ((void)(x))
#define FA_PIN2(x, y) ((void)(x), (void)(y))
