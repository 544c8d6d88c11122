/*
 * brt_rocm_kernels.h -- C ABI of libbrt_rocm_kernels.so, the device layer of the ROCm
 * execution provider: plain pointers and sizes, no C++ or framework types.
 *
 * Host code (the provider's op kernels, written in C++, or any FFI) reaches HIP only
 * through these entry points.  Every function returns a hipError_t value as int
 * (0 == success) unless stated otherwise; kernels are enqueued on `stream`
 * (a hipStream_t passed as void*, NULL = the default stream) and never synchronise.
 *
 * Citations name the interface of the reference (bytedance/byteir, paths relative to its
 * checkout) that each entry point stands in for.
 */
#ifndef BRT_ROCM_KERNELS_H_
#define BRT_ROCM_KERNELS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types (the subset of brt::DTypeEnum, runtime/include/brt/core/framework/dtype.h,
 * that the op kernels on this path accept) */
enum { BRT_ROCM_F32 = 0, BRT_ROCM_F16 = 1, BRT_ROCM_BF16 = 2 };
/* fold operators of
 * runtime/lib/backends/cuda/providers/default/reduction/kernels/reduction_helper.h:
 * SumOp :18-36, MaxOp :140-179 (the two the reference registers op kernels for) and MinOp
 * :98-137, ProdOp :80-95, MeanOp :37-56 (sum, then divided by float(B) at the store), SumSqrOp
 * :58-77 (elements squared in float as they are read), which the reference defines but never
 * instantiates.  Max and Min let a NaN on either side win. */
enum {
  BRT_ROCM_REDUCE_SUM = 0,
  BRT_ROCM_REDUCE_MAX = 1,
  BRT_ROCM_REDUCE_MIN = 2,
  BRT_ROCM_REDUCE_PROD = 3,
  BRT_ROCM_REDUCE_MEAN = 4,
  BRT_ROCM_REDUCE_SUMSQR = 5
};

/* library identification; returns a static string */
const char *brt_rocm_version(void);
/* hipGetErrorString for the int codes returned below */
const char *brt_rocm_error_string(int err);

/* ---- device plumbing ------------------------------------------------------------- */
/* Stand-ins for the CUDA runtime calls made by the reference's device layer:
 * allocator  runtime/lib/backends/cuda/device/cuda_allocator.cc:36-86 (cudaMalloc/cudaFree,
 *            cudaMallocHost/cudaFreeHost),
 * work queue runtime/lib/backends/cuda/device/cuda_work_queue.cc:139-177 (stream create /
 *            destroy / synchronize),
 * device API runtime/lib/backends/cuda/device/cuda_device_api.cc:29-55 (memcpy H2D/D2H/D2D,
 *            memset, set device). */
int brt_rocm_device_count(int *count);
int brt_rocm_set_device(int device_id);
int brt_rocm_malloc(void **ptr, size_t bytes);
int brt_rocm_free(void *ptr);
int brt_rocm_host_malloc(void **ptr, size_t bytes); /* pinned host memory */
int brt_rocm_host_free(void *ptr);
/* copies are asynchronous on `stream`; with pageable host memory HIP stages them */
int brt_rocm_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream);
int brt_rocm_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream);
int brt_rocm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
int brt_rocm_memset(void *dst, int value, size_t bytes, void *stream); /* a fill kernel, safe to capture in a HIP graph */
/* Launches a device function by its host-side handle (what `&kernel<...>` yields in a HIP
 * translation unit): grid and block are three extents each, kernel_args one pointer per kernel
 * parameter.  What WorkQueue::AddTask(kCompute, ...) enqueues; stands in for the cudaLaunchKernel
 * of CUDAWorkQueue's Compute (runtime/lib/backends/cuda/device/cuda_work_queue.cc:59-67). */
int brt_rocm_launch_kernel(const void *func, const unsigned grid[3], const unsigned block[3],
                           void **kernel_args, size_t shared_bytes, void *stream);
/* Enqueues fn(arg) on the host in stream order (cudaLaunchHostFunc in ComputeHost,
 * cuda_work_queue.cc:98-102); fn must not call into the HIP runtime. */
int brt_rocm_launch_host_func(void *stream, void (*fn)(void *), void *arg);
int brt_rocm_stream_create(void **stream);
int brt_rocm_stream_destroy(void *stream);
int brt_rocm_stream_synchronize(void *stream);
int brt_rocm_device_synchronize(void);
/* Measurement and test tooling that the same library exports (the benchmark's data generator,
 * event timing, a copy kernel of known traffic, a reduce call with a timing hook) is declared in
 * brt_rocm_bench.h: none of it stands in for a reference interface. */

/* ---- reductions ------------------------------------------------------------------ */
/* out[a, c] = fold_b in[a, b, c] for a dense row-major tensor viewed as [A, B, C];
 * f16 is folded in float.  Stands in for
 *   kernel::call_reduce<T, Op>(input, output, A, B, C, workspace, stream)
 * (runtime/lib/backends/cuda/providers/default/reduction/kernels/reduction.h:13-15,
 *  reduction.cu:415-426), and
 *   kernel::get_reduce_workspace_in_bytes<T>(A, B, C)          (reduction.h:17-18,
 *  reduction.cu:428-434).
 * A == 0 and B == 0 means "nothing to fold": C elements are copied device to device, as
 * ReduceImpl::Execute does for the (0, 0, numel) it sets up when every reduced dimension has
 * extent 1 (reduce_impl.h:55-58,61-75).  Tensors without elements: A == 0 or C == 0 writes
 * nothing; B == 0 with A, C > 0 (an empty fold axis, which the reference also sends to its copy
 * branch, reading C elements of an input that has none) writes the operator's identity to all
 * A * C outputs (0, -inf, +inf, 1, NaN for the mean, 0).
 * The workspace holds float partials of the split first pass; its size depends only on
 * (dtype, A, B, C), so it can be queried once when an execution plan is built.  A NULL or
 * too small workspace is an error (hipErrorInvalidValue) when the size is non-zero.
 * dtype: BRT_ROCM_F32 or BRT_ROCM_F16.  Max propagates NaN from either operand. */
size_t brt_rocm_reduce_workspace_bytes(int dtype, size_t A, size_t B, size_t C);
int brt_rocm_reduce(int op, int dtype, const void *input, void *output, size_t A, size_t B,
                    size_t C, void *workspace, size_t workspace_bytes, void *stream);
/* The same fold for callers that must not allocate and have no workspace to hand over (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference, whose ReduceImpl always takes its workspace from the frame's
 * allocator (reduce_impl.h:76-79).  The partials of the split first pass go to a device array
 * of BRT_ROCM_REDUCE_STATIC_SCRATCH_BYTES that is part of the library's code object (every GPU
 * the library runs on holds one for the life of the process); the call makes no hipMalloc,
 * hipFree or other allocating call.  A fold whose brt_rocm_reduce_workspace_bytes exceeds that
 * size is refused with BRT_ROCM_ERROR_STATIC_SCRATCH_TOO_SMALL (brt_rocm_error_string names the
 * limit) before anything is enqueued.  All calls on one GPU share the array: calls that can run
 * at the same time on one GPU (different streams, different threads) race on it and must be
 * ordered by the caller.  Nothing in the array needs clearing between calls.  The first call on
 * a device looks the array's address up (hipGetSymbolAddress); make it outside graph capture. */
#define BRT_ROCM_REDUCE_STATIC_SCRATCH_BYTES (8u << 20)
#define BRT_ROCM_ERROR_STATIC_SCRATCH_TOO_SMALL 20001
int brt_rocm_reduce_static(int op, int dtype, const void *input, void *output, size_t A, size_t B,
                           size_t C, void *stream);

/* ---- fused row softmax ----------------------------------------------------------- */
/* y[r, :] = exp(x[r, :] - max_j x[r, j]) / sum_j exp(...) over the last axis of a dense
 * [rows, cols] tensor; float internals for every storage type, one rounding at the store.
 * The reference runtime has no softmax kernel; the arithmetic contract is the compiler's
 * linalg_ext.softmax lowering (compiler/lib/Conversion/ToLinalg/LinalgExtToLinalg.cpp:286-410).
 * dtype: BRT_ROCM_F32, BRT_ROCM_F16 or BRT_ROCM_BF16.  In-place (output == input) is allowed.
 * Rows of any length and alignment; rows that do not start on 16 bytes are processed through
 * the 16-byte granules that cover them (bytes of the neighbouring rows in the first and last
 * granule are read and never written). */
int brt_rocm_softmax(int dtype, const void *input, void *output, size_t rows, size_t cols,
                     void *stream);

/* The same over the middle axis of a dense row-major [A, B, C] tensor (byteir.softmax with an
 * `axis` that is not the last one, compiler/lib/Conversion/ToLinalg/HloToLinalg.cpp:393-467:
 * A = product of the dimensions before the axis, C = product of those after).  C == 1 is the
 * row softmax above.  With few columns and a long axis the call takes a stream-ordered scratch
 * allocation (hipMallocAsync / hipFreeAsync on `stream`, 8 * A * segments * C bytes) and falls
 * back to one workgroup per column tile if that fails. */
int brt_rocm_softmax_axis(int dtype, const void *input, void *output, size_t A, size_t B, size_t C,
                          void *stream);
/* The same with the scratch supplied by the caller (the op kernel's per-frame workspace, asked
 * and allocated where the reference's kernels ask for theirs, op_kernel_impl_base.h:116-149):
 * brt_rocm_softmax_workspace_bytes is what the call takes for 16-byte aligned tensors (0: none);
 * a NULL, misaligned or too small workspace falls back to the stream-ordered allocation. */
size_t brt_rocm_softmax_workspace_bytes(int dtype, size_t A, size_t B, size_t C);
int brt_rocm_softmax_axis_ws(int dtype, const void *input, void *output, size_t A, size_t B, size_t C,
                             void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BRT_ROCM_KERNELS_H_ */
