/* Measurement and test tooling exported by libbrt_rocm_kernels.so next to the op-kernel C ABI of
 * brt_rocm_kernels.h.  Nothing here stands in for an interface of the reference runtime: the
 * benchmark and the tests use these to generate synthetic inputs on the device, to time launches
 * with events on the stream they run on, and to scale hardware byte counters against a launch
 * of known traffic.  A host that only runs ByRE modules never calls them. */
#ifndef BRT_ROCM_BENCH_H_
#define BRT_ROCM_BENCH_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* device-to-device copy done by a plain compute kernel (128-bit loads and stores) rather than
 * a DMA engine: for buffers that are multiples of 16 bytes and 16-byte aligned: the launch of known
 * traffic against which hardware byte counters (FETCH_SIZE, WRITE_SIZE) are scaled, and the
 * copy ceiling the softmax figures are compared with. */
int brt_rocm_copy_kernel(void *dst, const void *src, size_t bytes, void *stream);

/* The rate of v_mfma_f32_32x32x16_{f16,bf16} on operands of the caller's choosing, with nothing
 * else in the loop: `blocks` workgroups of eight waves each read 256 bytes of operands per lane
 * (operand_bytes >= blocks * 512 * 256) once, then issue iters * 16 matrix instructions per wave
 * on them; sink (blocks * 512 floats) receives the sums so that the work is not dead.  One launch
 * does blocks * 8 * iters * 16 * 32768 flops.  The clock that the chip holds under this load
 * depends on the operand bits, so the rate on zeros and the rate on normally distributed values
 * differ: the second is the ceiling for a kernel that is fed such data. */
int brt_rocm_mfma_rate_probe(int dtype, const void *operands, size_t operand_bytes, float *sink,
                             size_t sink_bytes, int blocks, int iters, void *stream);

/* events, for timing a launch on the stream it runs on */
int brt_rocm_event_create(void **event);
int brt_rocm_event_destroy(void *event);
int brt_rocm_event_record(void *event, void *stream);
int brt_rocm_event_synchronize(void *event);
int brt_rocm_event_elapsed_ms(float *ms, void *start, void *stop);


/* ---- synthetic data -------------------------------------------------------------- */
/* Fills `n` elements with a counter-based pseudo-random sequence: element i depends on
 * (seed, i) only -- splitmix64 output number i (uniform) or 3i .. 3i + 2 (normal) -- through
 * integer arithmetic and exact float operations, so a host restatement of the same lines gives
 * the same bits (the benchmark's and the tests' CPU side generates its own copy instead of
 * reading the buffer back).  BRT_ROCM_FILL_UNIFORM: x = fma(u, b - a, a), u = 24 random bits
 * * 2^-24 in [0, 1).  BRT_ROCM_FILL_NORMAL: x = b * (sum of twelve 16-bit fields - 393210) *
 * 2^-16, mean 0 and standard deviation b (twelve-term central limit, support +-6 b); a unused.
 * Stored as f32 / f16 / bf16 with round-to-nearest-even.  The reference has no counterpart: its
 * tests fill buffers on the host (runtime/test/include/brt/test/common/util.h). */
enum { BRT_ROCM_FILL_UNIFORM = 0, BRT_ROCM_FILL_NORMAL = 1 };
int brt_rocm_fill(int dtype, int dist, uint64_t seed, void *ptr, size_t n, float a, float b, void *stream);

/* brt_rocm_reduce (brt_rocm_kernels.h) with a timing hook: `first_pass_done`, when not NULL, is a hipEvent_t that is
 * recorded on `stream` right after the first (or only) pass has been enqueued, so that a caller
 * can time the split first pass apart from the combine pass.  No counterpart in the reference
 * (its hooks are host-side Before/AfterOpKernelRun events, framework/event.h:27-74). */
int brt_rocm_reduce_ex(int op, int dtype, const void *input, void *output, size_t A, size_t B,
                       size_t C, void *workspace, size_t workspace_bytes, void *stream,
                       void *first_pass_done);

/* Writes the first-pass kernel that brt_rocm_reduce plans for (dtype, A, B, C) on 16-byte aligned
 * tensors, spelled as a profiler prints the instantiation with the operator as "OP", followed by
 * the split (" S=128 col_tiles=2"), into buf.  A stored counter profile is valid for today's
 * library only if it names this kernel. */
int brt_rocm_reduce_plan_describe(int dtype, size_t A, size_t B, size_t C, char *buf, size_t len);

#ifdef __cplusplus
}
#endif
#endif /* BRT_ROCM_BENCH_H_ */
