/*
 * flash_api.h -- C ABI of libflash_attn.so, the MI355X drop-in for the flash-attention
 * custom library that ByRE's `custom` op kernel dlopen()s.
 *
 * The caller is CustomOpKernel::RunImpl (reference:
 * runtime/lib/backends/cuda/providers/default/custom/custom.cc:69-86):
 *     run_func_(tensor_args, extra_args, stream);
 * where tensor_args[i] is the device pointer of operand i, extra_args is a malloc'ed,
 * unpadded blob built from the op's `extra_args` array attribute (i64 -> 8 bytes,
 * f32 -> 4 bytes; runtime/lib/core/framework/op_accessor.cc:212-242) and stream is the work
 * queue's compute stream.  The custom op also requires a data symbol named VERSION
 * (custom.cc:50-53).
 *
 * These declarations replace external_libs/runtime/flash_attn/include/flash_api.h:75-82 of
 * the reference.  Streams are hipStream_t passed as void*.
 *
 * extra_args layout (192 bytes; compiler/lib/Conversion/HloToByreTensor/HloToByreCustom.cpp:149-176,
 * parsed at external_libs/runtime/flash_attn/lib/flash_api.cu:586-624):
 *   i64 q,k,v,o batch_stride; i64 q,k,v,o row_stride; i64 q,k,v,o head_stride  (elements)
 *   i64 b, h, h_k, d, d_rounded; f32 softmax_scale;
 *   i64 seqlen_q, seqlen_k, seqlen_q_rounded, seqlen_k_rounded; f32 p_dropout;
 *   i64 window_size_left, window_size_right      (causal = (-1, 0), full = (-1, -1))
 * Tensors are [batch, seqlen, heads, head_dim] with a contiguous head_dim; softmax_lse is
 * [batch, heads, seqlen_q] float.
 *
 * Supported here: head_dim a multiple of 8 up to 256 (the reference's range; 32, 64 and 128
 * have tuned kernels), 0 <= p_dropout < 1, any seqlen including 0 (tensors of a side without rows
 * may be NULL), h % h_k == 0
 * (backward with h_k < h: dK, dV of a key/value head are the sums over its query heads -- the
 * gradient; the reference's own addressing of dK / dV is only right for h == h_k).  Anything else is reported on stderr and the process aborts, since
 * the ABI has no error channel; the *_checked variants return an error code instead.
 * Calls with few query rows or few query blocks against many keys split the key axis over
 * workgroups and keep their partial results in a stream-ordered allocation
 * (hipMallocAsync / hipFreeAsync on `stream`); the backward call does so for partial dK / dV on
 * small grids when dq_accum cannot hold them; no other call allocates.
 */
#ifndef BYTEIR_AMD_FLASH_API_H_
#define BYTEIR_AMD_FLASH_API_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Must be a pointer variable, as in the reference (flash_api.cu:7-9). */
extern const char *VERSION;

/* tensors: {q, k, v, rng_state, o, softmax_lse, softmax_P}  (flash_api.cu:626-654).
 * fp16 storage.  rng_state is two 64-bit words {seed, offset} in device memory, read by the
 * kernel when p_dropout > 0 as in the reference (flash_fwd_kernel.h:46-47; the caller fills
 * it) and not touched otherwise; the keep-mask is the reference's function of (seed, offset,
 * batch, head, row, column) (lib/dropout.h, lib/philox.cuh).  softmax_P is never touched. */
void run_flash_attn_fwd(void **tensors, void *extra_args, void *stream);

/* tensors: {dout, q, k, v, out, softmax_lse, rng_state, dq, dk, dv, d_softmax, dq_accum}
 * (flash_api.cu:696-725).  fp16 storage.  d_softmax is [b, h, seqlen_q_rounded] float scratch
 * that receives rowsum(dout * out) (times 1 - p_dropout, as in the reference); rng_state must
 * hold what the forward call used; dq_accum ([b, seqlen_q_rounded, h, d_rounded] float, may be
 * NULL) is scratch: dQ is accumulated without atomics by a pass that is parallel over query
 * blocks, and with grouped heads and few key blocks the buffer holds partial dK / dV of the
 * group's query heads (a stream-ordered allocation supplies what it cannot hold). */
void run_flash_attn_bwd(void **tensors, void *extra_args, void *stream);

/* The same two entry points for bfloat16 storage.  The reference library is fp16 only
 * (params.is_bf16 = 0, flash_api.cu:295,421) and its blob carries no dtype field, so the
 * element type is selected by the op's `api_name` attribute. */
void run_flash_attn_fwd_bf16(void **tensors, void *extra_args, void *stream);
void run_flash_attn_bwd_bf16(void **tensors, void *extra_args, void *stream);

/* Decoding against a key/value cache: run_flash_attn_kvcache of the reference
 * (flash_api.cu:727-811 -> run_mha_fwd_with_kvcache :434-567).
 * tensors: {q, k_cache, v_cache, k_new, v_new, seqlens_k, o, softmax_lse}.
 *   q [b, seqlen_q, h, d]; k_cache, v_cache [b, seqlen_k, h_k, d] (seqlen_k = capacity);
 *   k_new, v_new [b, seqlen_knew, h_k, d]; seqlens_k int32 [b] = rows already valid per batch.
 * First k_new / v_new are written into the caches at rows seqlens_k[b] .. +seqlen_knew (in
 * place), then q attends to rows [0, seqlens_k[b] + seqlen_knew) of its batch, with the window
 * aligned to the end of that range (block_info.h:27-37, mask.h:160-200).  No rotary embedding
 * (the reference sets rotary_dim = 0; it also fixes one split, whereas here the key axis is
 * split over workgroups when that fills the chip).  k_new / v_new may both be NULL (no append);
 * seqlens_k may be NULL only then (all seqlen_k rows are attended).
 * extra_args (244 bytes): i64 q,k,v,knew,vnew,o batch_stride; the same six row_strides; the
 * same six head_strides; i64 b, h, h_k, d, d_rounded, seqlen_knew; f32 softmax_scale;
 * i64 seqlen_q, seqlen_k, seqlen_q_rounded, seqlen_k_rounded; i64 window_size_left, _right. */
void run_flash_attn_kvcache(void **tensors, void *extra_args, void *stream);
void run_flash_attn_kvcache_bf16(void **tensors, void *extra_args, void *stream);

/* Error-returning forms of the calls above: 0 on success, a positive hipError_t when a
 * launch failed, -1 when the arguments are unsupported (reason copied to a thread-local
 * buffer readable through flash_attn_last_error()).  dtype: 1 = fp16, 2 = bf16. */
int flash_attn_fwd_checked(void **tensors, const void *extra_args, int dtype, void *stream);
int flash_attn_bwd_checked(void **tensors, const void *extra_args, int dtype, void *stream);
int flash_attn_kvcache_checked(void **tensors, const void *extra_args, int dtype, void *stream);
const char *flash_attn_last_error(void);

/* The same calls with their scratch supplied by the caller, for hosts that own all device
 * memory (the runtime's per-frame workspace: the op kernel asks the size when a frame is set
 * up and allocates through the frame's allocator, as the reference's kernels do for their
 * workspaces, framework/op_kernel_impl_base.h:116-149; the reference library itself has no
 * scratch because it never splits).  *_workspace_bytes returns what the call with this blob
 * would take -- partial results of a key axis split over workgroups (forward, cache decode),
 * partial dK / dV beyond what a dq_accum tensor of `dq_accum_bytes` holds (backward) -- and 0
 * when it takes none or the blob is not supported; the size depends on the blob only.  The
 * *_ws calls use `workspace` when it is 16-byte aligned and at least that large, and fall back
 * to a stream-ordered allocation of their own otherwise (as the plain calls always do). */
size_t flash_attn_fwd_workspace_bytes(const void *extra_args, int dtype);
size_t flash_attn_bwd_workspace_bytes(const void *extra_args, int dtype, size_t dq_accum_bytes);
size_t flash_attn_kvcache_workspace_bytes(const void *extra_args, int dtype);
int flash_attn_fwd_ws(void **tensors, const void *extra_args, int dtype, void *workspace, size_t workspace_bytes, void *stream);
int flash_attn_bwd_ws(void **tensors, const void *extra_args, int dtype, void *workspace, size_t workspace_bytes, void *stream);
int flash_attn_kvcache_ws(void **tensors, const void *extra_args, int dtype, void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BYTEIR_AMD_FLASH_API_H_ */
