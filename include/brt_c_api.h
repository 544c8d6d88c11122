/*
 * brt_c_api.h -- C ABI of libbrt.so, the host runtime (session / request context) of the ROCm
 * provider.  It is what a foreign-language binding links against; the reference binds the same
 * operations to Python with pybind11 (runtime/python/src/module.cc:252-423: brt.Session,
 * brt.RequestContext), and each function cites the method it stands for.
 *
 * All functions returning int return 0 on success and non-zero on failure; the failure text is
 * available from brt_last_error() (thread-local).  Handles are opaque.
 */
#ifndef BRT_C_API_H_
#define BRT_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct brt_session brt_session;
typedef struct brt_request brt_request;
typedef void *(*brt_alloc_fn)(size_t bytes);
typedef void (*brt_free_fn)(void *ptr);

const char *brt_last_error(void);

/* brt.Session(device="CUDA", alloc_func, free_func) (module.cc:340-372): creates a session with
 * the ROCm execution provider and allocators for the memory spaces "cuda"/"rocm" (device) and
 * "cpu".  alloc/free may be NULL (hipMalloc/hipFree) or a caller's caching allocator.
 * device_id < 0 creates a plan-only session for hosts without a GPU: modules load, kernels are
 * constructed (shape checks, dlopen of custom libraries), arguments can be bound, but
 * brt_session_run fails -- there is no host execution path. */
brt_session *brt_session_create(int device_id, brt_alloc_fn alloc, brt_free_fn free_fn);
void brt_session_destroy(brt_session *s);
/* Session.load(path) (module.cc:373-377) / Session::LoadFromMemory: ByRE text. */
int brt_session_load(brt_session *s, const char *path);
int brt_session_load_text(brt_session *s, const char *text);
/* ExecutionProvider::StaticRegisterKernelsFromDynlib (execution_provider.cc:29-41): load a
 * library of extra op kernels; call before brt_session_create. */
int brt_register_kernels_from_dynlib(const char *path);
/* 1 when the session's provider has a kernel registered under `key` */
int brt_session_has_kernel(brt_session *s, const char *key);

/* graph introspection: Session::GetArgNum, GetGraphArgOffset, GetInput/Output/WeightArgOffsets,
 * GetStaticShape, GetDType, GetSpace (session.h:80-131) */
size_t brt_session_arg_num(brt_session *s);
int brt_session_arg_offset(brt_session *s, const char *name);       /* -1 if absent */
const char *brt_session_arg_name(brt_session *s, size_t offset);
int brt_session_arg_kind(brt_session *s, size_t offset);            /* byre.argtype bits: 1 in, 2 out, 4 weight */
size_t brt_session_arg_rank(brt_session *s, size_t offset);
void brt_session_arg_shape(brt_session *s, size_t offset, int64_t *shape_out);
const char *brt_session_arg_dtype(brt_session *s, size_t offset);   /* "f32", "f16", "bf16", "i64", ... */
const char *brt_session_arg_space(brt_session *s, size_t offset);
/* bytes of the per-frame arena that holds all memref.alloc intermediates of memory space
 * `space`, laid out by the static memory plan (bump allocation in order of first use, every
 * tensor rounded up to 256 bytes; execution_plan.cc:473-578) */
size_t brt_session_intermediate_bytes(brt_session *s, const char *space);
size_t brt_session_op_num(brt_session *s);
const char *brt_session_op_key(brt_session *s, size_t op_index);
/* OpAccessor::GetAttrAsVoidPtr (op_accessor.cc:212-242) for op `op_index`: copies the packed
 * blob of array attribute `name` (i64 -> 8 bytes, f32 -> 4 bytes, no padding) into out[0..cap)
 * and returns its full size, or -1 when the attribute is missing or not an array. */
long brt_session_op_attr_blob(brt_session *s, size_t op_index, const char *name, void *out, size_t cap);

/* Session.new_request_context(stream) (module.cc:378-406): `stream` is a caller-owned
 * hipStream_t used as the compute stream, or NULL for a stream owned by the request. */
brt_request *brt_request_create(brt_session *s, void *stream, int use_external_stream);
void brt_request_destroy(brt_request *r);
/* RequestContext.bind_arg / get_arg / finish_io_binding / sync (module.cc:252-303) */
int brt_request_bind_arg(brt_request *r, size_t offset, void *device_ptr);
void *brt_request_get_arg(brt_request *r, size_t offset);
int brt_request_finish_io_binding(brt_request *r);
int brt_request_sync(brt_request *r);
/* Session.run(request): enqueues every op kernel on the request's stream; does not wait */
int brt_session_run(brt_session *s, brt_request *r);
/* per-op listener (Before/AfterOpKernelRun events, framework/event.h:27-74):
 * cb(user, op_key, op_index, after) */
typedef void (*brt_op_listener)(void *user, const char *op_key, int op_index, int after);
void brt_request_add_op_listener(brt_request *r, brt_op_listener cb, void *user);

#ifdef __cplusplus
}
#endif
#endif /* BRT_C_API_H_ */
