// C ABI over the C++ runtime (include/brt_c_api.h); exceptions stop here.
#include <cstdlib>
#include <cstring>

#include "brt.h"
#include "brt_c_api.h"

using namespace brt;

struct brt_session {
  Session session;
  std::string scratch;
  bool plan_only = false;  // built without a device: modules load and plan, nothing runs
};
struct brt_request {
  brt_session *owner;
  std::unique_ptr<RequestContext> ctx;
};

namespace {
thread_local std::string g_error;
int Fail(const std::string &m) { g_error = m; return 1; }
int FromStatus(const common::Status &s) { return s.IsOK() ? 0 : Fail(s.ErrorMessage()); }
template <typename F> int Guard(F f) {
  try {
    return f();
  } catch (const std::exception &e) {
    return Fail(e.what());
  }
}
}  // namespace

extern "C" {

const char *brt_last_error(void) { return g_error.c_str(); }

brt_session *brt_session_create(int device_id, brt_alloc_fn alloc, brt_free_fn free_fn) {
  try {
    std::unique_ptr<brt_session> s(new brt_session);
    if (device_id < 0) {  // plan-only: host memory stands in for every space, Run is refused
      s->plan_only = true;
      for (const char *k : {"cuda", "rocm", "cpu", "cudaPinned"}) s->session.AddAllocator(MakeHostAllocator(k));
      s->session.SetWorkQueueFactory([]() { return MakeRocmExternalStreamWorkQueue(nullptr); });
      s->session.AddExecutionProvider(std::unique_ptr<ExecutionProvider>(new ExecutionProvider(DeviceKind::ROCM, ProviderType::BRT)));
      return s.release();
    }
    common::Status st = ROCMAllocatorFactory(&s->session, device_id);
    if (!st.IsOK()) { g_error = st.ErrorMessage(); return nullptr; }
    if (alloc && free_fn) {
      s->session.AddAllocator(MakeExternalAllocator("cuda", alloc, free_fn));
      s->session.AddAllocator(MakeExternalAllocator("rocm", alloc, free_fn));
    }
    st = DefaultROCMExecutionProviderFactory(&s->session, device_id);
    if (!st.IsOK()) { g_error = st.ErrorMessage(); return nullptr; }
    return s.release();
  } catch (const std::exception &e) {
    g_error = e.what();
    return nullptr;
  }
}
void brt_session_destroy(brt_session *s) { delete s; }

int brt_session_load(brt_session *s, const char *path) {
  return Guard([&] { return FromStatus(s->session.Load(path, "byre")); });
}
int brt_session_load_text(brt_session *s, const char *text) {
  return Guard([&] { return FromStatus(s->session.LoadFromMemory(text, "byre")); });
}
int brt_register_kernels_from_dynlib(const char *path) {
  return Guard([&] { return FromStatus(ExecutionProvider::StaticRegisterKernelsFromDynlib(path)); });
}
int brt_session_has_kernel(brt_session *, const char *key) {
  ExecutionProvider probe(DeviceKind::ROCM, ProviderType::BRT);
  return probe.GetKernelRegistry()->HasKernel(key) ? 1 : 0;
}

size_t brt_session_arg_num(brt_session *s) { return s->session.GetArgNum(); }
size_t brt_session_intermediate_bytes(brt_session *s, const char *space) {
  return s->session.GetIntermediateBytes(space ? space : "");
}
int brt_session_arg_offset(brt_session *s, const char *name) { return s->session.GetGraphArgOffset(name); }
const char *brt_session_arg_name(brt_session *s, size_t offset) {
  try { s->scratch = s->session.GetArgName(offset); } catch (...) { s->scratch.clear(); }
  return s->scratch.c_str();
}
int brt_session_arg_kind(brt_session *s, size_t offset) {
  int k = 0;
  for (size_t o : s->session.GetInputArgOffsets()) if (o == offset) k |= 1;
  for (size_t o : s->session.GetOutputArgOffsets()) if (o == offset) k |= 2;
  for (size_t o : s->session.GetWeightArgOffsets()) if (o == offset) k |= 4;
  return k;
}
size_t brt_session_arg_rank(brt_session *s, size_t offset) {
  try { return s->session.GetStaticShape(offset).size(); } catch (...) { return 0; }
}
void brt_session_arg_shape(brt_session *s, size_t offset, int64_t *out) {
  try {
    const Shape sh = s->session.GetStaticShape(offset);
    for (size_t i = 0; i < sh.size(); ++i) out[i] = sh[i];
  } catch (...) {}
}
const char *brt_session_arg_dtype(brt_session *s, size_t offset) {
  try { return GetDTypeName(s->session.GetDType(offset)); } catch (...) { return "invalid"; }
}
const char *brt_session_arg_space(brt_session *s, size_t offset) {
  try { s->scratch = s->session.GetSpace(offset); } catch (...) { s->scratch.clear(); }
  return s->scratch.c_str();
}
size_t brt_session_op_num(brt_session *s) { return s->session.GetOpNum(); }
const char *brt_session_op_key(brt_session *s, size_t i) {
  return i < s->session.GetOpNum() ? s->session.GetOpKey(i).c_str() : "";
}

long brt_session_op_attr_blob(brt_session *s, size_t op_index, const char *name, void *out, size_t cap) {
  try {
    const OpKernelInfo *info = s->session.GetOpKernelInfo(op_index);
    if (!info) return -1;
    OpAccessor acc(*info);
    size_t n = 0;
    void *blob = acc.GetAttrAsVoidPtr(name, &n);
    std::memcpy(out, blob, n < cap ? n : cap);
    std::free(blob);
    return (long)n;
  } catch (const std::exception &e) {
    g_error = e.what();
    return -1;
  }
}

brt_request *brt_request_create(brt_session *s, void *stream, int use_external_stream) {
  try {
    std::unique_ptr<brt_request> r(new brt_request);
    r->owner = s;
    WorkQueue *wq = use_external_stream ? MakeRocmExternalStreamWorkQueue(stream) : nullptr;
    const common::Status st = s->session.NewRequestContext(&r->ctx, wq);
    if (!st.IsOK()) { g_error = st.ErrorMessage(); return nullptr; }
    return r.release();
  } catch (const std::exception &e) {
    g_error = e.what();
    return nullptr;
  }
}
void brt_request_destroy(brt_request *r) { delete r; }

int brt_request_bind_arg(brt_request *r, size_t offset, void *ptr) {
  return Guard([&] { return FromStatus(r->ctx->BindArg(offset, ptr)); });
}
void *brt_request_get_arg(brt_request *r, size_t offset) {
  try { return r->ctx->GetArg(offset); } catch (const std::exception &e) { g_error = e.what(); return nullptr; }
}
int brt_request_finish_io_binding(brt_request *r) {
  return Guard([&] { r->ctx->FinishIOBinding(); return 0; });
}
int brt_request_sync(brt_request *r) {
  if (r->owner->plan_only) return 0;
  return Guard([&] { return FromStatus(r->ctx->Sync()); });
}
int brt_session_run(brt_session *s, brt_request *r) {
  if (s->plan_only) return Fail("this session was created without a device (device_id < 0): it can load and plan, not run");
  return Guard([&] { return FromStatus(s->session.Run(*r->ctx)); });
}
void brt_request_add_op_listener(brt_request *r, brt_op_listener cb, void *user) {
  r->ctx->AddOpRunListener([cb, user](const OpRunEvent &e) {
    cb(user, e.info->GetOp().key.c_str(), e.info->GetOpId(), e.after ? 1 : 0);
  });
}

}  // extern "C"
