// The ROCm execution provider: allocators, work queues and the op kernels of the hot path,
// registered under the reference's op keys so that a ByRE module written for the CUDA provider
// runs unchanged.  Device work goes through the C ABI of libbrt_rocm_kernels.so; this file
// includes no HIP header.
//
// Reference counterparts (runtime/lib/backends/cuda/...):
//   device/cuda_allocator.cc, device/cuda_work_queue.cc:139-177,287-316,
//   providers/default/cuda_provider.cc:46-59,
//   providers/default/reduction/{reduce_impl.h, op_registration.cc},
//   providers/default/custom/custom.cc, providers/default/copy/copy.cc.
#include <dlfcn.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "brt.h"
#include "brt_rocm_kernels.h"

namespace brt {
namespace {

std::string HipErr(int e) { return std::string(brt_rocm_error_string(e)); }
common::Status HipStatus(int e, const char *what) {
  return e == 0 ? common::Status::OK() : common::Status::Fail(std::string(what) + ": " + HipErr(e));
}

// ---- allocators ------------------------------------------------------------------------------
class RocmAllocator : public IAllocator {
public:
  using IAllocator::IAllocator;
  void *Alloc(size_t size) override {
    void *p = nullptr;
    const int e = brt_rocm_malloc(&p, size);
    BRT_ENFORCE(e == 0, "device allocation of " + std::to_string(size) + " bytes failed: " + HipErr(e));
    return p;
  }
  void Free(void *p) override { if (p) brt_rocm_free(p); }
};

class ExternalAllocator : public IAllocator {  // e.g. a framework's caching allocator
public:
  ExternalAllocator(const std::string &key, ExternalAllocFn a, ExternalFreeFn f) : IAllocator(key), a_(a), f_(f) {}
  void *Alloc(size_t size) override { return a_(size); }
  void Free(void *p) override { if (p) f_(p); }

private:
  ExternalAllocFn a_;
  ExternalFreeFn f_;
};

class RocmPinnedAllocator : public IAllocator {  // page-locked host memory (hipHostMalloc)
public:
  using IAllocator::IAllocator;
  void *Alloc(size_t size) override {
    void *p = nullptr;
    const int e = brt_rocm_host_malloc(&p, size ? size : kAllocAlignment);
    BRT_ENFORCE(e == 0, "pinned host allocation of " + std::to_string(size) + " bytes failed: " + HipErr(e));
    return p;
  }
  void Free(void *p) override { if (p) brt_rocm_host_free(p); }
};

class HostAllocator : public IAllocator {
public:
  using IAllocator::IAllocator;
  void *Alloc(size_t size) override {
    void *p = nullptr;
    if (posix_memalign(&p, kAllocAlignment, size ? size : kAllocAlignment) != 0) BRT_THROW("host allocation failed");
    return p;
  }
  void Free(void *p) override { std::free(p); }
};

// ---- work queues ---------------------------------------------------------------------------------
class RocmWorkQueue : public WorkQueue {
public:
  RocmWorkQueue(const std::string &name, void *stream, bool owned) : WorkQueue(name), stream_(stream), owned_(owned) {}
  ~RocmWorkQueue() override {
    if (owned_ && stream_) brt_rocm_stream_destroy(stream_);
  }
  common::Status Sync() override { return HipStatus(brt_rocm_stream_synchronize(stream_), "stream synchronize"); }
  void *GetComputeStream() override { return stream_; }
  // One stream: tasks run in the order they are enqueued, so op_id and dependency need no
  // events here (CUDASingleStreamWorkQueue::AddTask, cuda_work_queue.cc:150-172).  There is no
  // driver-API module loading in this provider, hence no kComputeDrv.
  common::Status AddTask(int task_type, const void *func, void **args, int /*op_id*/, const std::vector<int> & /*dependency*/) override {
    switch (task_type) {
    case kCompute: {
      BRT_ENFORCE(func != nullptr && args != nullptr, "kCompute needs a device function and {grid, block, shared bytes, arguments...}");
      const Dim3 *grid = static_cast<const Dim3 *>(args[0]), *block = static_cast<const Dim3 *>(args[1]);
      const size_t shared = *static_cast<const size_t *>(args[2]);
      const unsigned g[3] = {grid->x, grid->y, grid->z}, b[3] = {block->x, block->y, block->z};
      return HipStatus(brt_rocm_launch_kernel(func, g, b, args + 3, shared, stream_), "kernel launch");
    }
    case kH2D: case kD2H: case kD2D: {
      BRT_ENFORCE(args != nullptr, "a copy task needs {dst, src, byte count}");
      void *dst = *static_cast<void **>(args[0]), *src = *static_cast<void **>(args[1]);
      const size_t count = *static_cast<const size_t *>(args[2]);
      const int e = task_type == kH2D ? brt_rocm_memcpy_h2d(dst, src, count, stream_)
                    : task_type == kD2H ? brt_rocm_memcpy_d2h(dst, src, count, stream_)
                                        : brt_rocm_memcpy_d2d(dst, src, count, stream_);
      return HipStatus(e, "copy task");
    }
    default:
      return common::Status::Fail("unsupported task type " + std::to_string(task_type));
    }
  }
  // The task is copied and runs on the host once everything enqueued before it has finished
  // (hipLaunchHostFunc), so a task may read what earlier kernels wrote.  The reference's
  // single-stream queue calls the function on the spot instead (cuda_work_queue.h:68-73) and
  // its multi-stream queue enqueues it (cuda_work_queue.cc:258-264); the DispatchHostTask macro
  // hands over a function object that dies with its scope, which is why it is copied here.
  common::Status AddHostTask(const void *task, void ** /*args*/, int /*op_id*/, const std::vector<int> & /*dependency*/) override {
    BRT_ENFORCE(task != nullptr, "AddHostTask needs a std::function<void(void)>");
    auto *held = new std::function<void(void)>(*static_cast<const std::function<void(void)> *>(task));
    const int e = brt_rocm_launch_host_func(stream_, &RocmWorkQueue::CallHostTask, held);
    if (e != 0) delete held;
    return HipStatus(e, "host task");
  }

private:
  static void CallHostTask(void *task) {
    auto *f = static_cast<std::function<void(void)> *>(task);
    (*f)();
    delete f;
  }
  void *stream_;
  bool owned_;
};

void *StreamOf(const ExecutionContext &ctx) {
  BRT_ENFORCE(ctx.work_queue != nullptr, "op kernel needs a work queue");
  return ctx.work_queue->GetComputeStream();
}

// ---- ReduceSumOp / ReduceMaxOp ----------------------------------------------------------------------
// Canonicalises the reduced dimensions to [A, B, C] exactly as ReduceImpl's constructor
// (reduce_impl.h:30-59) and owns a per-frame workspace sized at plan time.
class ReduceOpKernel : public OpKernelWithWorkspace {
public:
  ReduceOpKernel(const OpKernelInfo &info, int op, int dtype) : OpKernelWithWorkspace(info), op_(op), dtype_(dtype) {
    OpAccessor acc(info_);
    BRT_ENFORCE(acc.GetNumArgs() == 2, "reduce takes an input and an output");
    Shape shape = acc.GetArgShape(0);
    const Shape tshape = acc.GetArgShape(1);
    std::vector<int64_t> dims = acc.GetAttrAsIntArray("dimensions");
    const DTypeEnum want = dtype == BRT_ROCM_F32 ? DTypeEnum::Float32 : DTypeEnum::Float16;
    BRT_ENFORCE(acc.GetArgDTypeEnum(0) == want && acc.GetArgDTypeEnum(1) == want, "element type does not match the op key");
    BRT_ENFORCE(tshape == reduction::DeduceOutputShape(shape, dims), "output shape is not the input shape without the reduced dimensions");
    dims.erase(std::remove_if(dims.begin(), dims.end(), [&](int64_t d) { return shape[(size_t)d] == 1; }), dims.end());
    if (dims.empty()) {  // nothing to fold: a plain copy of every element
      A_ = B_ = 0;
      C_ = (size_t)LinearizedShape(shape);
      return;
    }
    std::sort(dims.begin(), dims.end());
    for (size_t i = 0; i + 1 < dims.size(); ++i)
      BRT_ENFORCE(dims[i + 1] - dims[i] == 1, "Only consecutive dimensions reduction is supported now.");
    A_ = B_ = C_ = 1;
    for (int64_t i = 0; i < dims.front(); ++i) A_ *= (size_t)shape[(size_t)i];
    for (int64_t d : dims) B_ *= (size_t)shape[(size_t)d];
    for (size_t i = (size_t)dims.back() + 1; i < shape.size(); ++i) C_ *= (size_t)shape[i];
  }

  // asked once per frame, where the reference asks ReduceImpl::GetWorkspaceSize (reduce_impl.h:76-79)
  size_t GetWorkspaceSize(const ExecutionContext &) const override { return brt_rocm_reduce_workspace_bytes(dtype_, A_, B_, C_); }

  common::Status RunImpl(const ExecutionContext &ctx) override {
    OpAccessor acc(info_, ctx.exec_frame);
    const int e = brt_rocm_reduce(op_, dtype_, acc.GetArgAsyncValueRef(0), acc.GetArgAsyncValueRef(1), A_, B_, C_,
                                  GetWorkspace(ctx), GetWorkspaceSize(ctx), StreamOf(ctx));
    return HipStatus(e, "reduce");
  }

private:
  int op_, dtype_;
  size_t A_ = 0, B_ = 0, C_ = 0;
};

// ---- byteir.softmax -----------------------------------------------------------------------------------
// A new op kernel (the reference runtime has none): operands (input, output), attribute `axis`,
// (any axis of the tensor, the last one by default); element type f32, f16 or bf16.
class SoftmaxOpKernel : public OpKernelWithWorkspace {
public:
  explicit SoftmaxOpKernel(const OpKernelInfo &info) : OpKernelWithWorkspace(info) {
    OpAccessor acc(info_);
    BRT_ENFORCE(acc.GetNumArgs() == 2, "softmax takes an input and an output");
    const Shape s = acc.GetArgShape(0);
    BRT_ENFORCE(s == acc.GetArgShape(1), "softmax output shape differs from the input shape");
    BRT_ENFORCE(acc.GetArgDTypeEnum(0) == acc.GetArgDTypeEnum(1), "softmax output type differs from the input type");
    BRT_ENFORCE(!s.empty(), "softmax of a rank-0 tensor");
    int64_t axis = acc.HasAttr("axis") ? acc.GetAttrAsInt("axis") : (int64_t)s.size() - 1;
    if (axis < 0) axis += (int64_t)s.size();
    BRT_ENFORCE(axis >= 0 && axis < (int64_t)s.size(), "softmax axis out of range");
    switch (acc.GetArgDTypeEnum(0)) {
    case DTypeEnum::Float32: dtype_ = BRT_ROCM_F32; break;
    case DTypeEnum::Float16: dtype_ = BRT_ROCM_F16; break;
    case DTypeEnum::BFloat16: dtype_ = BRT_ROCM_BF16; break;
    default: BRT_THROW("softmax element type must be f32, f16 or bf16");
    }
    a_ = b_ = c_ = 1;
    for (int64_t i = 0; i < (int64_t)s.size(); ++i) (i < axis ? a_ : i == axis ? b_ : c_) *= (size_t)s[i];
  }
  // segment partials of an inner-axis softmax with few columns and a long axis; 0 otherwise
  size_t GetWorkspaceSize(const ExecutionContext &) const override { return brt_rocm_softmax_workspace_bytes(dtype_, a_, b_, c_); }
  common::Status RunImpl(const ExecutionContext &ctx) override {
    OpAccessor acc(info_, ctx.exec_frame);
    return HipStatus(brt_rocm_softmax_axis_ws(dtype_, acc.GetArgAsyncValueRef(0), acc.GetArgAsyncValueRef(1), a_, b_, c_,
                                              GetWorkspace(ctx), GetWorkspaceSize(ctx), StreamOf(ctx)), "softmax");
  }

private:
  int dtype_ = 0;
  size_t a_ = 1, b_ = 1, c_ = 1;  // softmax over the middle axis of [a, b, c]
};

// ---- custom -----------------------------------------------------------------------------------------------
// Loads `lib_path`, resolves `api_name` and calls it as  f(void **tensors, void *extra_args, stream)
// (custom.cc:38-86).  The library must export a data symbol VERSION.  The reference compares the
// bytes of that pointer variable with the `version` attribute and passes when they differ, which
// in practice only tests that the symbol exists; the same is required here, and a version string
// that really differs is reported on stderr.
// A relative lib_path that does not resolve from the working directory is looked up by file name
// in $BRT_CUSTOM_LIB_DIR and next to this runtime library, so modules carrying the reference's
// paths ("external_libs/libs/libflash_attn.so") run without a matching directory layout.
class CustomOpKernel : public OpKernelWithWorkspace {
public:
  explicit CustomOpKernel(const OpKernelInfo &info) : OpKernelWithWorkspace(info) {
    OpAccessor acc(info_);
    const std::string lib_path = acc.GetAttrAsString("lib_path");
    const std::string api_name = acc.GetAttrAsString("api_name");
    const std::string version = acc.GetAttrAsString("version");
    handle_ = Open(lib_path);
    BRT_ENFORCE(handle_ != nullptr, "Custom lib " + lib_path + " load failed");
    run_ = reinterpret_cast<RunFn>(dlsym(handle_, api_name.c_str()));
    BRT_ENFORCE(run_ != nullptr, "Couldn't find function: " + api_name);
    void *ver = dlsym(handle_, "VERSION");
    BRT_ENFORCE(ver != nullptr, "Version doesn't exist in custom library!");
    const char *lib_version = *static_cast<const char **>(ver);
    if (lib_version && version != lib_version)
      std::fprintf(stderr, "brt: custom library %s reports version %s, the module asks for %s\n", lib_path.c_str(), lib_version, version.c_str());
    // The (tensors, extra_args, stream) ABI has no error channel and no way to hand over
    // scratch: this library's plain entry points abort on arguments they cannot serve and
    // allocate their scratch themselves.  When the library also exports the extended forms
    // (flash_attn_{fwd,bwd,kvcache}_ws + _workspace_bytes + flash_attn_last_error), the op kernel
    // uses those: a bad module fails Session::Run instead of ending the process, and the
    // scratch is a per-frame workspace from the frame's allocator, sized when the frame is set up.
    static const struct { const char *api, *stem; int dtype; } kExtended[] = {
        {"run_flash_attn_fwd", "flash_attn_fwd", 1},         {"run_flash_attn_fwd_bf16", "flash_attn_fwd", 2},
        {"run_flash_attn_bwd", "flash_attn_bwd", 1},         {"run_flash_attn_bwd_bf16", "flash_attn_bwd", 2},
        {"run_flash_attn_kvcache", "flash_attn_kvcache", 1}, {"run_flash_attn_kvcache_bf16", "flash_attn_kvcache", 2}};
    for (const auto &c : kExtended) {
      if (api_name != c.api) continue;
      const std::string stem(c.stem);
      with_ws_ = reinterpret_cast<WsFn>(dlsym(handle_, (stem + "_ws").c_str()));
      last_error_ = reinterpret_cast<LastErrorFn>(dlsym(handle_, "flash_attn_last_error"));
      is_bwd_ = stem == "flash_attn_bwd";
      if (is_bwd_) bwd_bytes_ = reinterpret_cast<BwdBytesFn>(dlsym(handle_, (stem + "_workspace_bytes").c_str()));
      else bytes_ = reinterpret_cast<BytesFn>(dlsym(handle_, (stem + "_workspace_bytes").c_str()));
      ext_dtype_ = c.dtype;
    }
    if (!with_ws_ || !last_error_ || (!bytes_ && !bwd_bytes_)) with_ws_ = nullptr;  // all or nothing
    // The packed extra_args blob and the scratch size depend on the op's attributes and static
    // shapes only: both are made once here (the reference packs and frees the blob on every run,
    // custom.cc:71-84; the libraries only read it) and live as long as the kernel.
    extra_ = acc.GetAttrAsVoidPtr("extra_args");
    if (with_ws_) {
      if (is_bwd_) {  // operand 11 is dq_accum (flash_api.cu:696-725): the library fills it first
        const size_t accum = acc.GetNumArgs() > 11 ? (size_t)LinearizedShape(acc.GetArgShape(11)) * GetDTypeByte(acc.GetArgDTypeEnum(11)) : 0;
        ws_bytes_ = bwd_bytes_(extra_, ext_dtype_, accum);
      } else {
        ws_bytes_ = bytes_(extra_, ext_dtype_);
      }
    }
  }
  ~CustomOpKernel() override { std::free(extra_); }
  size_t GetWorkspaceSize(const ExecutionContext &) const override { return ws_bytes_; }
  common::Status RunImpl(const ExecutionContext &ctx) override {
    OpAccessor acc(info_, ctx.exec_frame);
    std::vector<void *> tensors(acc.GetNumArgs());
    for (size_t i = 0; i < tensors.size(); ++i) tensors[i] = acc.GetArgAsyncValueRef(i);
    common::Status st = common::Status::OK();
    if (with_ws_) {
      const int e = with_ws_(tensors.data(), extra_, ext_dtype_, GetWorkspace(ctx), ws_bytes_, StreamOf(ctx));
      if (e < 0) st = common::Status::Fail(std::string("custom op: ") + last_error_());
      else if (e > 0) st = HipStatus(e, "custom op launch");
    } else {
      run_(tensors.data(), extra_, StreamOf(ctx));
    }
    return st;
  }

private:
  using RunFn = void (*)(void **, void *, void *);
  using WsFn = int (*)(void **, const void *, int, void *, size_t, void *);
  using BytesFn = size_t (*)(const void *, int);
  using BwdBytesFn = size_t (*)(const void *, int, size_t);
  using LastErrorFn = const char *(*)();
  static void *Open(const std::string &path) {
    if (void *h = dlopen(path.c_str(), RTLD_LAZY | RTLD_GLOBAL)) return h;
    const std::string base = path.substr(path.find_last_of('/') == std::string::npos ? 0 : path.find_last_of('/') + 1);
    if (const char *dir = std::getenv("BRT_CUSTOM_LIB_DIR"))
      if (void *h = dlopen((std::string(dir) + "/" + base).c_str(), RTLD_LAZY | RTLD_GLOBAL)) return h;
    Dl_info self;
    if (dladdr(reinterpret_cast<void *>(&CustomOpKernel::Open), &self) && self.dli_fname) {
      std::string dir(self.dli_fname);
      dir = dir.substr(0, dir.find_last_of('/') == std::string::npos ? 0 : dir.find_last_of('/'));
      if (void *h = dlopen((dir + "/" + base).c_str(), RTLD_LAZY | RTLD_GLOBAL)) return h;
    }
    return nullptr;
  }
  void *handle_ = nullptr;
  RunFn run_ = nullptr;
  WsFn with_ws_ = nullptr;
  BytesFn bytes_ = nullptr;
  BwdBytesFn bwd_bytes_ = nullptr;
  LastErrorFn last_error_ = nullptr;
  bool is_bwd_ = false;
  int ext_dtype_ = 0;
  void *extra_ = nullptr;  // the packed extra_args blob (malloc'ed by the accessor)
  size_t ws_bytes_ = 0;
};

// ---- copies: cpu2cuda, cuda2cpu, cuda2cuda (operands: src, dst) ---------------------------------------------
class CopyOpKernel : public OpKernel {
public:
  CopyOpKernel(const OpKernelInfo &info, int kind) : OpKernel(info), kind_(kind) {
    OpAccessor acc(info_);
    BRT_ENFORCE(acc.GetNumArgs() == 2, "copy takes a source and a destination");
    BRT_ENFORCE(acc.GetArgShape(0) == acc.GetArgShape(1) && acc.GetArgDTypeEnum(0) == acc.GetArgDTypeEnum(1), "copy operands differ in type");
    bytes_ = (size_t)LinearizedShape(acc.GetArgShape(0)) * GetDTypeByte(acc.GetArgDTypeEnum(0));
  }
  common::Status RunImpl(const ExecutionContext &ctx) override {
    OpAccessor acc(info_, ctx.exec_frame);
    void *src = acc.GetArgAsyncValueRef(0), *dst = acc.GetArgAsyncValueRef(1);
    void *s = StreamOf(ctx);
    const int e = kind_ == 0 ? brt_rocm_memcpy_h2d(dst, src, bytes_, s)
                  : kind_ == 1 ? brt_rocm_memcpy_d2h(dst, src, bytes_, s)
                               : brt_rocm_memcpy_d2d(dst, src, bytes_, s);
    return HipStatus(e, "copy");
  }

private:
  int kind_;
  size_t bytes_ = 0;
};

void RegisterRocmOps(KernelRegistry *r) {
  auto reduce = [r](const char *key, int op, int dtype) {
    r->Register(key, [op, dtype](const OpKernelInfo &info) -> std::shared_ptr<OpKernel> {
      return std::make_shared<ReduceOpKernel>(info, op, dtype);
    });
  };
  reduce("ReduceSumOp_f32_f32", BRT_ROCM_REDUCE_SUM, BRT_ROCM_F32);
  reduce("ReduceSumOp_f16_f16", BRT_ROCM_REDUCE_SUM, BRT_ROCM_F16);
  reduce("ReduceMaxOp_f32_f32", BRT_ROCM_REDUCE_MAX, BRT_ROCM_F32);
  reduce("ReduceMaxOp_f16_f16", BRT_ROCM_REDUCE_MAX, BRT_ROCM_F16);
  // The reference defines these four operators (reduction_helper.h:37-137) but instantiates no
  // op kernel for them; the keys follow the naming of the registered ones
  // (reduction/op_registration.cc:27-49).
  reduce("ReduceMinOp_f32_f32", BRT_ROCM_REDUCE_MIN, BRT_ROCM_F32);
  reduce("ReduceMinOp_f16_f16", BRT_ROCM_REDUCE_MIN, BRT_ROCM_F16);
  reduce("ReduceProdOp_f32_f32", BRT_ROCM_REDUCE_PROD, BRT_ROCM_F32);
  reduce("ReduceProdOp_f16_f16", BRT_ROCM_REDUCE_PROD, BRT_ROCM_F16);
  reduce("ReduceMeanOp_f32_f32", BRT_ROCM_REDUCE_MEAN, BRT_ROCM_F32);
  reduce("ReduceMeanOp_f16_f16", BRT_ROCM_REDUCE_MEAN, BRT_ROCM_F16);
  reduce("ReduceSumSqrOp_f32_f32", BRT_ROCM_REDUCE_SUMSQR, BRT_ROCM_F32);
  reduce("ReduceSumSqrOp_f16_f16", BRT_ROCM_REDUCE_SUMSQR, BRT_ROCM_F16);
  r->Register("byteir.softmax", [](const OpKernelInfo &info) -> std::shared_ptr<OpKernel> {
    return std::make_shared<SoftmaxOpKernel>(info);
  });
  r->Register("custom", [](const OpKernelInfo &info) -> std::shared_ptr<OpKernel> {
    return std::make_shared<CustomOpKernel>(info);
  });
  const char *copies[] = {"cpu2cuda", "cuda2cpu", "cuda2cuda"};
  for (int k = 0; k < 3; ++k)
    r->Register(copies[k], [k](const OpKernelInfo &info) -> std::shared_ptr<OpKernel> {
      return std::make_shared<CopyOpKernel>(info, k);
    });
}

}  // namespace

BRT_STATIC_KERNEL_REGISTRATION(DeviceKind::ROCM, ProviderType::BRT, RegisterRocmOps)

std::unique_ptr<IAllocator> MakeRocmAllocator(const std::string &key) { return std::unique_ptr<IAllocator>(new RocmAllocator(key)); }
std::unique_ptr<IAllocator> MakeExternalAllocator(const std::string &key, ExternalAllocFn a, ExternalFreeFn f) {
  return std::unique_ptr<IAllocator>(new ExternalAllocator(key, a, f));
}
std::unique_ptr<IAllocator> MakeHostAllocator(const std::string &key) { return std::unique_ptr<IAllocator>(new HostAllocator(key)); }
std::unique_ptr<IAllocator> MakeRocmPinnedAllocator(const std::string &key) { return std::unique_ptr<IAllocator>(new RocmPinnedAllocator(key)); }

WorkQueue *MakeRocmSingleStreamWorkQueue(int device_id) {
  BRT_ENFORCE(brt_rocm_set_device(device_id) == 0, "cannot select device " + std::to_string(device_id));
  void *s = nullptr;
  const int e = brt_rocm_stream_create(&s);
  BRT_ENFORCE(e == 0, "cannot create a stream: " + HipErr(e));
  return new RocmWorkQueue("rocm_single_stream", s, true);
}
WorkQueue *MakeRocmExternalStreamWorkQueue(void *stream) { return new RocmWorkQueue("rocm_external_stream", stream, false); }

common::Status DefaultROCMExecutionProviderFactory(Session *session, int device_id) {
  session->SetWorkQueueFactory([device_id]() { return MakeRocmSingleStreamWorkQueue(device_id); });
  return session->AddExecutionProvider(std::unique_ptr<ExecutionProvider>(new ExecutionProvider(DeviceKind::ROCM, ProviderType::BRT)));
}

// The device allocator is keyed "cuda": allocator lookup goes by the memref's memory-space string
// (execution_plan.cc:94-95), and existing modules say "cuda".  "rocm" is accepted as well.
common::Status ROCMAllocatorFactory(Session *session, int device_id) {
  const int e = brt_rocm_set_device(device_id);
  if (e != 0) return HipStatus(e, "set device");
  session->AddAllocator(MakeRocmAllocator("cuda"));
  session->AddAllocator(MakeRocmAllocator("rocm"));
  session->AddAllocator(MakeHostAllocator("cpu"));
  // page-locked host memory, the key the reference's CUDAAllocatorFactory registers beside
  // "cuda" (runtime/lib/backends/cuda/device/cuda_allocator.cc:88-110)
  session->AddAllocator(MakeRocmPinnedAllocator("cudaPinned"));
  return common::Status::OK();
}

}  // namespace brt
