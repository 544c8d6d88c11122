// brt.h -- a compact, MLIR-free host runtime with the shape of ByteIR's BRT, sized to the
// op-kernel hot path: a ByRE text reader, the kernel registry, execution providers, op kernels
// with per-frame workspaces, allocators, work queues, sessions and request contexts.
//
// Names and call protocol follow the reference so that provider code reads the same
// (paths relative to the reference checkout, runtime/include/brt/core/...):
//   common::Status                       common/status.h:29-181
//   IAllocator                           framework/allocator.h:49-62
//   WorkQueue                            context/work_queue.h:48-89
//   OpKernelInfo / OpAccessor            framework/op_kernel_info.h:53-68, op_accessor.h:36-97
//   OpKernel                             framework/op_kernel.h:69-178
//   KernelRegistry + static registration framework/kernel_registry.h:28-94
//   ExecutionProvider                    framework/execution_provider.h:41-115
//   ExecutionContext / ExecutionFrame    context/execution_context.h:36-50, execution_frame.h:97-160
//   Events / EventListenerManager        framework/event.h:27-74
//   OpKernelWithWorkspace                framework/op_kernel_impl_base.h:116-149 (the Workspace argument)
//   Session / RequestContext             session/session.h:50-146, request_context.h:44-92
// This host code includes no HIP header: devices are reached through the C ABI of
// libbrt_rocm_kernels.so (include/brt_rocm_kernels.h).
#pragma once

#include <array>
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace brt {

// ---- status and errors ------------------------------------------------------------------
namespace common {
class Status {
public:
  Status() = default;  // OK
  static Status OK() { return Status(); }
  static Status Fail(const std::string &msg) { Status s; s.ok_ = false; s.msg_ = msg; return s; }
  bool IsOK() const { return ok_; }
  const std::string &ErrorMessage() const { return msg_; }

private:
  bool ok_ = true;
  std::string msg_;
};
}  // namespace common

class BrtException : public std::runtime_error {
public:
  using std::runtime_error::runtime_error;
};
[[noreturn]] void Throw(const char *file, int line, const std::string &msg);
#define BRT_THROW(msg) ::brt::Throw(__FILE__, __LINE__, (msg))
#define BRT_ENFORCE(cond, ...)                                                         \
  do {                                                                                 \
    if (!(cond)) ::brt::Throw(__FILE__, __LINE__, std::string(#cond " was false. ") + std::string(__VA_ARGS__)); \
  } while (0)

// ---- element types -----------------------------------------------------------------------
enum class DTypeEnum { Invalid = 0, Float32, Float16, BFloat16, Float64, Int8, Int16, Int32, Int64, UInt8, Bool };
size_t GetDTypeByte(DTypeEnum t);
const char *GetDTypeName(DTypeEnum t);
using Shape = std::vector<int64_t>;
int64_t LinearizedShape(const Shape &shape);

namespace reduction {
// dims dropped from src_shape; throws on an out-of-range dimension
Shape DeduceOutputShape(const Shape &src_shape, const std::vector<int64_t> &dimensions);
}

// ---- ByRE IR (text) ------------------------------------------------------------------------
namespace ir {

struct MemRefType {
  Shape shape;
  DTypeEnum dtype = DTypeEnum::Invalid;
  std::string space;  // memory-space string, selects the allocator ("cuda", "cpu", ...)
  size_t Bytes() const { return (size_t)LinearizedShape(shape) * GetDTypeByte(dtype); }
};

struct Scalar {  // one element of an array attribute
  bool is_float = false;
  int64_t i = 0;
  double f = 0.0;
};

struct Attr {
  enum Kind { Unit, Int, Float, String, Bool, Array, DenseInt, DenseFloat } kind = Unit;
  int64_t i = 0;
  double f = 0.0;
  bool b = false;
  std::string s;
  std::vector<Scalar> elems;  // Array / DenseInt / DenseFloat
};

enum ArgType { kInput = 1, kOutput = 2, kWeight = 4 };  // byre.argtype bits

struct Value {
  std::string name;   // SSA name including '%'
  MemRefType type;
  int arg_index = -1;      // position in the entry function signature, or -1
  int alias_of = -1;       // value id this one aliases (byre.alias), or -1
  int64_t alias_offset = 0;  // in elements of the aliased value's type
  bool is_alloc = false;   // produced by memref.alloc
};

struct Op {
  std::string name;             // "byre.compute", "byre.custom", ...
  std::string key;              // callee symbol == kernel registry key
  std::vector<int> operands;    // value ids
  std::map<std::string, Attr> attrs;
  int line = 0;
};

struct EntryArg {
  int value = -1;
  std::string argname;  // byre.argname
  int argtype = 0;      // byre.argtype
};

// Parsed module: one entry function (the reference also assumes one, ir.cc:222).
class ByREHandle {
public:
  common::Status LoadFromFile(const std::string &path);
  common::Status LoadFromText(const std::string &text);

  std::string entry_name;
  std::vector<Value> values;
  std::vector<EntryArg> args;
  std::vector<Op> ops;  // compute/custom ops in program order (alias/alloc are folded into values)
  std::map<std::string, Attr> func_attrs;
};

}  // namespace ir

// ---- allocators ----------------------------------------------------------------------------
constexpr size_t kAllocAlignment = 256;

class IAllocator {
public:
  explicit IAllocator(std::string key) : key_(std::move(key)) {}
  virtual ~IAllocator() = default;
  virtual void *Alloc(size_t size) = 0;
  virtual void Free(void *p) = 0;
  const std::string &Key() const { return key_; }  // matched against the memref memory space

private:
  std::string key_;
};

// ---- work queues -----------------------------------------------------------------------------
// A device pointer as op kernels see it (core/framework/value.h: AsyncValue is void *).
using AsyncValue = void *;
using AsyncValueRef = void *;
namespace cuda {}  // sources written for the CUDA provider say `using namespace brt::cuda;`
namespace rocm {}

// Task kinds of a device work queue, with the reference's numbering
// (include/brt/backends/cuda/device/cuda_work_queue.h:32-40); kernels written for the CUDA
// provider pass them as plain integers.
enum ROCMTaskType : int { kCompute = 0, kH2D = 1, kD2H = 2, kRecordEvent = 3, kWaitEvent = 4, kComputeDrv = 5, kD2D = 6 };
using CUDATaskType = ROCMTaskType;

// Launch extents as the args array of a kCompute task carries them: three 32-bit extents, the
// layout of the CUDA / HIP dim3, so that a kernel source that includes <hip/hip_runtime.h> can
// hand its own dim3 objects over.
struct Dim3 {
  unsigned x = 1, y = 1, z = 1;
  Dim3() = default;
  Dim3(unsigned x_, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
// 1-D launch shape for `work_item` items, 256 per block (MakeCUDAGridAndBlock,
// include/brt/backends/cuda/device/common/util.h:39-45)
inline std::pair<Dim3, Dim3> MakeROCMGridAndBlock(int64_t work_item) {
  return {Dim3((unsigned)((work_item + 255) / 256)), Dim3(256)};
}
inline std::pair<Dim3, Dim3> MakeCUDAGridAndBlock(int64_t work_item) { return MakeROCMGridAndBlock(work_item); }

class WorkQueue {
public:
  explicit WorkQueue(std::string name) : name_(std::move(name)) {}
  virtual ~WorkQueue() = default;
  const std::string &name() const { return name_; }
  // Enqueue a call (core/context/work_queue.h:62-68).  kCompute: func is the host-side handle
  // of a device function and args = {grid, block, dynamic LDS bytes (size_t), kernel
  // argument 0, ...}, each a pointer to the value; kH2D / kD2H / kD2D: args = {dst, src, byte
  // count}, each a pointer to the value.  op_id and dependency name the op and the ops it
  // waits for; a single-stream queue orders by enqueueing and ignores them.
  virtual common::Status AddTask(int task_type, const void *func, void **args, int op_id, const std::vector<int> &dependency) = 0;
  // Enqueue a call on the host in queue order: `task` points to a std::function<void(void)>
  // (what the DispatchHostTask macro below passes); the queue copies it.
  virtual common::Status AddHostTask(const void *task, void **args, int op_id, const std::vector<int> &dependency) = 0;
  // Enqueue through a functor, which is called immediately.
  common::Status AddTask(std::function<common::Status()> enqueue_functor) { return enqueue_functor(); }
  virtual common::Status Sync() = 0;
  // device queues expose the stream kernels are enqueued on (void* == hipStream_t)
  virtual void *GetComputeStream() { return nullptr; }

protected:
  std::unordered_map<int, int> id_to_stream_map_;

private:
  std::string name_;
  WorkQueue(const WorkQueue &) = delete;
  WorkQueue &operator=(const WorkQueue &) = delete;
};

// ---- events ----------------------------------------------------------------------------------
class OpKernelInfo;
// Event kinds and their payloads, as the reference's Events (framework/event.h:27-50): a
// listener is registered for one kind and receives that kind's struct.
struct Events {
  struct BeforeExecutionPlanRun { static constexpr uint8_t kIdx = 0; };
  struct AfterExecutionPlanRun { static constexpr uint8_t kIdx = 1; };
  struct BeforeOpKernelRun { static constexpr uint8_t kIdx = 2; const OpKernelInfo &info; };
  struct AfterOpKernelRun { static constexpr uint8_t kIdx = 3; const OpKernelInfo &info; };
  static constexpr uint8_t kSize = 4;
  template <typename T> using Listener = std::function<void(const T &)>;
};

class EventListenerManager {
public:
  template <typename T> void AddEventListener(Events::Listener<T> &&listener) {
    static_assert(T::kIdx < Events::kSize, "unknown event kind");
    auto held = std::make_shared<Events::Listener<T>>(std::move(listener));
    slots_[T::kIdx].push_back([held](const void *event) { (*held)(*static_cast<const T *>(event)); });
  }
  template <typename T> void SignalEvent(const T &event) {
    for (auto &call : slots_[T::kIdx]) call(&event);
  }

private:
  std::array<std::vector<std::function<void(const void *)>>, Events::kSize> slots_;
};

// the flat form the C ABI hands to foreign hosts: one callback for both op-kernel events
struct OpRunEvent {
  const OpKernelInfo *info;
  bool after;  // false: BeforeOpKernelRun, true: AfterOpKernelRun
};
using OpRunListener = std::function<void(const OpRunEvent &)>;

// ---- execution frame / context -----------------------------------------------------------------
class Session;
class ExecutionFrame {
public:
  // Names the per-frame state slots of a plan (workspaces, handles): a key gets one offset the
  // first time any frame asks for it, every frame then fills its own slot at that offset
  // (the reference's ExecutionFrame::StateInfo, context/execution_frame.h:97-160).
  struct StateInfo {
    bool HasState(const std::string &key);
    size_t GetStateOffset(const std::string &key);  // throws for an unknown key
    // creates the key's offset if needed, and this frame's state (by calling `make`) if the
    // frame has none at that offset
    common::Status CreateStateIfNotExist(const std::string &key, ExecutionFrame *frame, const std::function<void *()> &make);
    void Clear();  // forgets every key (a session does this when it loads another model)

  private:
    std::mutex mutex_;
    std::unordered_map<std::string, size_t> name_to_offset_;
  };

  // device pointer of a value id (entry argument, intermediate or alias)
  void *GetAsyncValue(int value_id) const;
  // per-frame state by StateInfo offset
  void *GetState(size_t offset) const { return offset < state_.size() ? state_[offset] : nullptr; }
  void SetState(size_t offset, void *p);
  void *GetAndResetState(size_t offset);

private:
  friend class Session;
  friend class RequestContext;
  std::vector<void *> base_;        // per value: bound/allocated pointer (aliases resolved lazily)
  std::vector<bool> owned_;         // allocated by the frame
  std::vector<void *> state_;       // per StateInfo offset
  std::vector<std::pair<std::string, void *>> arenas_;  // one block per memory space for the intermediates
  const ir::ByREHandle *ir_ = nullptr;
  bool prologue_done_ = false;
  size_t prologue_count_ = 0;       // kernels whose ProloguePerFrame has run on this frame (a prefix of the plan)
  bool io_bound_ = false;
};

// A light bundle of what an op kernel may touch while it runs; owns nothing
// (context/execution_context.h:36-50; the distributed backend of the reference is not part of
// this build).
struct ExecutionContext {
  ExecutionFrame *exec_frame;
  WorkQueue *work_queue;
  ExecutionFrame::StateInfo &frame_state_info;
  EventListenerManager *event_listener_manager;
  ExecutionContext(ExecutionFrame *frame, WorkQueue *wq, ExecutionFrame::StateInfo &fs_info, EventListenerManager *event_mgr)
      : exec_frame(frame), work_queue(wq), frame_state_info(fs_info), event_listener_manager(event_mgr) {}
};

// ---- op kernels --------------------------------------------------------------------------------
class ExecutionProvider;

class OpKernelInfo {
public:
  OpKernelInfo(const ExecutionProvider &provider, const ir::ByREHandle &ir, int op_index,
               const std::unordered_map<std::string, std::unique_ptr<IAllocator>> &allocators,
               std::vector<int> dependency = {})
      : provider_(provider), ir_(ir), op_index_(op_index), allocators_(allocators), dependency_(std::move(dependency)) {}
  const ExecutionProvider &GetExecutionProvider() const { return provider_; }
  const ir::ByREHandle &GetIR() const { return ir_; }
  const ir::Op &GetOp() const { return ir_.ops[op_index_]; }
  int GetOpId() const { return op_index_; }
  // ids of the earlier ops whose results this op consumes, by the operands' memory effects
  // (framework/op_kernel_info.h:95, computed as in execution_plan.cc:243-308)
  const std::vector<int> &GetDependency() const { return dependency_; }
  IAllocator *GetAllocator(const std::string &space) const;

private:
  const ExecutionProvider &provider_;
  const ir::ByREHandle &ir_;
  int op_index_;
  const std::unordered_map<std::string, std::unique_ptr<IAllocator>> &allocators_;
  std::vector<int> dependency_;
};

// Reads operands and attributes of one op; the only window op kernels have on the IR.
class OpAccessor {
public:
  explicit OpAccessor(const OpKernelInfo &info, ExecutionFrame *frame = nullptr) : info_(info), frame_(frame) {}
  size_t GetNumArgs() const;
  Shape GetArgShape(size_t i) const;
  DTypeEnum GetArgDTypeEnum(size_t i) const;
  std::string GetArgSpace(size_t i) const;
  bool HasAttr(const std::string &name) const;
  bool GetAttrAsBool(const std::string &name) const;
  int64_t GetAttrAsInt(const std::string &name) const;
  float GetAttrAsFloat(const std::string &name) const;
  std::string GetAttrAsString(const std::string &name) const;
  std::vector<int64_t> GetAttrAsIntArray(const std::string &name) const;
  // malloc'ed, unpadded blob: i64 -> 8 bytes, f32 -> 4 bytes; caller frees
  void *GetAttrAsVoidPtr(const std::string &name, size_t *size = nullptr) const;
  std::string GetUID() const;
  static int64_t GetNumElementsOfShape(const Shape &shape) { return LinearizedShape(shape); }
  // needs a frame
  AsyncValueRef GetArgAsyncValueRef(size_t i) const;

private:
  const ir::Attr &Find(const std::string &name) const;
  const OpKernelInfo &info_;
  ExecutionFrame *frame_;
};

class OpKernel {
public:
  // The four flags say which hooks the kernel implements; the plan calls only those
  // (framework/op_kernel.h:69-78, execution_plan.cc:313-352).
  explicit OpKernel(const OpKernelInfo &info, bool prologue_per_session = false, bool epilogue_per_session = false,
                    bool prologue_per_frame = false, bool epilogue_per_frame = false)
      : info_(info), has_prologue_per_session_(prologue_per_session), has_epilogue_per_session_(epilogue_per_session),
        has_prologue_per_frame_(prologue_per_frame), has_epilogue_per_frame_(epilogue_per_frame) {}
  virtual ~OpKernel() = default;
  OpKernel(const OpKernel &) = delete;
  OpKernel &operator=(const OpKernel &) = delete;
  // once when the model has been loaded / when the session ends
  virtual common::Status ProloguePerSession() { return common::Status::Fail("OpKernel no implemented."); }
  virtual common::Status EpiloguePerSession() { return common::Status::Fail("OpKernel no implemented."); }
  // once per frame before its first run / when the frame is destroyed (workspace life cycle)
  virtual common::Status ProloguePerFrame(const ExecutionContext &) { return common::Status::Fail("OpKernel no implemented."); }
  virtual common::Status EpiloguePerFrame(const ExecutionContext &) { return common::Status::Fail("OpKernel no implemented."); }
  // enqueue on ctx.work_queue; never synchronises
  virtual common::Status RunImpl(const ExecutionContext &) { return common::Status::Fail("OpKernel no implemented."); }
  common::Status Run(const ExecutionContext &ctx);  // Before/AfterOpKernelRun events around RunImpl
  const OpKernelInfo &GetOpKernelInfo() const { return info_; }
  bool HasProloguePerSession() const { return has_prologue_per_session_; }
  bool HasEpiloguePerSession() const { return has_epilogue_per_session_; }
  bool HasProloguePerFrame() const { return has_prologue_per_frame_; }
  bool HasEpiloguePerFrame() const { return has_epilogue_per_frame_; }

protected:
  const OpKernelInfo info_;
  bool has_prologue_per_session_, has_epilogue_per_session_, has_prologue_per_frame_, has_epilogue_per_frame_;
};

// An op kernel with a temporary workspace: the size is asked once per frame, the buffer comes
// from the allocator of the kernel's last operand, lives in the frame's state under the op's
// UID and is released with the frame -- what the reference's `Workspace` kernel argument does
// (framework/op_kernel_impl_base.h:116-149).
class OpKernelWithWorkspace : public OpKernel {
public:
  explicit OpKernelWithWorkspace(const OpKernelInfo &info) : OpKernel(info, false, false, true, true) {}
  virtual size_t GetWorkspaceSize(const ExecutionContext &ctx) const = 0;
  common::Status ProloguePerFrame(const ExecutionContext &ctx) override;
  common::Status EpiloguePerFrame(const ExecutionContext &ctx) override;

protected:
  void *GetWorkspace(const ExecutionContext &ctx) const;  // nullptr when the size is 0
  IAllocator *GetAllocator() const;
  std::string GetOpUID() const;
};

using KernelCreateFn = std::function<std::shared_ptr<OpKernel>(const OpKernelInfo &)>;

class KernelRegistry {
public:
  common::Status Register(const std::string &key, KernelCreateFn fn) {
    map_.emplace(key, std::move(fn));
    return common::Status::OK();
  }
  bool HasKernel(const std::string &key) const { return map_.count(key) != 0; }
  std::shared_ptr<OpKernel> operator()(const std::string &key, const OpKernelInfo &info) const {
    auto it = map_.find(key);
    return it == map_.end() ? nullptr : it->second(info);
  }
  std::vector<std::string> Keys() const;

private:
  std::unordered_map<std::string, KernelCreateFn> map_;
};

using KernelRegistration = std::function<void(KernelRegistry *)>;
void AddKernelRegistration(const std::string &device_kind, const std::string &provider_name, KernelRegistration fn);
void RegisterKernels(const std::string &device_kind, const std::string &provider_name, KernelRegistry *registry);

#define BRT_STATIC_KERNEL_REGISTRATION(KIND, PROVIDER, FUNC) BRT_STATIC_KERNEL_REGISTRATION_1(KIND, PROVIDER, FUNC, __COUNTER__)
#define BRT_STATIC_KERNEL_REGISTRATION_1(KIND, PROVIDER, FUNC, N) BRT_STATIC_KERNEL_REGISTRATION_2(KIND, PROVIDER, FUNC, N)
#define BRT_STATIC_KERNEL_REGISTRATION_2(KIND, PROVIDER, FUNC, N) \
  [[gnu::unused]] static bool brt_kernel_registration_##N = [] {  \
    ::brt::AddKernelRegistration(KIND, PROVIDER, FUNC);           \
    return true;                                                  \
  }();

namespace DeviceKind {
constexpr const char *CPU = "CPU";
constexpr const char *CUDA = "CUDA";
constexpr const char *ROCM = "ROCM";
}  // namespace DeviceKind
namespace ProviderType {
constexpr const char *BRT = "BRT";
}

class ExecutionProvider {
public:
  ExecutionProvider(const std::string &device_kind, const std::string &name);
  virtual ~ExecutionProvider() = default;
  KernelRegistry *GetKernelRegistry() const { return registry_.get(); }
  const std::string &DeviceKindName() const { return device_kind_; }
  const std::string &Type() const { return name_; }
  // dlopen a shared library whose static initialisers call AddKernelRegistration; must run
  // before the providers that should see those kernels are constructed
  static common::Status StaticRegisterKernelsFromDynlib(const std::string &path);

private:
  std::string device_kind_, name_;
  std::unique_ptr<KernelRegistry> registry_;
};

// ---- session / request context --------------------------------------------------------------------
enum class BrtOwnershipType { OwnedByExternal, OwnedByRuntime };

class RequestContext {
public:
  ~RequestContext();
  common::Status BindArg(size_t offset, const void *value, BrtOwnershipType own = BrtOwnershipType::OwnedByExternal);
  void *GetArg(size_t offset);
  void FinishIOBinding();
  common::Status Sync();
  void AddOpRunListener(OpRunListener l);  // both op-kernel events through one callback
  EventListenerManager &GetEventListenerManager() { return events_; }
  ExecutionFrame *GetExecutionFrame() { return frame_.get(); }
  WorkQueue *GetWorkQueue() { return wq_.get(); }

private:
  friend class Session;
  explicit RequestContext(Session &s) : session_(s) {}
  Session &session_;
  std::unique_ptr<ExecutionFrame> frame_;
  std::unique_ptr<WorkQueue> wq_;
  EventListenerManager events_;
};

class Session {
public:
  Session();
  ~Session();
  common::Status AddExecutionProvider(std::unique_ptr<ExecutionProvider> provider);
  common::Status AddAllocator(std::unique_ptr<IAllocator> allocator);
  IAllocator *GetAllocator(const std::string &key);

  common::Status Load(const std::string &url, const std::string &fmt);         // fmt: "byre"
  common::Status LoadFromMemory(const std::string &text, const std::string &fmt);
  // the request context takes ownership of work_queue; without one, the first provider's
  // default queue is created
  common::Status NewRequestContext(std::unique_ptr<RequestContext> *request, WorkQueue *work_queue = nullptr);
  common::Status Run(RequestContext &request);
  void Cleanup(RequestContext &request) noexcept;

  size_t GetArgNum() const;
  int GetGraphArgOffset(const std::string &name) const;
  const std::vector<size_t> &GetInputArgOffsets() const { return in_offsets_; }
  // bytes of the per-frame arena that holds the intermediates of memory space `space`
  size_t GetIntermediateBytes(const std::string &space) const {
    auto it = arena_bytes_.find(space);
    return it == arena_bytes_.end() ? 0 : it->second;
  }
  const std::vector<size_t> &GetOutputArgOffsets() const { return out_offsets_; }
  const std::vector<size_t> &GetWeightArgOffsets() const { return weight_offsets_; }
  std::string GetArgName(size_t offset) const;
  Shape GetStaticShape(size_t offset) const;
  DTypeEnum GetDType(size_t offset) const;
  std::string GetSpace(size_t offset) const;
  size_t GetOpNum() const { return kernels_.size(); }
  const std::string &GetOpKey(size_t i) const { return ir_->ops[i].key; }
  const OpKernelInfo *GetOpKernelInfo(size_t i) const { return i < infos_.size() ? infos_[i].get() : nullptr; }
  // default work-queue factory, set by the device layer (the reference hard-wires CUDA here,
  // runtime/lib/core/framework/execution_plan.cc:592-601)
  void SetWorkQueueFactory(std::function<WorkQueue *()> f) { wq_factory_ = std::move(f); }

private:
  friend class RequestContext;
  common::Status BuildPlan();
  std::vector<std::unique_ptr<ExecutionProvider>> providers_;
  std::unordered_map<std::string, std::unique_ptr<IAllocator>> allocators_;
  std::unique_ptr<ir::ByREHandle> ir_;
  std::vector<std::shared_ptr<OpKernel>> kernels_;
  std::vector<bool> session_prologue_done_;  // per kernel: ProloguePerSession has returned OK
  void EndPlan() noexcept;                   // EpiloguePerSession of the kernels prepared so far, then drops the plan
  std::vector<std::unique_ptr<OpKernelInfo>> infos_;
  std::vector<size_t> in_offsets_, out_offsets_, weight_offsets_;
  // static memory plan of the memref.alloc intermediates: byte offset of each value inside the
  // arena of its memory space (SIZE_MAX: not an intermediate, or never used by an op), and
  // the arena sizes
  std::vector<size_t> intermediate_offset_;
  std::unordered_map<std::string, size_t> arena_bytes_;
  std::function<WorkQueue *()> wq_factory_;
  ExecutionFrame::StateInfo frame_state_info_;  // shared by every frame of this session
};

// ---- ROCm device layer (rocm_provider.cc) ------------------------------------------------------------
// Allocators answering to the memory spaces "cuda" (so existing ByRE modules run unchanged),
// "cudaPinned" (page-locked host memory) and "cpu"; work queues on an owned or a caller-supplied HIP stream; the provider itself.
using ExternalAllocFn = void *(*)(size_t);
using ExternalFreeFn = void (*)(void *);
std::unique_ptr<IAllocator> MakeRocmAllocator(const std::string &key = "cuda");
std::unique_ptr<IAllocator> MakeExternalAllocator(const std::string &key, ExternalAllocFn a, ExternalFreeFn f);
std::unique_ptr<IAllocator> MakeHostAllocator(const std::string &key = "cpu");
std::unique_ptr<IAllocator> MakeRocmPinnedAllocator(const std::string &key = "cudaPinned");
WorkQueue *MakeRocmSingleStreamWorkQueue(int device_id);
WorkQueue *MakeRocmExternalStreamWorkQueue(void *stream);
common::Status DefaultROCMExecutionProviderFactory(Session *session, int device_id = 0);
common::Status ROCMAllocatorFactory(Session *session, int device_id = 0);

}  // namespace brt

// core/context/work_queue.h:91-101
#define DispatchHostTask(wq, op_id, dependency, stmt)                                              \
  if (wq) {                                                                                        \
    std::function<void(void)> func = [=]() { stmt };                                               \
    wq->AddHostTask(&func, nullptr, op_id, dependency);                                            \
  } else {                                                                                         \
    do {                                                                                           \
      stmt                                                                                         \
    } while (0);                                                                                   \
  }
