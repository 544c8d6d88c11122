// Runtime core: kernel registry, op accessor, execution plan, session and request context.
// Counterparts in the reference (runtime/lib/core/...): framework/kernel_registry.cc,
// framework/op_accessor.cc, framework/execution_plan.cc:62-691, session/session.cc,
// session/request_context.cc, context/execution_frame.cc.
#include <dlfcn.h>

#include <algorithm>
#include <cstring>
#include <mutex>

#include "brt.h"

namespace brt {

void Throw(const char *file, int line, const std::string &msg) {
  const char *base = std::strrchr(file, '/');
  throw BrtException(std::string(base ? base + 1 : file) + ":" + std::to_string(line) + " " + msg);
}

size_t GetDTypeByte(DTypeEnum t) {
  switch (t) {
  case DTypeEnum::Float32: case DTypeEnum::Int32: return 4;
  case DTypeEnum::Float16: case DTypeEnum::BFloat16: case DTypeEnum::Int16: return 2;
  case DTypeEnum::Float64: case DTypeEnum::Int64: return 8;
  case DTypeEnum::Int8: case DTypeEnum::UInt8: case DTypeEnum::Bool: return 1;
  default: return 0;
  }
}

const char *GetDTypeName(DTypeEnum t) {
  switch (t) {
  case DTypeEnum::Float32: return "f32";
  case DTypeEnum::Float16: return "f16";
  case DTypeEnum::BFloat16: return "bf16";
  case DTypeEnum::Float64: return "f64";
  case DTypeEnum::Int8: return "i8";
  case DTypeEnum::Int16: return "i16";
  case DTypeEnum::Int32: return "i32";
  case DTypeEnum::Int64: return "i64";
  case DTypeEnum::UInt8: return "ui8";
  case DTypeEnum::Bool: return "i1";
  default: return "invalid";
  }
}

int64_t LinearizedShape(const Shape &shape) {
  int64_t n = 1;
  for (int64_t d : shape) n *= d;
  return n;
}

namespace reduction {
Shape DeduceOutputShape(const Shape &src_shape, const std::vector<int64_t> &dimensions) {
  std::vector<bool> reduced(src_shape.size(), false);
  for (int64_t d : dimensions) {
    BRT_ENFORCE(0 <= d && d < (int64_t)src_shape.size(), "invalid dimension");
    reduced[(size_t)d] = true;
  }
  Shape out;
  for (size_t i = 0; i < src_shape.size(); ++i)
    if (!reduced[i]) out.push_back(src_shape[i]);
  return out;
}
}  // namespace reduction

// ---- static kernel registration ---------------------------------------------------------------
namespace {
std::mutex &RegMutex() { static std::mutex m; return m; }
std::unordered_map<std::string, std::vector<KernelRegistration>> &RegMap() {
  static std::unordered_map<std::string, std::vector<KernelRegistration>> m;
  return m;
}
}  // namespace

void AddKernelRegistration(const std::string &device_kind, const std::string &provider_name, KernelRegistration fn) {
  std::lock_guard<std::mutex> g(RegMutex());
  RegMap()[device_kind + ":" + provider_name].push_back(std::move(fn));
}

void RegisterKernels(const std::string &device_kind, const std::string &provider_name, KernelRegistry *registry) {
  std::vector<KernelRegistration> regs;
  {
    std::lock_guard<std::mutex> g(RegMutex());
    auto it = RegMap().find(device_kind + ":" + provider_name);
    if (it != RegMap().end()) regs = it->second;
  }
  for (auto &r : regs) r(registry);
}

std::vector<std::string> KernelRegistry::Keys() const {
  std::vector<std::string> k;
  for (auto &kv : map_) k.push_back(kv.first);
  std::sort(k.begin(), k.end());
  return k;
}

ExecutionProvider::ExecutionProvider(const std::string &device_kind, const std::string &name)
    : device_kind_(device_kind), name_(name), registry_(new KernelRegistry) {
  RegisterKernels(device_kind, name, registry_.get());
}

common::Status ExecutionProvider::StaticRegisterKernelsFromDynlib(const std::string &path) {
  if (!dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL))
    return common::Status::Fail(std::string("cannot load kernel library: ") + dlerror());
  return common::Status::OK();
}

// ---- OpKernelInfo / OpAccessor ------------------------------------------------------------------
IAllocator *OpKernelInfo::GetAllocator(const std::string &space) const {
  auto it = allocators_.find(space);
  return it == allocators_.end() ? nullptr : it->second.get();
}

size_t OpAccessor::GetNumArgs() const { return info_.GetOp().operands.size(); }

Shape OpAccessor::GetArgShape(size_t i) const {
  BRT_ENFORCE(i < GetNumArgs(), "operand index out of range");
  return info_.GetIR().values[info_.GetOp().operands[i]].type.shape;
}
DTypeEnum OpAccessor::GetArgDTypeEnum(size_t i) const {
  BRT_ENFORCE(i < GetNumArgs(), "operand index out of range");
  return info_.GetIR().values[info_.GetOp().operands[i]].type.dtype;
}
std::string OpAccessor::GetArgSpace(size_t i) const {
  BRT_ENFORCE(i < GetNumArgs(), "operand index out of range");
  return info_.GetIR().values[info_.GetOp().operands[i]].type.space;
}
bool OpAccessor::HasAttr(const std::string &name) const { return info_.GetOp().attrs.count(name) != 0; }

const ir::Attr &OpAccessor::Find(const std::string &name) const {
  auto it = info_.GetOp().attrs.find(name);
  if (it == info_.GetOp().attrs.end()) BRT_THROW("Attribute " + name + " is not set");
  return it->second;
}
bool OpAccessor::GetAttrAsBool(const std::string &name) const {
  const ir::Attr &a = Find(name);
  if (a.kind == ir::Attr::Bool) return a.b;
  if (a.kind == ir::Attr::Int) return a.i != 0;
  BRT_THROW("Attribute " + name + " is not a bool");
}
int64_t OpAccessor::GetAttrAsInt(const std::string &name) const {
  const ir::Attr &a = Find(name);
  if (a.kind != ir::Attr::Int) BRT_THROW("Attribute " + name + " is not an integer");
  return a.i;
}
float OpAccessor::GetAttrAsFloat(const std::string &name) const {
  const ir::Attr &a = Find(name);
  if (a.kind != ir::Attr::Float && a.kind != ir::Attr::Int) BRT_THROW("Attribute " + name + " is not a float");
  return (float)a.f;
}
std::string OpAccessor::GetAttrAsString(const std::string &name) const {
  const ir::Attr &a = Find(name);
  if (a.kind != ir::Attr::String) BRT_THROW("Attribute " + name + " is not a string");
  return a.s;
}
// accepts [0 : i64, 1 : i64] and dense<[0, 1]> : tensor<2xi64> (op_accessor.cc:98-122)
std::vector<int64_t> OpAccessor::GetAttrAsIntArray(const std::string &name) const {
  const ir::Attr &a = Find(name);
  if (a.kind != ir::Attr::Array && a.kind != ir::Attr::DenseInt) BRT_THROW("Attribute " + name + " is not an integer array");
  std::vector<int64_t> out;
  for (const ir::Scalar &s : a.elems) {
    if (s.is_float) BRT_THROW("Cannot cast " + name + " to array of IntAttr");
    out.push_back(s.i);
  }
  return out;
}
// i64 -> 8 bytes, f32 -> 4 bytes, no padding (op_accessor.cc:212-242)
void *OpAccessor::GetAttrAsVoidPtr(const std::string &name, size_t *size) const {
  const ir::Attr &a = Find(name);
  if (a.kind != ir::Attr::Array) BRT_THROW("Attribute " + name + " is not supported to get as void *");
  size_t total = 0;
  for (const ir::Scalar &s : a.elems) total += s.is_float ? sizeof(float) : sizeof(int64_t);
  char *blob = static_cast<char *>(std::malloc(total ? total : 1));
  size_t pos = 0;
  for (const ir::Scalar &s : a.elems) {
    if (s.is_float) { const float v = (float)s.f; std::memcpy(blob + pos, &v, 4); pos += 4; }
    else { const int64_t v = s.i; std::memcpy(blob + pos, &v, 8); pos += 8; }
  }
  if (size) *size = total;
  return blob;
}
std::string OpAccessor::GetUID() const { return info_.GetOp().key + "#" + std::to_string(info_.GetOpId()); }

void *OpAccessor::GetArgAsyncValueRef(size_t i) const {
  BRT_ENFORCE(frame_ != nullptr, "need active execution frame by: GetArgAsyncValueRef");
  BRT_ENFORCE(i < GetNumArgs(), "operand index out of range");
  return frame_->GetAsyncValue(info_.GetOp().operands[i]);
}

common::Status OpKernel::Run(const ExecutionContext &ctx) {
  if (ctx.event_listener_manager) ctx.event_listener_manager->SignalEvent<Events::BeforeOpKernelRun>({info_});
  common::Status s;
  try {
    s = RunImpl(ctx);
  } catch (const std::exception &e) {
    s = common::Status::Fail(e.what());
  }
  if (ctx.event_listener_manager) ctx.event_listener_manager->SignalEvent<Events::AfterOpKernelRun>({info_});
  return s;
}

// ---- op kernels with a workspace ---------------------------------------------------------------------
std::string OpKernelWithWorkspace::GetOpUID() const { return OpAccessor(info_).GetUID(); }
IAllocator *OpKernelWithWorkspace::GetAllocator() const {
  OpAccessor acc(info_);
  return info_.GetAllocator(acc.GetArgSpace(acc.GetNumArgs() - 1));  // the last operand's memory space
}
common::Status OpKernelWithWorkspace::ProloguePerFrame(const ExecutionContext &ctx) {
  const size_t bytes = GetWorkspaceSize(ctx);
  return ctx.frame_state_info.CreateStateIfNotExist(GetOpUID(), ctx.exec_frame, [&]() -> void * {
    if (bytes == 0) return nullptr;
    IAllocator *a = GetAllocator();
    BRT_ENFORCE(a != nullptr, "no allocator for the workspace of " + GetOpUID());
    return a->Alloc(bytes);
  });
}
common::Status OpKernelWithWorkspace::EpiloguePerFrame(const ExecutionContext &ctx) {
  if (!ctx.frame_state_info.HasState(GetOpUID())) return common::Status::OK();
  if (void *p = ctx.exec_frame->GetAndResetState(ctx.frame_state_info.GetStateOffset(GetOpUID())))
    if (IAllocator *a = GetAllocator()) a->Free(p);
  return common::Status::OK();
}
void *OpKernelWithWorkspace::GetWorkspace(const ExecutionContext &ctx) const {
  if (!ctx.frame_state_info.HasState(GetOpUID())) return nullptr;
  return ctx.exec_frame->GetState(ctx.frame_state_info.GetStateOffset(GetOpUID()));
}

// ---- frame ------------------------------------------------------------------------------------------
void *ExecutionFrame::GetAsyncValue(int value_id) const {
  const ir::Value &v = ir_->values[value_id];
  if (v.alias_of >= 0) {  // offset counts elements of the aliased value's type (op_helper.cc:44-52)
    char *base = static_cast<char *>(GetAsyncValue(v.alias_of));
    return base + v.alias_offset * (int64_t)GetDTypeByte(ir_->values[v.alias_of].type.dtype);
  }
  return base_[value_id];
}
void ExecutionFrame::SetState(size_t offset, void *p) {
  if (offset >= state_.size()) state_.resize(offset + 1, nullptr);
  state_[offset] = p;
}
void *ExecutionFrame::GetAndResetState(size_t offset) {
  void *p = GetState(offset);
  if (offset < state_.size()) state_[offset] = nullptr;
  return p;
}
bool ExecutionFrame::StateInfo::HasState(const std::string &key) {
  std::lock_guard<std::mutex> lock(mutex_);
  return name_to_offset_.count(key) != 0;
}
size_t ExecutionFrame::StateInfo::GetStateOffset(const std::string &key) {
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = name_to_offset_.find(key);
  BRT_ENFORCE(it != name_to_offset_.end(), "no frame state named " + key);
  return it->second;
}
common::Status ExecutionFrame::StateInfo::CreateStateIfNotExist(const std::string &key, ExecutionFrame *frame,
                                                                const std::function<void *()> &make) {
  size_t offset;
  {
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = name_to_offset_.find(key);
    if (it == name_to_offset_.end()) it = name_to_offset_.emplace(key, name_to_offset_.size()).first;
    offset = it->second;
  }
  // every frame fills its own slot, also when another frame created the offset
  if (frame->GetState(offset) == nullptr) frame->SetState(offset, make());
  return common::Status::OK();
}

void ExecutionFrame::StateInfo::Clear() {
  std::lock_guard<std::mutex> lock(mutex_);
  name_to_offset_.clear();
}

// ---- session ------------------------------------------------------------------------------------------
Session::Session() = default;
Session::~Session() { EndPlan(); }

// The per-session epilogue belongs to the kernels whose per-session prologue has run (a kernel
// that was constructed but never prepared, because an earlier one failed, is only destroyed).
void Session::EndPlan() noexcept {
  for (size_t i = 0; i < kernels_.size(); ++i) {
    const bool prepared = !kernels_[i]->HasProloguePerSession() || (i < session_prologue_done_.size() && session_prologue_done_[i]);
    if (prepared && kernels_[i]->HasEpiloguePerSession()) { try { kernels_[i]->EpiloguePerSession(); } catch (...) {} }
  }
  kernels_.clear();
  session_prologue_done_.clear();
}

common::Status Session::AddExecutionProvider(std::unique_ptr<ExecutionProvider> provider) {
  providers_.push_back(std::move(provider));
  return common::Status::OK();
}
common::Status Session::AddAllocator(std::unique_ptr<IAllocator> allocator) {
  const std::string key = allocator->Key();
  allocators_[key] = std::move(allocator);
  return common::Status::OK();
}
IAllocator *Session::GetAllocator(const std::string &key) {
  auto it = allocators_.find(key);
  return it == allocators_.end() ? nullptr : it->second.get();
}

common::Status Session::Load(const std::string &url, const std::string &fmt) {
  if (fmt != "byre") return common::Status::Fail("unsupported IR format " + fmt);
  ir_.reset(new ir::ByREHandle);
  common::Status s = ir_->LoadFromFile(url);
  if (!s.IsOK()) return s;
  return BuildPlan();
}
common::Status Session::LoadFromMemory(const std::string &text, const std::string &fmt) {
  if (fmt != "byre") return common::Status::Fail("unsupported IR format " + fmt);
  ir_.reset(new ir::ByREHandle);
  common::Status s = ir_->LoadFromText(text);
  if (!s.IsOK()) return s;
  return BuildPlan();
}

// Binds every op to the first provider that has a kernel under the op's key and constructs the
// kernels (shape checks and dlopen happen here), as StaticBRTExecutionPlan::ProloguePerSession
// does (execution_plan.cc:314-438).
common::Status Session::BuildPlan() {
  EndPlan();  // a model loaded earlier ends here
  frame_state_info_.Clear();  // its per-frame state keys and offsets do not carry over
  infos_.clear();
  in_offsets_.clear(); out_offsets_.clear(); weight_offsets_.clear();
  for (size_t i = 0; i < ir_->args.size(); ++i) {
    const int t = ir_->args[i].argtype;
    if (t & ir::kInput) in_offsets_.push_back(i);
    if (t & ir::kOutput) out_offsets_.push_back(i);
    if (t & ir::kWeight) weight_offsets_.push_back(i);
  }
  for (const ir::Value &v : ir_->values) {
    if ((v.arg_index >= 0 || v.is_alloc) && !allocators_.count(v.type.space))
      return common::Status::Fail("no allocator for memory space \"" + v.type.space + "\" (value " + v.name + ")");
  }
  // Static memory plan (execution_plan.cc:473-578): walking the ops in order, every
  // memref.alloc intermediate gets, at its first use, the next kAllocAlignment-rounded offset
  // in the arena of its memory space; aliases resolve through their source.  No reuse of
  // dead ranges, as in the reference.
  intermediate_offset_.assign(ir_->values.size(), SIZE_MAX);
  arena_bytes_.clear();
  for (const ir::Op &op : ir_->ops) {
    for (int operand : op.operands) {
      int v = operand;
      while (ir_->values[(size_t)v].alias_of >= 0) v = ir_->values[(size_t)v].alias_of;
      const ir::Value &val = ir_->values[(size_t)v];
      if (!val.is_alloc || intermediate_offset_[(size_t)v] != SIZE_MAX) continue;
      size_t &total = arena_bytes_[val.type.space];
      intermediate_offset_[(size_t)v] = total;
      total += (val.type.Bytes() + kAllocAlignment - 1) / kAllocAlignment * kAllocAlignment;
    }
  }
  // Op dependencies (execution_plan.cc:243-308): an op depends on the last writer of every
  // operand it reads.  memory_effects names read (1), write (2) or both per operand; without
  // it every operand counts as read and written; a copy reads operand 0 and writes operand 1.
  std::vector<std::vector<int>> dependency(ir_->ops.size());
  {
    std::unordered_map<int, int> last_writer;  // value id -> op id
    for (size_t i = 0; i < ir_->ops.size(); ++i) {
      const ir::Op &op = ir_->ops[i];
      auto fx = op.attrs.find("memory_effects");
      const bool is_copy = op.name == "byre.copy";
      for (size_t k = 0; k < op.operands.size(); ++k) {
        int effect = 3;
        if (is_copy) effect = k == 0 ? 1 : 2;
        else if (fx != op.attrs.end() && fx->second.elems.size() == op.operands.size()) effect = (int)fx->second.elems[k].i;
        const int v = op.operands[k];
        if (effect & 1) {
          auto w = last_writer.find(v);
          if (w != last_writer.end()) dependency[i].push_back(w->second);
        }
        if (effect & 2) last_writer[v] = (int)i;
      }
    }
  }
  for (size_t i = 0; i < ir_->ops.size(); ++i) {
    const std::string &key = ir_->ops[i].key;
    ExecutionProvider *chosen = nullptr;
    for (auto &p : providers_)
      if (p->GetKernelRegistry()->HasKernel(key)) { chosen = p.get(); break; }
    if (!chosen) return common::Status::Fail("No providers support Op " + key);
    infos_.emplace_back(new OpKernelInfo(*chosen, *ir_, (int)i, allocators_, dependency[i]));
    try {
      std::shared_ptr<OpKernel> k = (*chosen->GetKernelRegistry())(key, *infos_.back());
      if (!k) return common::Status::Fail("kernel factory returned null for " + key);
      kernels_.push_back(std::move(k));
    } catch (const std::exception &e) {
      return common::Status::Fail("constructing " + key + " (line " + std::to_string(ir_->ops[i].line) + "): " + e.what());
    }
  }
  // one-time preparation of the kernels that ask for it (the reference calls this from
  // Session::Load through ExecutionPlan::ProloguePerSession, execution_plan.cc:313-330)
  session_prologue_done_.assign(kernels_.size(), false);
  for (size_t i = 0; i < kernels_.size(); ++i) {
    if (!kernels_[i]->HasProloguePerSession()) continue;
    common::Status s = kernels_[i]->ProloguePerSession();
    if (!s.IsOK()) return s;
    session_prologue_done_[i] = true;
  }
  return common::Status::OK();
}

common::Status Session::NewRequestContext(std::unique_ptr<RequestContext> *request, WorkQueue *work_queue) {
  if (!ir_) return common::Status::Fail("no model loaded");
  std::unique_ptr<RequestContext> r(new RequestContext(*this));
  if (work_queue) {
    r->wq_.reset(work_queue);
  } else {
    if (!wq_factory_) return common::Status::Fail("no work queue given and no default work-queue factory set");
    r->wq_.reset(wq_factory_());
  }
  r->frame_.reset(new ExecutionFrame);
  ExecutionFrame &f = *r->frame_;
  f.ir_ = ir_.get();
  f.base_.assign(ir_->values.size(), nullptr);
  f.owned_.assign(ir_->values.size(), false);
  f.state_.clear();
  *request = std::move(r);
  return common::Status::OK();
}

void RequestContext::AddOpRunListener(OpRunListener l) {
  auto shared = std::make_shared<OpRunListener>(std::move(l));
  events_.AddEventListener<Events::BeforeOpKernelRun>([shared](const Events::BeforeOpKernelRun &e) { (*shared)(OpRunEvent{&e.info, false}); });
  events_.AddEventListener<Events::AfterOpKernelRun>([shared](const Events::AfterOpKernelRun &e) { (*shared)(OpRunEvent{&e.info, true}); });
}

size_t Session::GetArgNum() const { return ir_ ? ir_->args.size() : 0; }
int Session::GetGraphArgOffset(const std::string &name) const {
  for (size_t i = 0; i < ir_->args.size(); ++i)
    if (ir_->args[i].argname == name) return (int)i;
  return -1;
}
std::string Session::GetArgName(size_t offset) const { return ir_->args.at(offset).argname; }
Shape Session::GetStaticShape(size_t offset) const { return ir_->values[ir_->args.at(offset).value].type.shape; }
DTypeEnum Session::GetDType(size_t offset) const { return ir_->values[ir_->args.at(offset).value].type.dtype; }
std::string Session::GetSpace(size_t offset) const { return ir_->values[ir_->args.at(offset).value].type.space; }

common::Status Session::Run(RequestContext &request) {
  ExecutionFrame &f = *request.frame_;
  if (!f.io_bound_) return common::Status::Fail("FinishIOBinding has not been called");
  ExecutionContext ctx(&f, request.wq_.get(), frame_state_info_, &request.events_);
  if (!f.prologue_done_) {  // first run of this frame: workspaces (op_kernel_impl_base.h:116-136)
    // A prologue that fails part-way (a status, or an exception from an allocator) leaves the
    // kernels before it prepared: prologue_count_ records how far it got, so that Cleanup
    // releases exactly their workspaces, and the next Run starts over from the first kernel
    // after releasing them.
    if (f.prologue_count_ > 0) {
      for (size_t i = 0; i < f.prologue_count_ && i < kernels_.size(); ++i)
        if (kernels_[i]->HasEpiloguePerFrame()) { try { kernels_[i]->EpiloguePerFrame(ctx); } catch (...) {} }
      f.prologue_count_ = 0;
    }
    for (size_t i = 0; i < kernels_.size(); ++i) {
      if (kernels_[i]->HasProloguePerFrame()) {
        common::Status s;
        try {
          s = kernels_[i]->ProloguePerFrame(ctx);
        } catch (const std::exception &e) {
          s = common::Status::Fail(std::string("ProloguePerFrame: ") + e.what());
        }
        if (!s.IsOK()) return s;
      }
      f.prologue_count_ = i + 1;
    }
    f.prologue_done_ = true;
  }
  request.events_.SignalEvent<Events::BeforeExecutionPlanRun>({});
  for (auto &k : kernels_) {
    common::Status s = k->Run(ctx);
    if (!s.IsOK()) return s;
  }
  request.events_.SignalEvent<Events::AfterExecutionPlanRun>({});
  return common::Status::OK();
}

void Session::Cleanup(RequestContext &request) noexcept {
  ExecutionFrame &f = *request.frame_;
  ExecutionContext ctx(&f, request.wq_.get(), frame_state_info_, nullptr);
  if (request.wq_) request.wq_->Sync();
  for (size_t i = 0; i < f.prologue_count_ && i < kernels_.size(); ++i) {  // also after a prologue that failed part-way
    if (!kernels_[i]->HasEpiloguePerFrame()) continue;
    try { kernels_[i]->EpiloguePerFrame(ctx); } catch (...) {}
  }
  f.prologue_count_ = 0;
  f.prologue_done_ = false;
  for (size_t i = 0; i < f.base_.size(); ++i) {
    if (f.owned_[i] && f.base_[i]) {
      if (IAllocator *a = GetAllocator(ir_->values[i].type.space)) a->Free(f.base_[i]);
      f.base_[i] = nullptr;
      f.owned_[i] = false;
    }
  }
  for (auto &arena : f.arenas_) {
    if (IAllocator *a = GetAllocator(arena.first)) a->Free(arena.second);
  }
  f.arenas_.clear();
}

// ---- request context --------------------------------------------------------------------------------------
RequestContext::~RequestContext() { session_.Cleanup(*this); }

common::Status RequestContext::BindArg(size_t offset, const void *value, BrtOwnershipType own) {
  const ir::ByREHandle &ir = *session_.ir_;
  if (offset >= ir.args.size()) return common::Status::Fail("argument offset out of range");
  const int v = ir.args[offset].value;
  if (frame_->owned_[v] && frame_->base_[v]) {
    if (IAllocator *a = session_.GetAllocator(ir.values[v].type.space)) a->Free(frame_->base_[v]);
  }
  frame_->base_[v] = const_cast<void *>(value);
  frame_->owned_[v] = own == BrtOwnershipType::OwnedByRuntime;
  return common::Status::OK();
}

// entry arguments the caller has not bound and memref.alloc intermediates are allocated here
// from the allocator named by the memref's memory space (execution_frame.cc:160-184)
void RequestContext::FinishIOBinding() {
  const ir::ByREHandle &ir = *session_.ir_;
  // intermediates: one arena per memory space, laid out by the session's static plan
  // (BRTInferenceExecutionFrame, execution_frame.cc:60-120)
  if (frame_->arenas_.empty()) {
    for (const auto &kv : session_.arena_bytes_) {
      if (kv.second == 0) continue;
      IAllocator *a = session_.GetAllocator(kv.first);
      BRT_ENFORCE(a != nullptr, "no allocator for space " + kv.first);
      void *block = a->Alloc(kv.second);
      BRT_ENFORCE(block != nullptr, "allocation of the intermediate arena failed");
      frame_->arenas_.emplace_back(kv.first, block);
    }
    for (size_t i = 0; i < ir.values.size(); ++i) {
      const size_t off = session_.intermediate_offset_[i];
      if (off == SIZE_MAX) continue;
      for (const auto &arena : frame_->arenas_)
        if (arena.first == ir.values[i].type.space) frame_->base_[i] = static_cast<char *>(arena.second) + off;
    }
  }
  for (size_t i = 0; i < ir.values.size(); ++i) {
    const ir::Value &v = ir.values[i];
    if (frame_->base_[i] || v.alias_of >= 0) continue;
    if (v.arg_index < 0) continue;  // an intermediate no op uses needs no memory
    IAllocator *a = session_.GetAllocator(v.type.space);
    BRT_ENFORCE(a != nullptr, "no allocator for space " + v.type.space);
    const size_t bytes = (v.type.Bytes() + kAllocAlignment - 1) / kAllocAlignment * kAllocAlignment;
    frame_->base_[i] = a->Alloc(bytes ? bytes : kAllocAlignment);
    frame_->owned_[i] = true;
  }
  frame_->io_bound_ = true;
}

void *RequestContext::GetArg(size_t offset) {
  const ir::ByREHandle &ir = *session_.ir_;
  BRT_ENFORCE(offset < ir.args.size(), "argument offset out of range");
  const int v = ir.args[offset].value;
  if (!frame_->base_[v]) {  // the reference's tests fetch arguments before binding is finished
    IAllocator *a = session_.GetAllocator(ir.values[v].type.space);
    BRT_ENFORCE(a != nullptr, "no allocator for space " + ir.values[v].type.space);
    const size_t bytes = (ir.values[v].type.Bytes() + kAllocAlignment - 1) / kAllocAlignment * kAllocAlignment;
    frame_->base_[v] = a->Alloc(bytes ? bytes : kAllocAlignment);
    frame_->owned_[v] = true;
  }
  return frame_->base_[v];
}

common::Status RequestContext::Sync() { return wq_ ? wq_->Sync() : common::Status::OK(); }

}  // namespace brt
