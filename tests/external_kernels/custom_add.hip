// An op-kernel library written the way the reference's external CUDA kernels are
// (runtime/test/external_kernels/cuda/kernels.cc:37-99 and kernels.cu): the reference's include
// lines, the five-argument OpKernel constructor with the hook flags, OpAccessor on the frame of
// the execution context, a __global__ function handed to WorkQueue::AddTask with
// {grid, block, dynamic shared bytes, kernel arguments...}, the op's id and its dependencies,
// and static registration from a lambda.  What differs from a source for the CUDA provider: the
// device function is HIP (this file is compiled by hipcc), the launch shape comes from
// MakeROCMGridAndBlock, and the registration names DeviceKind::ROCM.
#include <hip/hip_runtime.h>

#include <atomic>
#include <vector>

#include "brt/backends/common.h"
#include "brt/backends/rocm/device/common/util.h"
#include "brt/core/common/common.h"
#include "brt/core/common/status.h"
#include "brt/core/context/execution_context.h"
#include "brt/core/context/execution_frame.h"
#include "brt/core/context/work_queue.h"
#include "brt/core/framework/kernel_registry.h"
#include "brt/core/framework/op_accessor.h"
#include "brt/core/framework/op_kernel.h"

using namespace brt;
using namespace brt::rocm;
using namespace brt::common;
using namespace brt::ir;

namespace external_kernels {
template <typename T> __global__ void add_kernel(const T *a, const T *b, T *c, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) c[i] = a[i] + b[i];
}
}  // namespace external_kernels

extern "C" {
std::atomic<int> g_add_prologue_per_session{0}, g_add_prologue_per_frame{0}, g_add_host_tasks{0};
int ext_add_prologue_per_session() { return g_add_prologue_per_session.load(); }
int ext_add_prologue_per_frame() { return g_add_prologue_per_frame.load(); }
int ext_add_host_tasks() { return g_add_host_tasks.load(); }
int g_add_last_dependency_count = -1, g_add_last_op_id = -1;
int ext_add_last_dependency_count() { return g_add_last_dependency_count; }
int ext_add_last_op_id() { return g_add_last_op_id; }
}

namespace {
template <typename T> class CustomAdd final : public OpKernel {
public:
  explicit CustomAdd(const OpKernelInfo &info) : OpKernel(info, true, false, true, false) {}

  common::Status RunImpl(const ExecutionContext &) override;

  common::Status ProloguePerSession() override;

  common::Status ProloguePerFrame(const ExecutionContext &) override;
};

template <typename T> common::Status CustomAdd<T>::RunImpl(const ExecutionContext &ctx) {
  OpAccessor accessor(info_, ctx.exec_frame);
  Shape shape = accessor.GetArgShape(0);
  long long n = accessor.GetNumElementsOfShape(shape);

  auto p = MakeROCMGridAndBlock(n);
  size_t dyn_shared_size = 0;

  std::vector<void *> args;
  args.push_back(&p.first);          // grid
  args.push_back(&p.second);         // block
  args.push_back(&dyn_shared_size);  // dyn_shared_size

  auto num_arg = accessor.GetNumArgs();
  std::vector<AsyncValueRef> ptrs(num_arg);
  for (unsigned int i = 0; i < num_arg; ++i) {
    ptrs[i] = accessor.GetArgAsyncValueRef(i);
    args.push_back(&ptrs[i]);
  }

  args.push_back(&n);  // n

  g_add_last_op_id = info_.GetOpId();
  g_add_last_dependency_count = (int)info_.GetDependency().size();
  common::Status s = ctx.work_queue->AddTask(0, (void *)external_kernels::add_kernel<T>, args.data(), info_.GetOpId(),
                                             info_.GetDependency());
  if (!s.IsOK()) return s;
  // a host task in queue order, through the reference's macro
  WorkQueue *wq = ctx.work_queue;
  DispatchHostTask(wq, info_.GetOpId(), info_.GetDependency(), { ++g_add_host_tasks; });
  return Status::OK();
}

template <typename T> common::Status CustomAdd<T>::ProloguePerSession() {
  ++g_add_prologue_per_session;
  return Status::OK();
}

template <typename T> common::Status CustomAdd<T>::ProloguePerFrame(const ExecutionContext &) {
  ++g_add_prologue_per_frame;
  return Status::OK();
}

// statically register the op kernels of this library
BRT_STATIC_KERNEL_REGISTRATION(DeviceKind::ROCM, ProviderType::BRT, [](KernelRegistry *registry) {
  registry->Register("CustomAddOp", [](const brt::OpKernelInfo &info) -> std::shared_ptr<OpKernel> {
    auto kernel = std::shared_ptr<OpKernel>(new CustomAdd<float>(info));
    return kernel;
  });
});
}  // namespace
