"""Source of an op-kernel library written the way the reference's external kernels are
(runtime/test/external_kernels/cuda/kernels.cc:37-99): the five-argument OpKernel constructor
with the hook flags, ProloguePerSession / ProloguePerFrame overrides, OpAccessor on the frame of
the execution context, a per-frame state through frame_state_info, events through the
context's listener manager, static registration from a lambda.  What the CUDA original does
with AddTask and a __global__ function is a device-to-device copy through the kernel library's
C ABI here (the op computes out = in)."""

SRC = r"""
#include <atomic>
#include "brt.h"
#include "brt_rocm_kernels.h"

using namespace brt;
using namespace brt::common;

extern "C" {
std::atomic<int> g_prologue_per_session{0}, g_prologue_per_frame{0}, g_epilogue_per_frame{0}, g_runs{0};
int ext_prologue_per_session() { return g_prologue_per_session.load(); }
int ext_prologue_per_frame() { return g_prologue_per_frame.load(); }
int ext_epilogue_per_frame() { return g_epilogue_per_frame.load(); }
int ext_runs() { return g_runs.load(); }
}

namespace {
template <typename T> class CustomCopy final : public OpKernel {
public:
  explicit CustomCopy(const OpKernelInfo &info) : OpKernel(info, true, false, true, true) {}

  common::Status RunImpl(const ExecutionContext &ctx) override {
    OpAccessor accessor(info_, ctx.exec_frame);
    Shape shape = accessor.GetArgShape(0);
    int64_t n = accessor.GetNumElementsOfShape(shape);
    // the state this kernel created for the frame: a run counter
    size_t offset = ctx.frame_state_info.GetStateOffset(accessor.GetUID());
    ++*static_cast<int *>(ctx.exec_frame->GetState(offset));
    ++g_runs;
    void *stream = ctx.work_queue->GetComputeStream();
    int e = brt_rocm_memcpy_d2d(accessor.GetArgAsyncValueRef(1), accessor.GetArgAsyncValueRef(0), (size_t)n * sizeof(T), stream);
    return e == 0 ? Status::OK() : Status::Fail(brt_rocm_error_string(e));
  }

  common::Status ProloguePerSession() override {
    ++g_prologue_per_session;
    return Status::OK();
  }

  common::Status ProloguePerFrame(const ExecutionContext &ctx) override {
    ++g_prologue_per_frame;
    OpAccessor accessor(info_);
    return ctx.frame_state_info.CreateStateIfNotExist(accessor.GetUID(), ctx.exec_frame, []() -> void * { return new int(0); });
  }

  common::Status EpiloguePerFrame(const ExecutionContext &ctx) override {
    ++g_epilogue_per_frame;
    OpAccessor accessor(info_);
    delete static_cast<int *>(ctx.exec_frame->GetAndResetState(ctx.frame_state_info.GetStateOffset(accessor.GetUID())));
    return Status::OK();
  }
};

BRT_STATIC_KERNEL_REGISTRATION(
    DeviceKind::ROCM, ProviderType::BRT, [](KernelRegistry *registry) {
      registry->Register(
          "CustomCopyOp",
          [](const brt::OpKernelInfo &info) -> std::shared_ptr<OpKernel> {
            auto kernel = std::shared_ptr<OpKernel>(new CustomCopy<float>(info));
            return kernel;
          });
    });
}  // namespace
"""


def build(tmp_path, root):
    """Compiles SRC into tmp_path/libcustom_copy.so against brt.h and the two in-tree libraries."""
    import os
    import subprocess
    src = tmp_path / "custom_copy.cc"
    src.write_text(SRC)
    lib = tmp_path / "libcustom_copy.so"
    libdir = os.path.join(root, "byteir_amd", "lib")
    subprocess.run(["g++", "-std=c++17", "-O1", "-shared", "-fPIC", f"-I{os.path.join(root, 'byteir_amd', 'csrc', 'brt')}",
                    f"-I{os.path.join(root, 'include')}", str(src), "-o", str(lib), f"-L{libdir}", "-lbrt", "-lbrt_rocm_kernels",
                    f"-Wl,-rpath,{libdir}"], check=True)
    return lib
