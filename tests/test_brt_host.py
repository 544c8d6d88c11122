"""Host logic of the BRT-shaped runtime, on a plan-only session (no GPU): the ByRE text reader,
the kernel registry, plan-time checks of the op kernels, the extra_args blob, and the export
lists of the three C ABI libraries."""
import os
import re
import struct

import pytest

from byre_text import memref, reduction_module, softmax_module

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture()
def session():
    from byteir_amd import brt
    s = brt.Session(device_id=-1)
    yield s
    s.close()


def exported_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"typedef[^;]*;", "", text)
    names = re.findall(r"\b([a-z][a-zA-Z0-9_]*)\s*\([^;{]*\)\s*;", text)
    return sorted(set(n for n in names if not n.endswith("_fn") and n != "brt_op_listener"))


@pytest.mark.parametrize("header,loader", [("brt_rocm_kernels.h", "kernels"), ("brt_rocm_bench.h", "kernels"), ("flash_api.h", "flash_attn"), ("brt_c_api.h", "brt")])
def test_c_abi_exports_every_declared_symbol(header, loader):
    from byteir_amd import _lib
    L = getattr(_lib, loader)()
    names = exported_functions(header)
    assert len(names) >= 4
    for n in names:
        assert hasattr(L, n), f"{header}: {n} is not exported"
    if header == "flash_api.h":
        import ctypes
        ver = ctypes.c_char_p.in_dll(L, "VERSION")  # a pointer variable, as in the reference
        assert ver.value == b"2.5.3"


def test_reference_flash_attn_modules_load_unchanged(session, golden_dir):
    # runtime/test/test_files/flash_attn_fwd.mlir, byte for byte
    session.load(os.path.join(golden_dir, "flash_attn_fwd.mlir"))
    assert session.get_arg_num() == 7
    assert session.get_op_keys() == ["custom"]
    assert [session.get_arg_name(i) for i in range(7)] == ["Q", "K", "V", "Out", "SoftmaxLse", "SoftmaxPtr", "RngState"]
    assert session.get_static_shape(0) == [1, 128, 3, 32] and session.get_data_type(0) == "float16"
    assert session.get_static_shape(4) == [1, 3, 128] and session.get_data_type(4) == "float32"
    assert session.get_static_shape(6) == [2] and session.get_data_type(6) == "int64"
    assert session.get_space(0) == "cuda"
    assert session.get_output_arg_offsets() == list(range(7))  # every arg carries byre.argtype = 2
    # the blob handed to the library: 17 i64, f32, 4 i64, f32, 2 i64, unpadded
    fields = [12288] * 4 + [96] * 4 + [32] * 4 + [1, 3, 3, 32, 32, 0.5, 128, 128, 128, 128, 0.0, -1, 0]
    want = b"".join(struct.pack("<f", f) if isinstance(f, float) else struct.pack("<q", f) for f in fields)
    assert session.get_op_attr_blob(0, "extra_args") == want
    session.load(os.path.join(golden_dir, "flash_attn_bwd.mlir"))
    assert session.get_op_keys() == ["custom", "custom"] and session.get_arg_num() == 13
    assert session.get_graph_arg_offset("d_Q") == 6 and session.get_graph_arg_offset("nope") == -1


def test_reader_accepts_the_compiler_s_attribute_forms(session):
    # dense<[..]>, splat dense<1> : tensor<1xi64>, unsorted dims, ArrayAttr, rank-0 memref,
    # memref.alloc and byre.alias (runtime/test/test_files/resnet18_fw_bw_host_cuda.mlir:59,178,185,300)
    text = """
module attributes {byre.container_module} {
  func.func @main(%arg0: memref<4x1000xf32, "cuda"> {byre.argname = "in", byre.argtype = 1 : i32},
                  %arg1: memref<f32, "cuda"> {byre.argname = "out0", byre.argtype = 2 : i32},
                  %arg2: memref<4xf32, "cuda"> {byre.argname = "out1", byre.argtype = 2 : i32},
                  %arg3: memref<2x3x8x5xf32, "cuda"> {byre.argname = "in2", byre.argtype = 1 : i32},
                  %arg4: memref<2x3xf32, "cuda"> {byre.argname = "out2", byre.argtype = 2 : i32}) attributes {byre.entry_point, device_file_name = "x.ptx"} {
    // intermediates
    %alloc = memref.alloc() : memref<1024xi8, "cuda">
    %0 = "byre.alias"(%alloc) {device = "cuda", offset = 256 : i64} : (memref<1024xi8, "cuda">) -> memref<4xf32, "cuda">
    byre.compute @ReduceSumOp_f32_f32(%arg0, %arg1) {device = "cuda", dimensions = dense<[0, 1]> : tensor<2xi64>, memory_effects = [1 : i32, 2 : i32]} : memref<4x1000xf32, "cuda">, memref<f32, "cuda">
    byre.compute @ReduceMaxOp_f32_f32(%arg0, %0) {dimensions = dense<1> : tensor<1xi64>} : memref<4x1000xf32, "cuda">, memref<4xf32, "cuda">
    byre.compute @ReduceSumOp_f32_f32(%arg0, %arg2) {dimensions = [1 : i64]} : memref<4x1000xf32, "cuda">, memref<4xf32, "cuda">
    byre.compute @ReduceSumOp_f32_f32(%arg3, %arg4) {dimensions = dense<[3, 2]> : tensor<2xi64>} : memref<2x3x8x5xf32, "cuda">, memref<2x3xf32, "cuda">
    return
  }
}
"""
    session.load_from_memory(text)
    assert session.get_op_keys() == ["ReduceSumOp_f32_f32", "ReduceMaxOp_f32_f32", "ReduceSumOp_f32_f32", "ReduceSumOp_f32_f32"]
    assert session.get_static_shape(1) == [] and session.get_input_arg_offsets() == [0, 3]
    req = session.new_request_context()
    req.finish_io_binding()  # allocates args and the memref.alloc intermediate (host memory here)
    assert req.get_arg(0) != 0
    with pytest.raises(RuntimeError, match="without a device"):
        req.run()


def test_registry_has_the_reference_keys(session):
    for key in ("ReduceSumOp_f32_f32", "ReduceSumOp_f16_f16", "ReduceMaxOp_f32_f32", "ReduceMaxOp_f16_f16",
                "custom", "byteir.softmax", "cpu2cuda", "cuda2cpu", "cuda2cuda"):
        assert session.has_kernel(key), key
    assert not session.has_kernel("MatmulOp_f32f32_f32")


def test_unknown_op_fails_at_load(session):
    # execution_plan.cc:435-438: "No providers support Op <key>"
    text = reduction_module("cuda", [4, 8], [1], "ReduceArgMaxOp_f32_f32")
    with pytest.raises(RuntimeError, match="No providers support Op ReduceArgMaxOp_f32_f32"):
        session.load_from_memory(text)


def test_unknown_memory_space_fails_at_load(session):
    with pytest.raises(RuntimeError, match="no allocator for memory space"):
        session.load_from_memory(reduction_module("tpu", [4, 8], [1], "ReduceSumOp_f32_f32"))


def test_reduce_plan_time_checks(session):
    # non-consecutive dims (reduce_impl.h:41-42)
    with pytest.raises(RuntimeError, match="consecutive"):
        session.load_from_memory(reduction_module("cuda", [2, 16, 32], [0, 2], "ReduceSumOp_f32_f32"))
    # {0, 2} over [1, 16, 32] is fine: size-1 dims are dropped first
    session.load_from_memory(reduction_module("cuda", [1, 16, 32], [0, 2], "ReduceSumOp_f32_f32"))
    # keep-dims output shape is rejected (reduce_impl.h:35)
    tin, tout = memref([4, 8], "f32", "cuda"), memref([4, 1], "f32", "cuda")
    bad = f"""func.func @t(%a : {tin}, %b : {tout}) attributes {{byre.entry_point}} {{
      byre.compute @ReduceSumOp_f32_f32(%a, %b) {{dimensions = dense<[1]> : tensor<1xi64>}} : {tin}, {tout}
      return }}"""
    with pytest.raises(RuntimeError, match="output shape"):
        session.load_from_memory(bad)
    # out-of-range dimension
    with pytest.raises(RuntimeError, match="invalid dimension"):
        session.load_from_memory(bad.replace("dense<[1]>", "dense<[2]>").replace("4x1xf32", "4x8xf32"))
    # element type must match the key
    with pytest.raises(RuntimeError, match="element type"):
        session.load_from_memory(reduction_module("cuda", [4, 8], [1], "ReduceSumOp_f16_f16", dtype="f32"))
    # missing attribute
    with pytest.raises(RuntimeError, match="dimensions is not set"):
        session.load_from_memory(reduction_module("cuda", [4, 8], [1], "ReduceSumOp_f32_f32").replace("dimensions = dense<[1]> : tensor<1xi64>, ", ""))


def test_softmax_plan_time_checks(session):
    session.load_from_memory(softmax_module("cuda", [10, 128], "bf16", 1))
    session.load_from_memory(softmax_module("cuda", [8, 12, 256, 256], "f32", -1))
    session.load_from_memory(softmax_module("cuda", [10, 128], "f32", 0))
    with pytest.raises(RuntimeError, match="axis out of range"):
        session.load_from_memory(softmax_module("cuda", [10, 128], "f32", 2))
    with pytest.raises(RuntimeError, match="f32, f16 or bf16"):
        session.load_from_memory(softmax_module("cuda", [10, 128], "i32", 1))


def test_custom_op_load_errors(session, golden_dir):
    text = open(os.path.join(golden_dir, "flash_attn_fwd.mlir")).read()
    with pytest.raises(RuntimeError, match="load failed"):
        session.load_from_memory(text.replace("libflash_attn.so", "libdoes_not_exist.so"))
    with pytest.raises(RuntimeError, match="Couldn't find function: run_flash_attn_nope"):
        session.load_from_memory(text.replace("run_flash_attn_fwd", "run_flash_attn_nope"))
    # a library without a VERSION symbol is refused (custom.cc:50-51)
    from byteir_amd import _lib
    with pytest.raises(RuntimeError, match="Version doesn't exist"):
        session.load_from_memory(text.replace("test/test_files/external_libs/libflash_attn.so", _lib.lib_path("libbrt_rocm_kernels.so"))
                                 .replace("run_flash_attn_fwd", "brt_rocm_softmax"))


def test_parse_errors_are_reported_with_a_line(session):
    with pytest.raises(RuntimeError, match="ByRE parse error: line 2"):
        session.load_from_memory('func.func @t(%a : memref<4xf32, "cuda">) attributes {byre.entry_point} {\n  byre.compute @X(%b) : memref<4xf32, "cuda">\n return }')
    with pytest.raises(RuntimeError, match="dynamic"):
        session.load_from_memory('func.func @t(%a : memref<?x4xf32, "cuda">) attributes {byre.entry_point} { return }')
    with pytest.raises(RuntimeError, match="entry_point"):
        session.load_from_memory('func.func @t(%a : memref<4xf32, "cuda">) { return }')


def test_python_side_canonicalisation_matches_oracle():
    import oracle
    from byteir_amd import ops
    for shape, dims in [((1, 16, 32), (0,)), ((2, 16, 8, 64), (1, 2)), ((4, 8, 3, 5), (3, 2)), ((1, 7, 1), (0, 2))]:
        out_shape = oracle.deduce_output_shape(shape, dims)
        st, A, B, C = oracle.reduce_canonicalize(shape, out_shape, dims)
        assert st == 0 and ops.canonicalize_reduce(list(shape), out_shape, list(dims)) == (A, B, C)
    with pytest.raises(ValueError):
        ops.canonicalize_reduce([2, 16, 32], [16], [0, 2])


def test_flash_blob_packer_matches_oracle():
    import numpy as np
    import torch
    import oracle
    from byteir_amd import ops
    q = torch.empty((4, 2048, 32, 128), dtype=torch.float16, device="meta")
    blob = ops.pack_flash_args(q, q, q, q, float(np.float32(1 / np.sqrt(128))), (-1, 0))
    a = oracle.fa_args(4, 2048, 2048, 32, 32, 128, 1 / np.sqrt(128), window=(-1, 0))
    assert blob == oracle.fa_pack_args(a).tobytes()


PLUGIN_SRC = r"""
// An op-kernel library outside the runtime: registers one kernel under the ROCm provider from a
// static initialiser, the way runtime/test/external_kernels/cuda/kernels.cc:91-99 does.
#include "brt.h"
namespace {
class Noop final : public brt::OpKernel {
public:
  explicit Noop(const brt::OpKernelInfo &info) : brt::OpKernel(info) {
    brt::OpAccessor acc(info);
    BRT_ENFORCE(acc.GetNumArgs() == 2, "test.external_noop takes two operands");
  }
  brt::common::Status RunImpl(const brt::ExecutionContext &) override { return brt::common::Status::OK(); }
};
void RegisterExternal(brt::KernelRegistry *r) {
  r->Register("test.external_noop", [](const brt::OpKernelInfo &info) -> std::shared_ptr<brt::OpKernel> {
    return std::make_shared<Noop>(info);
  });
}
}  // namespace
BRT_STATIC_KERNEL_REGISTRATION(brt::DeviceKind::ROCM, brt::ProviderType::BRT, RegisterExternal)
"""


def test_external_kernel_library_registers_statically(tmp_path):
    """ExecutionProvider::StaticRegisterKernelsFromDynlib (execution_provider.cc:29-41; used by
    runtime/test/unittest_main/test_main.cc:33-35): a library loaded before the session is created
    adds its kernels to the provider's registry; its constructor-time checks run at load."""
    import subprocess
    from byteir_amd import _lib, brt
    B = _lib.brt()
    src = tmp_path / "external_kernels.cc"
    src.write_text(PLUGIN_SRC)
    lib = tmp_path / "libexternal_kernels.so"
    libdir = os.path.join(ROOT, "byteir_amd", "lib")
    subprocess.run(["g++", "-std=c++17", "-O1", "-shared", "-fPIC", f"-I{os.path.join(ROOT, 'byteir_amd', 'csrc', 'brt')}",
                    str(src), "-o", str(lib), f"-L{libdir}", "-lbrt", f"-Wl,-rpath,{libdir}"], check=True)
    assert B.brt_register_kernels_from_dynlib(str(tmp_path / "missing.so").encode()) != 0
    assert B.brt_register_kernels_from_dynlib(str(lib).encode()) == 0, B.brt_last_error().decode()
    s = brt.Session(device_id=-1)
    try:
        assert s.has_kernel("test.external_noop")
        t = memref([4], "f32", "cuda")
        mod = f"""func.func @t(%a : {t} {{byre.argname = "a", byre.argtype = 1: i32}},
                     %b : {t} {{byre.argname = "b", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{
          byre.compute @test.external_noop(%a, %b) : {t}, {t}
          return }}"""
        s.load_from_memory(mod)
        assert s.get_op_keys() == ["test.external_noop"]
        with pytest.raises(RuntimeError, match="takes two operands"):
            s.load_from_memory(mod.replace("(%a, %b) : " + t + ", " + t, "(%a) : " + t))
    finally:
        s.close()


def test_reference_style_external_kernel_compiles_and_prepares(tmp_path):
    """An op kernel written against the reference's OpKernel surface -- five-argument
    constructor, ProloguePerSession, per-frame hooks using ExecutionContext::frame_state_info,
    registration from a lambda (runtime/test/external_kernels/cuda/kernels.cc:37-99) -- builds
    against brt.h; loading a module that uses it runs ProloguePerSession once per load."""
    import ctypes
    from byteir_amd import _lib, brt
    from external_kernel_src import build
    B = _lib.brt()
    lib = build(tmp_path, ROOT)
    assert B.brt_register_kernels_from_dynlib(str(lib).encode()) == 0, B.brt_last_error().decode()
    ext = ctypes.CDLL(str(lib))
    s = brt.Session(device_id=-1)
    try:
        assert s.has_kernel("CustomCopyOp")
        t, pinned = memref([64], "f32", "cuda"), memref([64], "f32", "cudaPinned")
        mod = f"""func.func @t(%a : {t} {{byre.argname = "a", byre.argtype = 1: i32}},
                     %b : {t} {{byre.argname = "b", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{
          byre.compute @CustomCopyOp(%a, %b) : {t}, {t}
          return }}"""
        before = ext.ext_prologue_per_session()
        s.load_from_memory(mod)
        assert ext.ext_prologue_per_session() == before + 1 and ext.ext_prologue_per_frame() == 0
        # a memref in page-locked host memory: the "cudaPinned" allocator key of the reference
        # (runtime/lib/backends/cuda/device/cuda_allocator.cc:104-108) is known to the session
        s.load_from_memory(mod.replace(f"%a : {t}", f"%a : {pinned}").replace(f"(%a, %b) : {t}", f"(%a, %b) : {pinned}"))
        assert s.get_space(0) == "cudaPinned"
        with pytest.raises(RuntimeError, match="no allocator for memory space"):
            s.load_from_memory(mod.replace('"cuda"', '"nowhere"'))
    finally:
        s.close()


def test_reference_kvcache_module_loads_unchanged(session, golden_dir):
    """flash_attn_kvcache.mlir of the reference: eight operands (one of them memref<2xi32>), the
    library is found by file name, the 244-byte blob is what the oracle packs."""
    import oracle
    session.load(os.path.join(golden_dir, "flash_attn_kvcache.mlir"))
    assert session.get_op_keys() == ["custom"]
    assert session.get_arg_num() == 8
    assert session.get_static_shape(5) == [2] and session.get_data_type(5) == "int32"
    assert session.get_static_shape(1) == [2, 128, 3, 32]
    blob = session.get_op_attr_blob(0, "extra_args")
    assert blob == oracle.fa_kvcache_pack_args(2, 1, 128, 3, 3, 32, 1, 0.5, (-1, -1)).tobytes()


def test_static_memory_plan_of_intermediates(session):
    """memref.alloc intermediates share one arena per memory space: offsets in order of first
    use, every tensor rounded up to 256 bytes, an alias adds nothing, an alloc no op uses gets
    no room (StaticBRTExecutionPlan, execution_plan.cc:473-578)."""
    text = """func.func @t(%h : memref<1000xf32, "cpu"> {byre.argname = "h", byre.argtype = 1: i32},
                      %o : memref<1000xf32, "cpu"> {byre.argname = "o", byre.argtype = 2: i32}) attributes {byre.entry_point} {
      %unused = memref.alloc() : memref<77xf32, "cuda">
      %d0 = memref.alloc() : memref<1000xf32, "cuda">
      %d1 = memref.alloc() : memref<4000xi8, "cuda">
      %v1 = "byre.alias"(%d1) {offset = 0 : i64} : (memref<4000xi8, "cuda">) -> memref<1000xf32, "cuda">
      %s0 = memref.alloc() : memref<3xf32, "cpu">
      byre.compute @cpu2cuda(%h, %d0) : memref<1000xf32, "cpu">, memref<1000xf32, "cuda">
      byre.compute @cuda2cuda(%d0, %v1) : memref<1000xf32, "cuda">, memref<1000xf32, "cuda">
      byre.compute @cuda2cpu(%v1, %o) : memref<1000xf32, "cuda">, memref<1000xf32, "cpu">
      return }"""
    session.load_from_memory(text)
    assert session.get_intermediate_bytes("cuda") == 4096 + 4096   # 4000 B -> 4096, twice
    assert session.get_intermediate_bytes("cpu") == 0              # %s0 is never used
    assert session.get_intermediate_bytes("nowhere") == 0


def test_product_code_never_touches_the_oracle():
    """The oracle is test infrastructure: nothing under the shipped package may import, load or
    name it, and the package has no CPU fallback to fall back on."""
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "byteir_amd")
    for dirpath, _, files in os.walk(root):
        for name in files:
            if name.endswith((".py", ".hip", ".cc", ".h", ".c", ".cpp")):
                text = open(os.path.join(dirpath, name), errors="replace").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, name)
                # the host execution of the kernels (tests/emu) is test infrastructure too: only the
                # build script may name it, nothing that runs may load it
                if name != "build.py":
                    assert "flash_attn_emu" not in text and "wave_emu" not in text, os.path.join(dirpath, name)


def test_missing_kernel_library_fails_loudly(tmp_path, monkeypatch):
    """Without its HIP library the package must raise, not compute something else."""
    import importlib
    from byteir_amd import _lib
    fresh = importlib.reload(_lib)
    try:
        monkeypatch.setattr(fresh, "LIB_DIR", str(tmp_path), raising=False)
        monkeypatch.setattr(fresh, "_kernels", None, raising=False)
        monkeypatch.setattr(fresh, "_flash", None, raising=False)
        with pytest.raises((OSError, RuntimeError)):
            fresh.flash_attn()
    finally:
        importlib.reload(_lib)


def test_op_dependencies_follow_the_memory_effects():
    """OpKernelInfo::GetDependency (framework/op_kernel_info.h:95) as the reference computes it
    (execution_plan.cc:243-308): an op depends on the last writer of each operand it reads;
    without memory_effects every operand counts as read and written.  Seen through a kernel
    compiled against brt.h with the reference's include paths (no GPU: plan-only session)."""
    import subprocess, tempfile, ctypes
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = r'''
#include "brt/core/framework/op_kernel.h"
#include "brt/core/framework/op_kernel_info.h"
#include "brt/core/framework/kernel_registry.h"
#include "brt/core/context/work_queue.h"
#include "brt/backends/common.h"
using namespace brt;
static int g_deps[16][4], g_ndeps[16], g_nops = 0;
extern "C" int dep_nops() { return g_nops; }
extern "C" int dep_count(int op) { return g_ndeps[op]; }
extern "C" int dep_at(int op, int k) { return g_deps[op][k]; }
namespace {
class Probe final : public OpKernel {
public:
  explicit Probe(const OpKernelInfo &info) : OpKernel(info, false, false, false, false) {
    const int id = info.GetOpId();
    g_ndeps[id] = (int)info.GetDependency().size();
    for (int k = 0; k < g_ndeps[id] && k < 4; ++k) g_deps[id][k] = info.GetDependency()[(size_t)k];
    if (id + 1 > g_nops) g_nops = id + 1;
  }
  common::Status RunImpl(const ExecutionContext &) override { return common::Status::OK(); }
};
BRT_STATIC_KERNEL_REGISTRATION(DeviceKind::ROCM, ProviderType::BRT, [](KernelRegistry *registry) {
  registry->Register("ProbeOp", [](const brt::OpKernelInfo &info) -> std::shared_ptr<OpKernel> { return std::make_shared<Probe>(info); });
});
}
'''
    from byteir_amd import _lib, brt
    with tempfile.TemporaryDirectory() as tmp:
        cc, so = os.path.join(tmp, "probe.cc"), os.path.join(tmp, "libprobe.so")
        open(cc, "w").write(src)
        libdir = os.path.join(root, "byteir_amd", "lib")
        subprocess.run(["g++", "-std=c++17", "-O1", "-shared", "-fPIC", f"-I{os.path.join(root, 'byteir_amd', 'csrc', 'brt')}",
                        f"-I{os.path.join(root, 'include')}", cc, "-o", so, f"-L{libdir}", "-lbrt", f"-Wl,-rpath,{libdir}"], check=True)
        assert _lib.brt().brt_register_kernels_from_dynlib(so.encode()) == 0
        ext = ctypes.CDLL(so)
        s = brt.Session(device="ROCM", device_id=-1)  # plan only: no GPU needed
        try:
            t = 'memref<8xf32, "cuda">'
            s.load_from_memory(f"""func.func @t(%a : {t} {{byre.argname = "a", byre.argtype = 1: i32}},
                         %b : {t} {{byre.argname = "b", byre.argtype = 2: i32}},
                         %c : {t} {{byre.argname = "c", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{
              byre.compute @ProbeOp(%a, %b) {{memory_effects = [1 : i32, 2 : i32]}} : {t}, {t}
              byre.compute @ProbeOp(%a, %c) {{memory_effects = [1 : i32, 2 : i32]}} : {t}, {t}
              byre.compute @ProbeOp(%b, %c) {{memory_effects = [1 : i32, 3 : i32]}} : {t}, {t}
              byre.compute @ProbeOp(%a, %b) : {t}, {t}
              return }}""")
            assert ext.dep_nops() == 4
            deps = [[ext.dep_at(i, k) for k in range(ext.dep_count(i))] for i in range(4)]
            # op 0 and 1 read only %a (an input: no writer); op 2 reads %b (op 0) and reads+writes %c (op 1);
            # op 3 has no memory_effects: %a never written -> none, %b last written by op 0
            assert deps == [[], [], [0, 1], [0]], deps
        finally:
            s.close()


RESNET_DIR = "/root/reference/runtime/test/test_files"
RESNET_FILES = ["resnet18_fw_bw_host_cuda.mlir", "resnet18_fw_host_cuda.mlir", "resnet18_bw_host_cuda.mlir"]

_RESNET_CHILD = r'''
import ctypes, json, os, re, subprocess, sys, tempfile
root, path = sys.argv[1], sys.argv[2]
sys.path.insert(0, root)
from byteir_amd import _lib, brt
text = open(path).read()
keys = sorted(set(re.findall(r"byre\.compute @([\w.]+)", text)) | set(re.findall(r'byre\.copy\(.*callee = "(\w+)"', text)))
probe = brt.Session(device_id=-1)
missing = [k for k in keys if not probe.has_kernel(k)]
probe.close()
# kernels that do nothing for the op keys this provider has no kernel for (cuDNN / cuBLAS / PTX ops)
src = '#include "brt.h"\nnamespace { class Stub final : public brt::OpKernel { public: explicit Stub(const brt::OpKernelInfo &i) : brt::OpKernel(i) {}\n' \
      '  brt::common::Status RunImpl(const brt::ExecutionContext &) override { return brt::common::Status::OK(); } };\n' \
      'void Reg(brt::KernelRegistry *r) {\n' + "".join(
          f'  r->Register("{k}", [](const brt::OpKernelInfo &i) -> std::shared_ptr<brt::OpKernel> {{ return std::make_shared<Stub>(i); }});\n' for k in missing) + \
      '} }\nBRT_STATIC_KERNEL_REGISTRATION(brt::DeviceKind::ROCM, brt::ProviderType::BRT, Reg)\n'
with tempfile.TemporaryDirectory() as tmp:
    cc, so = os.path.join(tmp, "stubs.cc"), os.path.join(tmp, "libstubs.so")
    open(cc, "w").write(src)
    libdir = os.path.join(root, "byteir_amd", "lib")
    subprocess.run(["g++", "-std=c++17", "-O0", "-shared", "-fPIC", "-I" + os.path.join(root, "byteir_amd", "csrc", "brt"),
                    cc, "-o", so, "-L" + libdir, "-lbrt", "-Wl,-rpath," + libdir], check=True)
    assert _lib.brt().brt_register_kernels_from_dynlib(so.encode()) == 0
    s = brt.Session(device_id=-1)
    s.load(path)
    print(json.dumps({"missing": missing, "ops": s.get_op_keys(), "args": s.get_arg_num(),
                      "cuda_bytes": s.get_intermediate_bytes("cuda")}))
    s.close()
'''


@pytest.mark.skipif(not os.path.isdir(RESNET_DIR), reason="the reference checkout is not mounted")
@pytest.mark.parametrize("name", RESNET_FILES)
def test_reference_resnet_modules_parse_and_plan(name):
    """The reference's ResNet-18 host modules, as its compiler wrote them (module symbol name,
    nested dense attributes, byre.alias into one memref.alloc arena, byre.copy in custom assembly,
    hundreds of arguments).  With the provider's own kernels alone the load ends where the
    reference's would on a provider without cuDNN / PTX ops: `No providers support Op <key>`,
    not a parse error.  With do-nothing kernels registered for those keys from an external
    library (in a child process, so they do not stay registered) the whole module loads: every
    op in file order, the reduce ops bound to this provider's kernels, the arena planned."""
    import json
    import subprocess
    import sys
    from byteir_amd import brt
    path = os.path.join(RESNET_DIR, name)
    text = open(path).read()
    s = brt.Session(device_id=-1)
    try:
        with pytest.raises(RuntimeError, match=r"^No providers support Op \w+"):
            s.load(path)
    finally:
        s.close()
    out = subprocess.run([sys.executable, "-c", _RESNET_CHILD, ROOT, path], check=True, capture_output=True, text=True).stdout
    got = json.loads(out.strip().splitlines()[-1])
    want_ops = re.findall(r"^\s*(?:byre\.compute @([\w.]+)|byre\.copy\(.*callee = \"(\w+)\")", text, flags=re.M)
    want_ops = [a or b for a, b in want_ops]
    assert got["ops"] == want_ops and len(want_ops) > 100
    assert not any(k.startswith("Reduce") for k in got["missing"])  # the reduce ops are this provider's
    assert sum(k.startswith("Reduce") for k in got["ops"]) == len(re.findall(r"byre\.compute @Reduce", text))
    assert got["args"] == len(re.findall(r"byre\.argname", text))
    alloc = re.search(r"memref\.alloc\(\) : memref<(\d+)xi8", text)
    assert alloc and got["cuda_bytes"] >= int(alloc.group(1))


def test_reader_accepts_copy_in_custom_assembly_and_nested_dense(session):
    """byre.copy(%src, %dst) {callee = ...} : type, type (ByreOps.td:170-186; the key is the callee,
    ByreBase.td:170-190) and dense<[[..], [..]]> attributes, as in resnet18_fw_host_cuda.mlir:16,184."""
    t = memref([64], "f32", "cuda")
    session.load_from_memory(f"""module @IrToMhlo.77 attributes {{byre.container_module, gpu.container_module}} {{
      func.func @main(%a : {t} {{byre.argname = "a", byre.argtype = 1 : i32}},
                      %b : {t} {{byre.argname = "b", byre.argtype = 2 : i32}}) attributes {{byre.entry_point}} {{
        byre.copy(%a, %b) {{callee = "cuda2cuda", device = "cuda", padding = dense<[[0, 0], [1, 1]]> : tensor<2x2xi64>}} : {t}, {t}
        return
      }}
    }}""")
    assert session.get_op_keys() == ["cuda2cuda"]
    # inherent attributes printed as a property dictionary (Distributed/ccl.mlir:8): the alias offset
    t2 = memref([8, 4], "f32", "cuda")
    session.load_from_memory(f"""func.func @main(%a : {t} {{byre.argname = "a", byre.argtype = 1 : i32}},
                      %b : {memref([8], "f32", "cuda")} {{byre.argname = "b", byre.argtype = 2 : i32}}) attributes {{byre.entry_point}} {{
        %alloc = memref.alloc() : memref<512xi8, "cuda">
        %0 = "byre.alias"(%alloc) <{{offset = 256 : i64}}> {{device = "cuda"}} : (memref<512xi8, "cuda">) -> {t2}
        byre.compute @ReduceSumOp_f32_f32(%0, %b) {{dimensions = dense<1> : tensor<1xi64>}} : {t2}, {memref([8], "f32", "cuda")}
        return }}""")
    assert session.get_op_keys() == ["ReduceSumOp_f32_f32"] and session.get_intermediate_bytes("cuda") == 512
    with pytest.raises(RuntimeError, match="byre.copy without callee"):
        session.load_from_memory(f"""func.func @main(%a : {t} {{byre.argname = "a", byre.argtype = 1 : i32}},
                      %b : {t} {{byre.argname = "b", byre.argtype = 2 : i32}}) attributes {{byre.entry_point}} {{
        byre.copy(%a, %b) : {t}, {t}
        return }}""")
