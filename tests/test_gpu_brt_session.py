"""End-to-end through the BRT-shaped runtime on the GPU: a ByRE module is loaded into a Session
with the ROCm provider, arguments are bound, Session::Run enqueues the op kernels and the results
are compared with the CPU oracle -- the structure of the reference's op tests
(runtime/test/backends/cuda/providers/default/kernel/{reduction,flash_attn_fwd,flash_attn_bwd}_test.cc)."""
import os

import numpy as np
import pytest
import torch

import oracle
from byre_text import reduction_module, softmax_module
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

REF_CASES = [
    ((1, 16, 32), (0,)), ((1, 16, 32), (1,)), ((1, 16, 32), (2,)), ((1, 16, 32), (0, 1)),
    ((1, 16, 32), (0, 2)), ((1, 128, 128), (0, 1)), ((2, 128, 256), (0, 1)), ((2, 16, 8, 64), (1, 2)),
    ((16384, 8192), (0,)),  # the headline benchmark shape: needs the per-frame workspace
]


@pytest.fixture()
def session():
    from byteir_amd import brt
    s = brt.Session(device="ROCM")
    yield s
    s.close()


@pytest.mark.parametrize("op_name,op", [("ReduceSumOp_f32_f32", oracle.SUM), ("ReduceMaxOp_f32_f32", oracle.MAX)])
@pytest.mark.parametrize("shape,dims", REF_CASES)
def test_reduction_through_session_twice(session, shape, dims, op_name, op):
    session.load_from_memory(reduction_module("cuda", list(shape), list(dims), op_name))
    req = session.new_request_context()  # the request owns its stream
    rng = np.random.default_rng(7)
    out_shape = oracle.deduce_output_shape(shape, dims)
    st, A, B, C = oracle.reduce_canonicalize(shape, out_shape, dims)
    x = dev(rng.random(shape, dtype=np.float32))
    y = torch.full(out_shape, -7.0, device="cuda")
    req.bind_arg(0, x.data_ptr())
    req.bind_arg(1, y.data_ptr())
    req.finish_io_binding()
    for run in range(2):  # second run on the same frame re-uses the workspace (reduction_test.cc:147-164)
        if run:
            x.copy_(dev(rng.random(shape, dtype=np.float32) - 0.5))
            torch.cuda.synchronize()
        req.run()
        req.sync()
        xh, got = host(x), host(y)
        if op == oracle.MAX or not (A and B and C):
            assert np.array_equal(got, oracle.reduce_op(op, xh, dims))
        else:
            s64, sabs = oracle.reduce_sum_f64(xh, A, B, C)
            assert np.all(np.abs(got.reshape(-1) - s64) <= 1e-5 * np.maximum(np.abs(s64), 1e-2 * sabs) + 1e-30)
    req.close()


@pytest.mark.parametrize("op_name,op", [("ReduceMinOp_f32_f32", oracle.MIN), ("ReduceProdOp_f32_f32", oracle.PROD),
                                        ("ReduceMeanOp_f32_f32", oracle.MEAN), ("ReduceSumSqrOp_f32_f32", oracle.SUMSQR)])
@pytest.mark.parametrize("shape,dims", [((2, 16, 8, 64), (1, 2)), ((3000, 520), (0,))])
def test_unregistered_reference_operators_through_session(session, shape, dims, op_name, op):
    """Keys for the operators reduction_helper.h:37-137 defines and no reference op kernel uses."""
    session.load_from_memory(reduction_module("cuda", list(shape), list(dims), op_name))
    req = session.new_request_context()
    rng = np.random.default_rng(9)
    if op == oracle.PROD:  # signs and rare factors of two: exact in any order
        xs = np.where(rng.random(shape) < 0.005, 2.0, 1.0) * rng.choice(np.array([-1.0, 1.0]), size=shape)
    else:
        xs = rng.integers(-2, 3, size=shape)
    x = dev(xs.astype(np.float32))
    y = torch.full(oracle.deduce_output_shape(shape, dims), -7.0, device="cuda")
    req.bind_arg(0, x.data_ptr())
    req.bind_arg(1, y.data_ptr())
    req.finish_io_binding()
    req.run()
    req.sync()
    assert np.array_equal(host(y), oracle.reduce_op(op, host(x), dims))
    req.close()


def test_reduce_ops_of_the_reference_resnet_modules_run_as_written(session, golden_dir):
    """Every `byre.compute @Reduce*` line of the reference's ResNet-18 host modules
    (runtime/test/test_files/resnet18_{fw_bw,fw,bw}_host_cuda.mlir), character for character as the
    reference's compiler wrote them (tests/golden/make_resnet_reduce_module.py gathers them into
    one entry function): f16 and f32, `dense<[3, 2]>` dimensions in descending order, a fold of
    all dimensions into a rank-0 memref, and a fold of a dimension of extent 1."""
    session.load(os.path.join(golden_dir, "resnet18_reduce_ops.mlir"))
    keys = session.get_op_keys()
    assert len(keys) == 8 and set(keys) == {"ReduceSumOp_f16_f16", "ReduceMaxOp_f16_f16", "ReduceSumOp_f32_f32"}
    dims_of = [(1,), (3, 2), (1,), (1,), (0, 1), (0,), (3, 2), (0,)]  # the `dimensions` attributes, in file order
    req = session.new_request_context()
    rng = np.random.default_rng(18)
    bufs = []
    for i in range(len(keys)):
        shape, dt = session.get_static_shape(2 * i), session.get_data_type(2 * i)
        assert session.get_data_type(2 * i + 1) == dt
        tdt = getattr(torch, dt)  # "float16" / "float32"
        x = torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to("cuda", tdt)
        y = torch.full(tuple(session.get_static_shape(2 * i + 1)), -7.0, dtype=tdt, device="cuda")
        req.bind_arg(2 * i, x.data_ptr())
        req.bind_arg(2 * i + 1, y.data_ptr())
        bufs.append((x, y))
    req.finish_io_binding()
    req.run()
    req.sync()
    for key, dims, (x, y) in zip(keys, dims_of, bufs):
        x64 = x.double().cpu().numpy()
        if "Max" in key:
            assert np.array_equal(y.double().cpu().numpy(), x64.max(axis=dims))
            continue
        want, sabs = x64.sum(axis=dims), np.abs(x64).sum(axis=dims)
        got = y.double().cpu().numpy()
        assert got.shape == want.shape
        tol = 1e-5 if x.dtype == torch.float32 else 2.0 ** -10  # f16: one rounding of the float fold
        assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-2 * sabs) + (0 if x.dtype == torch.float32 else 2.0 ** -11 * np.abs(want))), key
    req.close()


def test_copy_in_custom_assembly_into_an_alias_with_a_property_offset(session):
    """byre.copy(%src, %dst) {callee = "cuda2cuda"} (resnet18_fw_host_cuda.mlir:184) into an alias
    whose offset is printed as a property dictionary (Distributed/ccl.mlir:8), then a fold of the
    alias: the copy's key is its callee, the alias lands 256 bytes into the arena."""
    t, to = 'memref<8x4xf32, "cuda">', 'memref<8xf32, "cuda">'
    session.load_from_memory(f"""module @M.1 attributes {{byre.container_module}} {{
      func.func @main(%a : {t} {{byre.argname = "a", byre.argtype = 1 : i32}},
                      %b : {to} {{byre.argname = "b", byre.argtype = 2 : i32}}) attributes {{byre.entry_point}} {{
        %alloc = memref.alloc() : memref<512xi8, "cuda">
        %0 = "byre.alias"(%alloc) <{{offset = 256 : i64}}> {{device = "cuda"}} : (memref<512xi8, "cuda">) -> {t}
        byre.copy(%a, %0) {{callee = "cuda2cuda", device = "cuda"}} : {t}, {t}
        byre.compute @ReduceSumOp_f32_f32(%0, %b) {{device = "cuda", dimensions = dense<1> : tensor<1xi64>, memory_effects = [1 : i32, 2 : i32]}} : {t}, {to}
        return
      }}
    }}""")
    assert session.get_op_keys() == ["cuda2cuda", "ReduceSumOp_f32_f32"]
    req = session.new_request_context()
    x = torch.arange(32, dtype=torch.float32, device="cuda").reshape(8, 4)
    y = torch.full((8,), -7.0, device="cuda")
    req.bind_arg(0, x.data_ptr())
    req.bind_arg(1, y.data_ptr())
    req.finish_io_binding()
    req.run()
    req.sync()
    assert torch.equal(y, x.sum(dim=1))
    req.close()


@pytest.mark.parametrize("op_name", ["ReduceSumOp_f32_f32", "ReduceMaxOp_f32_f32"])
def test_nan_propagation_through_session(session, op_name):
    # reduction_test.cc:182-215: 1024 elements, NaN first; runtime-allocated arguments
    session.load_from_memory(reduction_module("cuda", [1024], [0], op_name))
    req = session.new_request_context()
    x = np.random.default_rng(8).random(1024, dtype=np.float32)
    x[0] = np.nan
    from byteir_amd import _lib
    K = _lib.kernels()
    p_in = req.get_arg(0)  # allocated by the frame, like request->GetArg(0) in the reference test
    _lib.check(K.brt_rocm_memcpy_h2d(p_in, x.ctypes.data, x.nbytes, None))
    _lib.check(K.brt_rocm_device_synchronize())
    req.finish_io_binding()
    req.run()
    req.sync()
    out = np.zeros(1, np.float32)
    _lib.check(K.brt_rocm_memcpy_d2h(out.ctypes.data, req.get_arg(1), 4, None))
    _lib.check(K.brt_rocm_device_synchronize())
    assert np.isnan(out[0])


def test_flash_attn_fwd_module_unchanged(session, golden_dir):
    """SM80CUDATestFlashAttnFwd.Basic: the reference's fixture module and data; Q, K, V, Out and
    SoftmaxLse are bound, SoftmaxPtr and RngState are left to the frame."""
    session.load(os.path.join(golden_dir, "flash_attn_fwd.mlir"))
    req = session.new_request_context(torch.cuda.current_stream().cuda_stream)
    g = {n: np.load(os.path.join(golden_dir, f"fa_{n}.npy")) for n in ("q", "k", "v", "out")}
    q, k, v = dev(g["q"]), dev(g["k"]), dev(g["v"])
    o = torch.zeros_like(q)
    lse = torch.zeros((1, 3, 128), device="cuda")
    for i, t in enumerate((q, k, v, o, lse)):
        req.bind_arg(i, t.data_ptr())
    req.finish_io_binding()
    req.run()
    req.sync()
    got, want = host(o).astype(np.float32), g["out"].astype(np.float32)
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.abs(want) + 1e-7)  # one fp16 ulp
    _, lse_ref, _ = oracle.flash_fwd(g["q"], g["k"], g["v"], 0.5, (-1, 0))
    np.testing.assert_allclose(host(lse), lse_ref, atol=1e-4)


def test_flash_attn_bwd_module_unchanged(session, golden_dir):
    """SM80CUDATestFlashAttnBwd.Basic: forward then backward in one module."""
    session.load(os.path.join(golden_dir, "flash_attn_bwd.mlir"))
    req = session.new_request_context(torch.cuda.current_stream().cuda_stream)
    g = {n: np.load(os.path.join(golden_dir, f"fa_{n}.npy")) for n in ("q", "k", "v", "dout", "out", "dq", "dk", "dv")}
    do, q, k, v = dev(g["dout"]), dev(g["q"]), dev(g["k"]), dev(g["v"])
    o = torch.zeros_like(q)
    lse = torch.zeros((1, 3, 128), device="cuda")
    dq, dk, dv = torch.zeros_like(q), torch.zeros_like(q), torch.zeros_like(q)
    for i, t in enumerate((do, q, k, v, o, lse, dq, dk, dv)):
        req.bind_arg(i, t.data_ptr())
    req.finish_io_binding()  # RngState, d_SoftmaxLse, d_Q_accum, SoftmaxPtr come from the frame
    req.run()
    req.sync()
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        want = g[name].astype(np.float32)
        err = np.abs(host(t).astype(np.float32) - want)
        assert np.all(err <= 2 * 2.0 ** -10 * np.abs(want) + 4e-6), name


@pytest.mark.parametrize("dtype,code", [("f32", oracle.F32), ("bf16", oracle.BF16), ("f16", oracle.F16)])
def test_softmax_through_backend(dtype, code):
    """byteir.softmax via BRTBackend (torch's caching allocator and current stream), on the
    reference's own softmax test shapes."""
    import tempfile
    from byteir_amd.brt import BRTBackend
    for shape, axis in (([10, 128], 1), ([2, 3, 256, 256], -1), ([4, 50, 96], 1)):
        with tempfile.NamedTemporaryFile("w", suffix=".mlir", delete=False) as f:
            f.write(softmax_module("cuda", shape, dtype, axis))
        be = BRTBackend("cuda", f.name)
        x32 = (np.random.default_rng(9).standard_normal(shape) * 2).astype(np.float32)
        xs = oracle.from_f32(x32, code)
        (y,) = be.run([dev(xs)])
        got, want = oracle.to_f32(host(y)), oracle.to_f32(oracle.softmax(xs, axis=axis))
        rel = {oracle.F32: 1e-5, oracle.F16: 2.0 ** -10, oracle.BF16: 2.0 ** -7}[code]
        assert np.all(np.abs(got - want) <= rel * np.abs(want) + 6e-8)
        ms = be.profile_with_outputs([dev(xs)], [y], warmup=2, iters=3)
        assert ms > 0
        be.session.close()
        os.unlink(f.name)


def test_copy_ops_and_listener(session):
    text = """func.func @t(%h : memref<1000xf32, "cpu"> {byre.argname = "h", byre.argtype = 1: i32},
                      %o : memref<1000xf32, "cpu"> {byre.argname = "o", byre.argtype = 2: i32}) attributes {byre.entry_point} {
      %d0 = memref.alloc() : memref<1000xf32, "cuda">
      %d1 = memref.alloc() : memref<1000xf32, "cuda">
      byre.compute @cpu2cuda(%h, %d0) {device = "cuda"} : memref<1000xf32, "cpu">, memref<1000xf32, "cuda">
      byre.compute @cuda2cuda(%d0, %d1) : memref<1000xf32, "cuda">, memref<1000xf32, "cuda">
      byre.compute @cuda2cpu(%d1, %o) : memref<1000xf32, "cuda">, memref<1000xf32, "cpu">
      return }"""
    session.load_from_memory(text)
    req = session.new_request_context()
    seen = []
    req.add_op_listener(lambda key, idx, after: seen.append((key, idx, after)))
    src = np.arange(1000, dtype=np.float32)
    dst = np.zeros(1000, dtype=np.float32)
    req.bind_arg(0, src.ctypes.data)
    req.bind_arg(1, dst.ctypes.data)
    req.finish_io_binding()
    req.run()
    req.sync()
    assert np.array_equal(src, dst)
    assert seen == [("cpu2cuda", 0, False), ("cpu2cuda", 0, True), ("cuda2cuda", 1, False), ("cuda2cuda", 1, True),
                    ("cuda2cpu", 2, False), ("cuda2cpu", 2, True)]


# ---- request context, frames and work queues -------------------------------------------------
# Mirrors of CUDARequestContextTest.{NoBindArg,BindArg1,BindArg2}
# (runtime/test/backends/cuda/providers/default/request_context_test.cc:48-200),
# BRTInferenceExecutionFrameTest.TestStateInfoSharing (runtime/test/context/exec_frame_test.cc:94)
# and CUDAWorkQueueTest.{CUDASingleStreamWorkQueue,CUDAExternalStreamWorkQueue}
# (runtime/test/backends/cuda/device/cuda_work_queue_test.cc:82,190), with a reduction standing in
# for the reference's AddOp.

def _h2d(ptr, arr):
    from byteir_amd import _lib
    K = _lib.kernels()
    _lib.check(K.brt_rocm_memcpy_h2d(ptr, arr.ctypes.data, arr.nbytes, None))
    _lib.check(K.brt_rocm_device_synchronize())


def _d2h(ptr, shape, dtype=np.float32):
    from byteir_amd import _lib
    K = _lib.kernels()
    out = np.empty(shape, dtype)
    _lib.check(K.brt_rocm_memcpy_d2h(out.ctypes.data, ptr, out.nbytes, None))
    _lib.check(K.brt_rocm_device_synchronize())
    return out


def test_request_context_without_binding(session):
    """Nothing bound: the frame allocates every entry argument, get_arg hands out the pointers."""
    session.load_from_memory(reduction_module("cuda", [64, 4096], [1], "ReduceMaxOp_f32_f32"))
    req = session.new_request_context()
    x = np.random.default_rng(3).standard_normal((64, 4096)).astype(np.float32)
    p_in, p_out = req.get_arg(0), req.get_arg(1)
    assert p_in and p_out and p_in != p_out
    _h2d(p_in, x)
    req.finish_io_binding()
    req.run()
    req.sync()
    assert req.get_arg(1) == p_out
    assert np.array_equal(_d2h(p_out, (64,)), x.max(axis=1))
    req.close()


def test_request_context_partial_binding_and_rebinding(session):
    """One argument bound by the caller, the other owned by the frame; binding over a
    frame-owned argument releases it; a rebound argument is what the next run uses."""
    session.load_from_memory(reduction_module("cuda", [64, 4096], [1], "ReduceMaxOp_f32_f32"))
    req = session.new_request_context()
    rng = np.random.default_rng(4)
    x0 = rng.standard_normal((64, 4096)).astype(np.float32)
    x1 = rng.standard_normal((64, 4096)).astype(np.float32)
    y = torch.zeros(64, device="cuda")
    p_in = req.get_arg(0)           # frame-owned input
    req.bind_arg(1, y.data_ptr())   # caller-owned output
    _h2d(p_in, x0)
    req.finish_io_binding()
    req.run()
    req.sync()
    assert np.array_equal(host(y), x0.max(axis=1))
    dx1 = dev(x1)
    req.bind_arg(0, dx1.data_ptr())  # replaces (and frees) the frame-owned buffer
    assert req.get_arg(0) == dx1.data_ptr()
    req.finish_io_binding()
    req.run()
    req.sync()
    assert np.array_equal(host(y), x1.max(axis=1))
    req.close()


def test_run_before_finish_io_binding_is_an_error(session):
    session.load_from_memory(reduction_module("cuda", [8, 8], [1], "ReduceSumOp_f32_f32"))
    req = session.new_request_context()
    with pytest.raises(RuntimeError, match="FinishIOBinding"):
        req.run()
    req.close()


def test_two_requests_of_one_session_are_independent(session):
    """Two frames of one plan: each has its own arguments and its own reduce workspace, runs
    interleave on two streams."""
    shape = (16384, 2048)
    session.load_from_memory(reduction_module("cuda", list(shape), [0], "ReduceSumOp_f32_f32"))
    reqs, xs, ys = [], [], []
    gen = torch.Generator(device="cuda").manual_seed(11)
    for i in range(2):
        r = session.new_request_context()
        x = torch.rand(shape, generator=gen, device="cuda") - 0.5
        y = torch.empty(shape[1], device="cuda")
        r.bind_arg(0, x.data_ptr())
        r.bind_arg(1, y.data_ptr())
        r.finish_io_binding()
        reqs.append(r), xs.append(x), ys.append(y)
    torch.cuda.synchronize()
    for _ in range(3):
        for r in reqs:
            r.run()
    for r in reqs:
        r.sync()
    for x, y in zip(xs, ys):
        want = x.double().sum(dim=0)
        sabs = x.double().abs().sum(dim=0)
        assert bool(((y.double() - want).abs() <= 1e-5 * torch.maximum(want.abs(), 1e-2 * sabs)).all())
    for r in reqs:
        r.close()


def test_workspace_is_allocated_once_per_frame_and_freed_with_it():
    """The reduce workspace is per-frame state: allocated at the frame's first run through the
    session's allocator, reused by later runs, released when the request goes away."""
    from byteir_amd import brt
    live, allocs = {}, []

    def alloc(n):
        p = torch.cuda.caching_allocator_alloc(n)
        live[p] = n
        allocs.append(n)
        return p

    def free(p):
        del live[p]
        torch.cuda.caching_allocator_delete(p)

    s = brt.Session(device="ROCM", alloc_func=alloc, free_func=free)
    shape = (16384, 8192)
    s.load_from_memory(reduction_module("cuda", list(shape), [0], "ReduceMaxOp_f32_f32"))
    from byteir_amd import ops
    need = ops.reduce_workspace_bytes(torch.float32, 1, *shape)
    assert need > 0
    x = torch.rand(shape, device="cuda")
    y = torch.empty(shape[1], device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    reqs = []
    for _ in range(2):
        r = s.new_request_context(stream)
        r.bind_arg(0, x.data_ptr())
        r.bind_arg(1, y.data_ptr())
        r.finish_io_binding()
        reqs.append(r)
    assert allocs == []                      # nothing is allocated before the first run
    reqs[0].run()
    assert allocs == [need]
    for _ in range(3):
        reqs[0].run()
    assert allocs == [need]                  # later runs of the same frame reuse it
    reqs[1].run()
    assert allocs == [need, need]            # a second frame has its own
    reqs[0].sync()
    assert torch.equal(y, x.amax(dim=0))
    reqs[0].close()
    assert len(live) == 1
    reqs[1].close()
    assert live == {}
    s.close()


def test_external_stream_work_queue_keeps_stream_order(session):
    """A request on a caller's stream is ordered after the work already enqueued there (the
    producer of its input) without any host synchronisation; a request that owns its stream is
    synchronised by its own sync()."""
    shape = (8192, 8192)
    session.load_from_memory(reduction_module("cuda", list(shape), [1], "ReduceMaxOp_f32_f32"))
    side = torch.cuda.Stream()
    x = torch.zeros(shape, device="cuda")
    y = torch.zeros(shape[0], device="cuda")
    torch.cuda.synchronize()
    req = session.new_request_context(side.cuda_stream)
    req.bind_arg(0, x.data_ptr())
    req.bind_arg(1, y.data_ptr())
    req.finish_io_binding()
    with torch.cuda.stream(side):
        for k in range(1, 9):           # eight full passes over 256 MiB, then the reduction, no host wait
            x.add_(float(k))
        req.run()
    req.sync()                          # waits for the caller's stream
    assert torch.equal(y, torch.full((shape[0],), 36.0, device="cuda"))
    req.close()


def test_flash_attn_kvcache_module_unchanged(session, golden_dir):
    """SM80CUDATestFlashAttnKVCache.Basic through the session: the reference's module text and
    data, all eight arguments bound (flash_attn_fwd_test.cc:183-330)."""
    session.load(os.path.join(golden_dir, "flash_attn_kvcache.mlir"))
    req = session.new_request_context(torch.cuda.current_stream().cuda_stream)
    g = {n: np.load(os.path.join(golden_dir, f"fa_kv_{n}.npy")) for n in
         ("q", "knew", "vnew", "kcache", "vcache", "out", "kcache_out", "vcache_out", "seqlens")}
    q, kc, vc, kn, vn, lens = (dev(g[n]) for n in ("q", "kcache", "vcache", "knew", "vnew", "seqlens"))
    o = torch.zeros_like(q)
    lse = torch.zeros((2, 3, 1), device="cuda")
    for i, t in enumerate((q, kc, vc, kn, vn, lens, o, lse)):
        req.bind_arg(i, t.data_ptr())
    req.finish_io_binding()
    req.run()
    req.sync()
    got, want = host(o).astype(np.float32), g["out"].astype(np.float32)
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.abs(want) + 1e-7)  # one fp16 ulp
    assert np.array_equal(host(kc), g["kcache_out"]) and np.array_equal(host(vc), g["vcache_out"])


def test_intermediates_live_in_one_arena_per_frame():
    """The memref.alloc intermediates of a module come out of ONE allocation per frame and
    memory space (the static plan's arena), not one allocation each; data still flows through
    them correctly, an alias included."""
    from byteir_amd import brt
    allocs = []

    def alloc(n):
        allocs.append(n)
        return torch.cuda.caching_allocator_alloc(n)

    s = brt.Session(device="ROCM", alloc_func=alloc, free_func=torch.cuda.caching_allocator_delete)
    text = """func.func @t(%x : memref<64x4096xf32, "cuda"> {byre.argname = "x", byre.argtype = 1: i32},
                      %y : memref<64xf32, "cuda"> {byre.argname = "y", byre.argtype = 2: i32}) attributes {byre.entry_point} {
      %a = memref.alloc() : memref<64x4096xf32, "cuda">
      %b = memref.alloc() : memref<1048576xi8, "cuda">
      %bv = "byre.alias"(%b) {offset = 0 : i64} : (memref<1048576xi8, "cuda">) -> memref<64x4096xf32, "cuda">
      %m = memref.alloc() : memref<64xf32, "cuda">
      byre.compute @cuda2cuda(%x, %a) : memref<64x4096xf32, "cuda">, memref<64x4096xf32, "cuda">
      byre.compute @cuda2cuda(%a, %bv) : memref<64x4096xf32, "cuda">, memref<64x4096xf32, "cuda">
      byre.compute @ReduceMaxOp_f32_f32(%bv, %m) {dimensions = dense<[1]> : tensor<1xi64>} : memref<64x4096xf32, "cuda">, memref<64xf32, "cuda">
      byre.compute @cuda2cuda(%m, %y) : memref<64xf32, "cuda">, memref<64xf32, "cuda">
      return }"""
    s.load_from_memory(text)
    arena = 2 * 64 * 4096 * 4 + 256
    assert s.get_intermediate_bytes("cuda") == arena
    x = torch.randn((64, 4096), device="cuda")
    y = torch.zeros(64, device="cuda")
    req = s.new_request_context(torch.cuda.current_stream().cuda_stream)
    req.bind_arg(0, x.data_ptr())
    req.bind_arg(1, y.data_ptr())
    req.finish_io_binding()
    assert allocs == [arena]
    for _ in range(2):
        req.run()
    req.sync()
    from byteir_amd import ops
    ws = ops.reduce_workspace_bytes(torch.float32, 64, 4096, 1)  # the reduce op's own per-frame workspace
    assert allocs == ([arena, ws] if ws else [arena])
    assert torch.equal(y, x.amax(dim=1))
    req.close()
    s.close()


def test_op_kernels_on_two_streams_at_once():
    """Nothing in the kernel libraries is shared between calls (workspaces are per call or
    stream-ordered): the same work issued on two streams at once gives the serial results."""
    from byteir_amd import ops, _lib
    gen = torch.Generator(device="cuda").manual_seed(3)
    work = []
    for i in range(2):
        x = torch.randn((4096, 2048), generator=gen, device="cuda")
        q = torch.randn((1, 64, 8, 128), generator=gen, device="cuda").half()      # few query blocks, many keys:
        k = torch.randn((1, 5000, 2, 128), generator=gen, device="cuda").half()    # key axis split, scratch allocation
        v = torch.randn_like(k)
        xs = torch.randn((1, 9000, 24), generator=gen, device="cuda")              # segmented inner-axis softmax
        work.append((x, q, k, v, xs))

    def run(i, stream):
        x, q, k, v, xs = work[i]
        r = ops.reduce(_lib.REDUCE_SUM, x, (0,), stream=stream)
        o, lse = ops.flash_attn_fwd(q, k, v, 0.1, (-1, 0), stream=stream)
        y = ops.softmax(xs, stream=stream, axis=1)
        return r, o, lse, y

    serial = [run(i, None) for i in range(2)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(3):
        both = []
        for i, s in enumerate(streams):
            with torch.cuda.stream(s):
                both.append(run(i, s))
        torch.cuda.synchronize()
        for got, want in zip(both, serial):
            for a, c in zip(got, want):
                assert torch.equal(a, c)


def test_device_memset_any_alignment_and_inside_a_graph():
    """brt_rocm_memset (the DeviceAPI memset of cuda_device_api.cc:29-55) is a fill kernel: every
    byte of the range and none outside it, for any alignment and length; replays of a captured
    call keep working."""
    import ctypes
    from byteir_amd import _lib
    K = _lib.kernels()
    buf = torch.zeros(5000, dtype=torch.uint8, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for off, n, val in ((0, 5000, 7), (1, 4998, 200), (13, 3, 9), (16, 16, 1), (31, 1000, 255), (5, 0, 3)):
        buf.fill_(0x55)
        _lib.check(K.brt_rocm_memset(ctypes.c_void_p(buf.data_ptr() + off), val, n, st), "memset")
        h = buf.cpu().numpy()
        assert np.all(h[off:off + n] == val) and np.all(h[:off] == 0x55) and np.all(h[off + n:] == 0x55), (off, n)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _lib.check(K.brt_rocm_memset(ctypes.c_void_p(buf.data_ptr() + 3), 0, 4001, ctypes.c_void_p(side.cuda_stream)), "memset")
    for _ in range(3):
        buf.fill_(0x77)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        h = buf.cpu().numpy()
        assert np.all(h[3:4004] == 0) and np.all(h[:3] == 0x77) and np.all(h[4004:] == 0x77)


def test_reference_style_external_kernel_runs_with_its_hooks(tmp_path):
    """The external kernel of tests/external_kernel_src.py on the GPU: ProloguePerFrame once per
    frame (also when the frame runs twice), its state found through frame_state_info on every
    run, events around each run, EpiloguePerFrame when the request is destroyed, and a custom
    op whose arguments the library refuses fails Session::Run instead of ending the process."""
    import ctypes
    from byteir_amd import _lib, brt
    from external_kernel_src import build
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = build(tmp_path, root)
    assert _lib.brt().brt_register_kernels_from_dynlib(str(lib).encode()) == 0
    ext = ctypes.CDLL(str(lib))
    s = brt.Session(device="ROCM")
    try:
        t = 'memref<1000xf32, "cuda">'
        s.load_from_memory(f"""func.func @t(%a : {t} {{byre.argname = "a", byre.argtype = 1: i32}},
                     %b : {t} {{byre.argname = "b", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{
          byre.compute @CustomCopyOp(%a, %b) : {t}, {t}
          return }}""")
        f0, e0, r0 = ext.ext_prologue_per_frame(), ext.ext_epilogue_per_frame(), ext.ext_runs()
        a = torch.arange(1000, dtype=torch.float32, device="cuda")
        b = torch.zeros(1000, device="cuda")
        req = s.new_request_context()
        seen = []
        req.add_op_listener(lambda key, idx, after: seen.append((key, after)))
        req.bind_arg(0, a.data_ptr()); req.bind_arg(1, b.data_ptr()); req.finish_io_binding()
        req.run(); req.run(); req.sync()
        assert torch.equal(a, b)
        assert ext.ext_prologue_per_frame() == f0 + 1 and ext.ext_runs() == r0 + 2
        assert seen == [("CustomCopyOp", False), ("CustomCopyOp", True)] * 2
        req2 = s.new_request_context()  # a second frame of the same plan: its own state, same offset
        req2.bind_arg(0, a.data_ptr()); req2.bind_arg(1, b.data_ptr()); req2.finish_io_binding()
        req2.run(); req2.sync()
        assert ext.ext_prologue_per_frame() == f0 + 2
        req.close(); req2.close()
        assert ext.ext_epilogue_per_frame() == e0 + 2
    finally:
        s.close()


def test_external_kernel_in_the_reference_launch_idiom():
    """tests/external_kernels/custom_add.hip (built ahead of time by byteir_amd.build): a
    __global__ function handed to WorkQueue::AddTask with {grid, block, shared bytes, arguments},
    the op id and GetDependency() -- the launch idiom of runtime/test/external_kernels/cuda/
    kernels.cc:52-79 -- plus a host task through DispatchHostTask.  Two chained adds: the second
    op reads what the first wrote, so its dependency list names the first."""
    import ctypes
    from byteir_amd import _lib, brt
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = os.path.join(root, "tests", "external_kernels", "libcustom_add.so")
    assert os.path.exists(lib), "run python -m byteir_amd.build test_kernels"
    assert _lib.brt().brt_register_kernels_from_dynlib(lib.encode()) == 0
    ext = ctypes.CDLL(lib)
    s = brt.Session(device="ROCM")
    try:
        t = 'memref<5000xf32, "cuda">'
        s.load_from_memory(f"""func.func @t(%a : {t} {{byre.argname = "a", byre.argtype = 1: i32}},
                     %b : {t} {{byre.argname = "b", byre.argtype = 1: i32}},
                     %c : {t} {{byre.argname = "c", byre.argtype = 2: i32}},
                     %d : {t} {{byre.argname = "d", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{
          byre.compute @CustomAddOp(%a, %b, %c) {{memory_effects = [1 : i32, 1 : i32, 2 : i32]}} : {t}, {t}, {t}
          byre.compute @CustomAddOp(%c, %b, %d) {{memory_effects = [1 : i32, 1 : i32, 2 : i32]}} : {t}, {t}, {t}
          return }}""")
        assert ext.ext_add_prologue_per_session() >= 2
        f0, h0 = ext.ext_add_prologue_per_frame(), ext.ext_add_host_tasks()
        gen = torch.Generator(device="cuda").manual_seed(7)
        a, b = (torch.randn(5000, generator=gen, device="cuda") for _ in range(2))
        c, d = torch.zeros(5000, device="cuda"), torch.zeros(5000, device="cuda")
        req = s.new_request_context()
        for i, x in enumerate((a, b, c, d)):
            req.bind_arg(i, x.data_ptr())
        req.finish_io_binding()
        req.run(); req.sync()
        assert torch.equal(c, a + b) and torch.equal(d, (a + b) + b)
        assert ext.ext_add_prologue_per_frame() == f0 + 2          # once per op and frame
        assert ext.ext_add_host_tasks() == h0 + 2                  # the host tasks ran, in queue order, before sync returned
        assert ext.ext_add_last_op_id() == 1 and ext.ext_add_last_dependency_count() == 1  # op 1 waits for op 0 (%c)
        req.close()
    finally:
        s.close()


def test_custom_op_with_unsupported_arguments_fails_the_run(session, golden_dir):
    """head_dim 20 is not a multiple of 8: through the plain ABI the library would abort the
    process; the custom op kernel uses the library's error-returning entry point instead."""
    text = open(os.path.join(golden_dir, "flash_attn_fwd.mlir")).read()
    # the fixture is b1 s128 h3 d32; declare d = 20 in the blob (fields 16..18 head strides stay)
    import re
    m = re.search(r"extra_args = \[([^\]]*)\]", text)
    fields = [f.strip() for f in m.group(1).split(",")]
    # blob order (flash_api.cu:586-624): 4 batch strides, 4 row strides, 4 head strides, b, h, h_k, d, ...
    assert fields[15].startswith("32")
    fields[15] = "20 : i64"
    text = text.replace(m.group(1), ", ".join(fields))
    session.load_from_memory(text)
    req = session.new_request_context()
    q, k, v = (torch.zeros((1, 128, 3, 32), dtype=torch.float16, device="cuda") for _ in range(3))
    o = torch.zeros_like(q)
    lse = torch.zeros((1, 3, 128), device="cuda")
    for name, t in (("Q", q), ("K", k), ("V", v), ("Out", o), ("SoftmaxLse", lse)):
        off = session.get_graph_arg_offset(name)
        if off >= 0:
            req.bind_arg(off, t.data_ptr())
    req.finish_io_binding()
    with pytest.raises(RuntimeError, match="custom op"):
        req.run()
    req.sync()
