"""Runs one scenario of tests/test_session_emulated.py in a process of its own: the Python mirror
of the runtime (byteir_amd.brt) is pointed at tests/emu/lib, where libbrt.so, libbrt_rocm_kernels.so
and libflash_attn.so are the host builds (HIP kernels executed lane by lane, "device" memory =
guarded host memory).  A separate process, because the GPU libraries of the same names may
already be loaded globally in the test process.  Exit code 0 = the scenario's checks passed."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import numpy as np

from byteir_amd import _lib

EMU_LIB_DIR = os.path.join(HERE, "emu", "lib")
_lib.LIB_DIR = EMU_LIB_DIR                       # before anything is loaded
os.environ["BRT_CUSTOM_LIB_DIR"] = EMU_LIB_DIR   # where `custom` ops look their library up by file name

from byteir_amd import brt  # noqa: E402
import oracle  # noqa: E402
from byre_text import reduction_module, softmax_module  # noqa: E402

GOLDEN = os.path.join(HERE, "golden")


def ptr(a):
    return a.ctypes.data


def run(session, arrays):
    req = session.new_request_context()
    for i, a in enumerate(arrays):
        req.bind_arg(i, ptr(a))
    req.finish_io_binding()
    req.run()
    req.sync()
    return req


def scenario_reductions():
    """The reference's reduction shape list through Session::Run, twice per frame (reduction_test.cc:147-180)."""
    cases = [((1, 16, 32), (0,)), ((1, 16, 32), (1,)), ((1, 16, 32), (2,)), ((1, 16, 32), (0, 1)), ((1, 16, 32), (0, 2)),
             ((1, 128, 128), (0, 1)), ((2, 128, 256), (0, 1)), ((2, 16, 8, 64), (1, 2)), ((3000, 520), (0,))]
    rng = np.random.default_rng(7)
    for shape, dims in cases:
        for key, op in (("ReduceSumOp_f32_f32", oracle.SUM), ("ReduceMaxOp_f32_f32", oracle.MAX)):
            s = brt.Session(device="ROCM")
            s.load_from_memory(reduction_module("cuda", list(shape), list(dims), key))
            out_shape = oracle.deduce_output_shape(shape, dims)
            x = rng.random(shape, dtype=np.float32)
            y = np.full(out_shape, -7.0, np.float32)
            req = s.new_request_context()
            req.bind_arg(0, ptr(x))
            req.bind_arg(1, ptr(y))
            req.finish_io_binding()
            for rep in range(2):
                if rep:
                    x[...] = rng.random(shape, dtype=np.float32) - 0.5
                req.run()
                req.sync()
                if op == oracle.MAX:
                    assert np.array_equal(y, oracle.reduce_op(op, x, dims)), (shape, dims, key)
                else:
                    want = x.astype(np.float64).sum(axis=dims)
                    mag = np.abs(x.astype(np.float64)).sum(axis=dims)
                    assert np.all(np.abs(y - want) <= 1e-5 * np.maximum(np.abs(want), 1e-2 * mag)), (shape, dims, key)
            req.close()
            s.close()


def scenario_resnet_reduce_ops():
    """Every Reduce* line of the reference's ResNet-18 host modules, as its compiler wrote them."""
    s = brt.Session(device="ROCM")
    s.load(os.path.join(GOLDEN, "resnet18_reduce_ops.mlir"))
    keys = s.get_op_keys()
    dims_of = [(1,), (3, 2), (1,), (1,), (0, 1), (0,), (3, 2), (0,)]
    rng = np.random.default_rng(18)
    bufs = []
    for i in range(len(keys)):
        shape, dt = s.get_static_shape(2 * i), s.get_data_type(2 * i)
        npdt = np.float16 if dt == "float16" else np.float32
        bufs.append((rng.standard_normal(shape).astype(npdt), np.full(s.get_static_shape(2 * i + 1), -7.0, npdt)))
    run(s, [a for pair in bufs for a in pair]).close()
    for key, dims, (x, y) in zip(keys, dims_of, bufs):
        x64 = x.astype(np.float64)
        if "Max" in key:
            assert np.array_equal(y.astype(np.float64), x64.max(axis=dims)), key
            continue
        want, mag = x64.sum(axis=dims), np.abs(x64).sum(axis=dims)
        tol = 1e-5 if x.dtype == np.float32 else 2.0 ** -10
        assert np.all(np.abs(y.astype(np.float64) - want) <= tol * np.maximum(np.abs(want), 1e-2 * mag) + 2.0 ** -11 * np.abs(want)), key
    s.close()


def scenario_flash_attn_golden():
    """The reference's flash-attention modules and golden vectors (SM80CUDATestFlashAttnFwd.Basic,
    ...Bwd.Basic, ...KVCache.Basic), byte for byte, on the host."""
    g = {n: np.load(os.path.join(GOLDEN, f"fa_{n}.npy")) for n in ("q", "k", "v", "dout", "out", "dq", "dk", "dv")}
    s = brt.Session(device="ROCM")
    s.load(os.path.join(GOLDEN, "flash_attn_fwd.mlir"))
    q, k, v = g["q"].copy(), g["k"].copy(), g["v"].copy()
    o, lse = np.zeros_like(q), np.zeros((1, 3, 128), np.float32)
    run(s, [q, k, v, o, lse]).close()
    want = g["out"].astype(np.float32)
    assert np.all(np.abs(o.astype(np.float32) - want) <= 2.0 ** -10 * np.abs(want) + 1e-7), "forward: one fp16 ulp"
    _, lse_ref, _ = oracle.flash_fwd(g["q"], g["k"], g["v"], 0.5, (-1, 0))
    np.testing.assert_allclose(lse, lse_ref, atol=1e-4)
    s.close()

    s = brt.Session(device="ROCM")
    s.load(os.path.join(GOLDEN, "flash_attn_bwd.mlir"))
    do = g["dout"].copy()
    o, lse = np.zeros_like(q), np.zeros((1, 3, 128), np.float32)
    dq, dk, dv = np.zeros_like(q), np.zeros_like(q), np.zeros_like(q)
    run(s, [do, q, k, v, o, lse, dq, dk, dv]).close()
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
        want = g[name].astype(np.float32)
        assert np.all(np.abs(t.astype(np.float32) - want) <= 2 * 2.0 ** -10 * np.abs(want) + 4e-6), name
    s.close()

    g = {n: np.load(os.path.join(GOLDEN, f"fa_kv_{n}.npy")) for n in
         ("q", "knew", "vnew", "kcache", "vcache", "out", "kcache_out", "vcache_out", "seqlens")}
    s = brt.Session(device="ROCM")
    s.load(os.path.join(GOLDEN, "flash_attn_kvcache.mlir"))
    q, kc, vc, kn, vn, lens = (g[n].copy() for n in ("q", "kcache", "vcache", "knew", "vnew", "seqlens"))
    o, lse = np.zeros_like(q), np.zeros((2, 3, 1), np.float32)
    run(s, [q, kc, vc, kn, vn, lens, o, lse]).close()
    want = g["out"].astype(np.float32)
    assert np.all(np.abs(o.astype(np.float32) - want) <= 2.0 ** -10 * np.abs(want) + 1e-7), "cache call: one fp16 ulp"
    assert np.array_equal(kc, g["kcache_out"]) and np.array_equal(vc, g["vcache_out"])
    s.close()


def scenario_softmax_and_copies():
    """byteir.softmax through the session, and a module that copies host -> device, folds, copies back."""
    rng = np.random.default_rng(3)
    for shape, dtype in (((32, 128), "f32"), ((7, 1000), "f16"), ((3, 4096), "f32")):
        s = brt.Session(device="ROCM")
        s.load_from_memory(softmax_module("cuda", list(shape), dtype, len(shape) - 1))
        npdt = np.float16 if dtype == "f16" else np.float32
        x = (rng.standard_normal(shape) * 2).astype(npdt)
        y = np.zeros(shape, npdt)
        run(s, [x, y]).close()
        e = np.exp(x.astype(np.float64) - x.astype(np.float64).max(-1, keepdims=True))
        want = e / e.sum(-1, keepdims=True)
        ulp = 2.0 ** -10 if dtype == "f16" else 2.0 ** -22
        assert np.all(np.abs(y - want) <= 2 * ulp * want + 2.0 ** -24), (shape, dtype)
        s.close()
    t_h, t_d, t_o = 'memref<8x4xf32, "cpu">', 'memref<8x4xf32, "cuda">', 'memref<8xf32, "cuda">'
    s = brt.Session(device="ROCM")
    s.load_from_memory(f"""func.func @main(%a : {t_h} {{byre.argname = "a", byre.argtype = 1 : i32}},
                      %b : memref<8xf32, "cpu"> {{byre.argname = "b", byre.argtype = 2 : i32}}) attributes {{byre.entry_point}} {{
        %0 = memref.alloc() : {t_d}
        %1 = memref.alloc() : {t_o}
        byre.compute @cpu2cuda(%a, %0) {{memory_effects = [1 : i32, 2 : i32]}} : {t_h}, {t_d}
        byre.compute @ReduceSumOp_f32_f32(%0, %1) {{dimensions = dense<1> : tensor<1xi64>, memory_effects = [1 : i32, 2 : i32]}} : {t_d}, {t_o}
        byre.compute @cuda2cpu(%1, %b) {{memory_effects = [1 : i32, 2 : i32]}} : {t_o}, memref<8xf32, "cpu">
        return }}""")
    x = np.arange(32, dtype=np.float32).reshape(8, 4)
    y = np.zeros(8, np.float32)
    run(s, [x, y]).close()
    assert np.array_equal(y, x.sum(1))
    s.close()


if __name__ == "__main__":
    globals()["scenario_" + sys.argv[1]]()
    print("ok", sys.argv[1])
