"""Scratch through the caller's workspace: the *_workspace_bytes queries and *_ws entry points of
the flash-attention library and of the inner-axis softmax.  A call with a workspace must give the
bits of the call without one (same kernels, same split); the backward's partial dK / dV must land
correctly whether they live in dq_accum, in the workspace, in both, or in the library's own
stream-ordered allocation (dq_accum absent or too small)."""
import numpy as np
import pytest
import torch

import oracle
from byteir_amd import ops

pytestmark = pytest.mark.gpu


def bits(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def ws_tensor(n, poison=True):
    w = torch.empty(max(n, 1), dtype=torch.uint8, device="cuda")
    if poison:
        w.fill_(0xFF)  # NaN patterns: anything read before it is written would show
    return w


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_forward_split_partials_in_the_callers_workspace(dtype):
    # few query blocks against many keys: the key axis is split over workgroups
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn((1, 256, 8, 128), generator=g, device="cuda").to(dtype)
    k, v = (torch.randn((1, 8192, 8, 128), generator=g, device="cuda").to(dtype) for _ in range(2))
    o = torch.empty_like(q)
    need = ops.flash_attn_workspace_bytes("fwd", dtype, ops.pack_flash_args(q, k, v, o, 0.088, (-1, 0)))
    assert need > 0
    o0, l0 = ops.flash_attn_fwd(q, k, v, 0.088, (-1, 0))
    o1, l1 = ops.flash_attn_fwd(q, k, v, 0.088, (-1, 0), workspace=ws_tensor(need))
    o2, l2 = ops.flash_attn_fwd(q, k, v, 0.088, (-1, 0), workspace=ws_tensor(need // 2))  # too small: own allocation
    torch.cuda.synchronize()
    assert torch.equal(bits(o0), bits(o1)) and torch.equal(l0, l1)
    assert torch.equal(bits(o0), bits(o2)) and torch.equal(l0, l2)
    # the benchmark's forward shapes take no scratch at all
    qq = torch.empty((4, 2048, 32, 128), dtype=dtype, device="meta")
    assert ops.flash_attn_workspace_bytes("fwd", dtype, ops.pack_flash_args(qq, qq, qq, qq, 0.088, (-1, 0))) == 0


def test_decode_split_partials_in_the_callers_workspace():
    g = torch.Generator(device="cuda").manual_seed(4)
    b, h, hk, d, cap = 2, 16, 4, 128, 4096
    q = torch.randn((b, 1, h, d), generator=g, device="cuda").half()
    kc, vc = (torch.randn((b, cap, hk, d), generator=g, device="cuda").half() for _ in range(2))
    kn, vn = (torch.randn((b, 1, hk, d), generator=g, device="cuda").half() for _ in range(2))
    lens = torch.tensor([4000, 17], dtype=torch.int32, device="cuda")
    o = torch.empty_like(q)
    need = ops.flash_attn_workspace_bytes("kvcache", q.dtype, ops.pack_flash_kvcache_args(q, kc, vc, kn, vn, o, 0.088, (-1, -1)))
    assert need > 0
    kc1, vc1 = kc.clone(), vc.clone()
    o0, l0 = ops.flash_attn_kvcache(q, kc, vc, kn, vn, lens, 0.088)
    o1, l1 = ops.flash_attn_kvcache(q, kc1, vc1, kn, vn, lens, 0.088, workspace=ws_tensor(need))
    torch.cuda.synchronize()
    assert torch.equal(bits(o0), bits(o1)) and torch.equal(l0, l1) and torch.equal(bits(kc), bits(kc1)) and torch.equal(bits(vc), bits(vc1))


# grouped heads on a small grid: the dK/dV workgroups of a key/value head are shared out and write
# float partials.  (b, s, h, h_k, d, causal)
GROUPED = [(1, 2048, 8, 2, 64, True), (1, 2048, 8, 2, 128, True), (1, 1024, 8, 2, 96, False)]


@pytest.mark.parametrize("where", ["dq_accum", "none", "workspace", "workspace_too_small"])
@pytest.mark.parametrize("case", GROUPED)
def test_backward_partials_wherever_they_live(case, where):
    b, s, h, hk, d, causal = case
    window = (-1, 0) if causal else (-1, -1)
    scale = 1.0 / np.sqrt(d)
    rng = np.random.default_rng(b + s + h + d)
    mk = lambda *shape: oracle.from_f32(rng.standard_normal(shape).astype(np.float32), oracle.BF16)
    q, k, v, do = mk(b, s, h, d), mk(b, s, hk, d), mk(b, s, hk, d), mk(b, s, h, d)
    dev = lambda a: torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    tq, tk, tv, tdo = dev(q), dev(k), dev(v), dev(do)
    to_, tlse = ops.flash_attn_fwd(tq, tk, tv, scale, window)
    dq, dk, dv, dsm, accum, rs = ops.flash_attn_bwd_buffers(tq, tk, tv)
    blob = ops.pack_flash_args(tq, tk, tv, to_, scale, window)
    full = accum.numel() * 4
    need_none = ops.flash_attn_workspace_bytes("bwd", tq.dtype, blob, 0)
    need_full = ops.flash_attn_workspace_bytes("bwd", tq.dtype, blob, full)
    assert need_none > 0, "the case is meant to split"
    one = need_none // 2  # dK partials and dV partials are the same size
    assert need_full in (0, one, 2 * one)  # a dq_accum of the reference's size holds both, one, or neither
    # (the size of dq_accum is not an argument of the reference's ABI: the library takes it to be
    # the reference's [b, seqlen_q_rounded, h, d_rounded] floats whenever the pointer is given)
    ws = None
    if where == "none":                 # partials in the library's own stream-ordered allocation
        accum = None
    elif where == "workspace":          # no dq_accum, everything in the caller's workspace
        accum, ws = None, ws_tensor(need_none)
    elif where == "workspace_too_small":  # ignored: falls back to the own allocation
        accum, ws = None, ws_tensor(one)
    gq, gk, gv = ops.flash_attn_bwd(tdo, tq, tk, tv, to_, tlse, scale, window, out=(dq, dk, dv, dsm, accum, rs), workspace=ws)
    torch.cuda.synchronize()
    rq, rk, rv, _ = oracle.flash_bwd(do, q, k, v, to_.view(torch.int16).cpu().numpy().view(np.uint16), tlse.cpu().numpy(), scale, window, round_p=False)
    for name, got, ref in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        ref = oracle.to_f32(ref)
        err = np.abs(got.float().cpu().numpy() - ref)
        tol = 2e-2 + 2.0 ** -8 * np.abs(ref)
        assert np.all(err <= tol), f"{name} ({where}): worst absolute error {err.max():.4f}"
    # and the same bits as the default placement
    dq0, dk0, dv0 = ops.flash_attn_bwd(tdo, tq, tk, tv, to_, tlse, scale, window)
    torch.cuda.synchronize()
    assert torch.equal(bits(gk), bits(dk0)) and torch.equal(bits(gv), bits(dv0)) and torch.equal(bits(gq), bits(dq0))


def test_inner_axis_softmax_partials_in_the_callers_workspace():
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((16, 50000, 128), generator=g, device="cuda")
    need = ops.softmax_workspace_bytes(x, axis=1)
    assert need > 0
    y0 = ops.softmax(x, axis=1)
    y1 = ops.softmax(x, axis=1, workspace=ws_tensor(need))
    torch.cuda.synchronize()
    assert torch.equal(bits(y0), bits(y1))
    ref = torch.softmax(x.double(), dim=1)
    assert float((y1.double() - ref).abs().max()) <= 1e-6
    assert ops.softmax_workspace_bytes(torch.empty((32768, 4096), dtype=torch.bfloat16, device="meta")) == 0


def test_custom_op_workspace_comes_from_the_frames_allocator(tmp_path):
    """Through the runtime the decode call's split partials are a per-frame workspace: asked
    once when the frame is set up, allocated by the session's allocator, freed with the frame."""
    from byteir_amd import brt
    allocs, live = [], {}

    def alloc(n):
        p = torch.cuda.caching_allocator_alloc(n)
        live[p] = n
        allocs.append(n)
        return p

    def free(p):
        del live[p]
        torch.cuda.caching_allocator_delete(p)

    b, h, hk, d, cap = 2, 16, 4, 128, 4096
    g = torch.Generator(device="cuda").manual_seed(6)
    q = torch.randn((b, 1, h, d), generator=g, device="cuda").half()
    kc, vc = (torch.randn((b, cap, hk, d), generator=g, device="cuda").half() for _ in range(2))
    kn, vn = (torch.randn((b, 1, hk, d), generator=g, device="cuda").half() for _ in range(2))
    lens = torch.tensor([4000, 17], dtype=torch.int32, device="cuda")
    o = torch.empty_like(q)
    lse = torch.empty((b, h, 1), device="cuda")
    blob = ops.pack_flash_kvcache_args(q, kc, vc, kn, vn, o, 0.088, (-1, -1))
    need = ops.flash_attn_workspace_bytes("kvcache", q.dtype, blob)
    import struct
    ints = list(struct.unpack("<24q", blob[:192])) + [struct.unpack("<f", blob[192:196])[0]] + list(struct.unpack("<6q", blob[196:244]))
    extra = ", ".join(f"{x} : f32" if isinstance(x, float) else f"{x} : i64" for x in ints)
    mr = lambda t, ty: f'memref<{"x".join(str(n) for n in t.shape)}x{ty}, "cuda">'
    types = [mr(q, "f16"), mr(kc, "f16"), mr(vc, "f16"), mr(kn, "f16"), mr(vn, "f16"), mr(lens, "i32"), mr(o, "f16"), mr(lse, "f32")]
    names = ["q", "kc", "vc", "kn", "vn", "lens", "o", "lse"]
    sig = ", ".join(f'%{n} : {t} {{byre.argname = "{n}", byre.argtype = {2 if n in ("o", "lse", "kc", "vc") else 1}: i32}}' for n, t in zip(names, types))
    text = f"""func.func @decode({sig}) attributes {{byre.entry_point}} {{
      "byre.custom"({", ".join("%" + n for n in names)}) {{callee = "custom", lib_path = "libflash_attn.so", api_name = "run_flash_attn_kvcache", version = "2.5.3", extra_args = [{extra}]}} : ({", ".join(types)}) -> ()
      return }}"""
    s = brt.Session(device="ROCM", alloc_func=alloc, free_func=free)
    try:
        s.load_from_memory(text)
        req = s.new_request_context(torch.cuda.current_stream().cuda_stream)
        kc1, vc1 = kc.clone(), vc.clone()
        for i, t in enumerate((q, kc1, vc1, kn, vn, lens, o, lse)):
            req.bind_arg(i, t.data_ptr())
        req.finish_io_binding()
        assert allocs == []
        req.run(); req.run(); req.sync()
        assert allocs == [need]
        o0, l0 = ops.flash_attn_kvcache(q, kc, vc, kn, vn, lens, 0.088)
        torch.cuda.synchronize()
        assert torch.equal(bits(o), bits(o0)) and torch.equal(lse, l0)
        req.close()
        assert live == {}
    finally:
        s.close()
