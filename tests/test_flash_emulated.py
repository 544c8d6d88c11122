"""The flash-attention kernels executed on the host, lane by lane (no GPU).

tests/emu/wave_emu.h stands in for the HIP runtime header: the .hip sources of
byteir_amd/csrc/flash_attn are compiled unchanged by a host compiler, a launch runs the grid's
workgroups one after the other, every lane is a fiber, and the cross-lane operations (MFMA, the
transposing LDS read, ballot, lane permutes, barriers) are rendezvous points that apply the
documented register layouts.  What that buys:

* the kernels' logic -- tiling, masks, online softmax, the backward's five products, grouped
  heads and their partial sums, the key-axis split, the cache append and the decode kernel --
  is checked against plain float32 attention without a GPU;
* bounds: tensors that end at (or begin behind) a protected page, buffer loads that apply the
  hardware's range check and must then land inside a tensor.  Every workgroup of the forward,
  D, dK/dV, group-sum and dQ launches of the two ragged shapes that once ran in a session which
  ended in a GPU memory fault (b4 h64/16 s1100 causal d64; b2 h64 sq2100 sk1500 d64) was executed
  this way, with the guard page at either end: no stray access (about 6 CPU-minutes per
  shape and placement; the test below repeats a sample of the workgroups).

The emulation says nothing about timing, and nothing about what the compiler makes of the
sources for the GPU."""
import os

import numpy as np
import pytest
import torch

import emu_util as E

ATOL = 2e-2

pytestmark = pytest.mark.skipif(not (os.path.exists(E.LIB) or os.path.exists("/opt/rocm/llvm/bin/clang++")),
                                reason="no host clang to build the emulated library with")


def reference(q, k, v, do, scale, window):
    """float32 attention with autograd -> (o, lse, dq, dk, dv)."""
    b, sq, h, d = q.shape
    sk, hk = k.shape[1], k.shape[2]
    qf, kf, vf = (t.float().detach().requires_grad_(True) for t in (q, k, v))
    kx, vx = kf.repeat_interleave(h // hk, 2), vf.repeat_interleave(h // hk, 2)
    s = torch.einsum("bqhd,bkhd->bhqk", qf, kx) * scale
    i = torch.arange(sq)[:, None] + (sk - sq)
    j = torch.arange(sk)[None, :]
    mask = torch.zeros(sq, sk, dtype=torch.bool)
    if window[1] >= 0:
        mask |= j > i + window[1]
    if window[0] >= 0:
        mask |= j < i - window[0]
    s = s.masked_fill(mask, float("-inf"))
    p = torch.nan_to_num(torch.softmax(s, -1))  # rows that see no key: zeros
    o = torch.einsum("bhqk,bkhd->bqhd", p, vx)
    if do is None:
        return o.detach(), torch.logsumexp(s.detach(), -1), None, None, None
    o.backward(do.float())
    return o.detach(), torch.logsumexp(s.detach(), -1), qf.grad, kf.grad, vf.grad


def randn(shape, dtype, gen):
    return torch.randn(shape, generator=gen).to(dtype)


CASES = [
    # b, sq, sk, h, h_k, d, window
    (1, 128, 128, 2, 2, 64, (-1, 0)),
    (1, 200, 333, 2, 1, 128, (-1, -1)),     # grouped heads, ragged, head_dim 128 (O staged through LDS)
    (1, 257, 130, 2, 2, 128, (-1, 0)),      # head_dim 128 backward without a head group: dK / dV staged through LDS
    (2, 77, 150, 2, 2, 32, (20, 5)),        # sliding window, surplus loader threads at head_dim 32
    (1, 300, 260, 4, 2, 64, (-1, 0)),       # more queries than keys, causal: rows that see no key
    (1, 100, 100, 1, 1, 96, (-1, 0)),       # a head_dim without a tuned kernel
    (1, 200, 300, 8, 2, 64, (-1, 0)),       # backward shares a head group out over workgroups (partials + group sum)
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_emulated_forward_and_backward_match_float32_attention(case, dtype):
    b, sq, sk, h, hk, d, window = case
    gen = torch.Generator().manual_seed(sq + sk + d)
    q, k, v, do = randn((b, sq, h, d), dtype, gen), randn((b, sk, hk, d), dtype, gen), randn((b, sk, hk, d), dtype, gen), randn((b, sq, h, d), dtype, gen)
    scale = 1.0 / np.sqrt(d)
    o, lse = E.fwd(q, k, v, scale, window)
    dq, dk, dv = E.bwd(do, q, k, v, o, lse, scale, window)
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = reference(q, k, v, do, scale, window)
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    for name, got, want in (("o", o, o_ref), ("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
        err = (got.float() - want).abs()
        assert bool(torch.all(err <= ATOL + ulp * want.abs())), (name, case, float(err.max()))
    seen = torch.isfinite(lse_ref)
    assert torch.equal(torch.isposinf(lse), ~seen)  # a row without keys: LSE = +inf, O = 0
    # head_dim 128 sums the rounded P (v_dot2c): with bf16 that moves the LSE of a row with few
    # keys by up to one rounding of its largest term, 2^-9
    assert float((lse[seen] - lse_ref[seen]).abs().max()) <= (4e-3 if d == 128 and dtype == torch.bfloat16 else 1e-3)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes_forward_and_backward_under_guarded_tensors(seed):
    """Head dimensions with and without a tuned kernel, one to three key/value heads with groups
    of one to four, lengths around the tile sizes, all window forms, both dtypes; every tensor
    guarded at a random end.  (A sweep of 960 such cases was run once: none faulted; four exceeded
    these bounds against float32 arithmetic, all bf16: the LSE at head_dim 128 on rows that see 7
    or 26 keys, by 2.1e-3 (the rounded-P row sum), and dK / dV of five keys summed over 500-1000
    query rows of bf16-rounded P and dS, by 0.05-0.07 on values of magnitude 10-20.)"""
    rng = np.random.default_rng(seed)
    for it in range(8):
        d = int(rng.choice([32, 64, 128, 40, 96, 160]))
        hk = int(rng.choice([1, 2, 3]))
        h = hk * int(rng.choice([1, 2, 4]))
        b = int(rng.choice([1, 2]))
        sq = int(rng.choice([1, 7, 64, 65, 129, 200, 257]))
        sk = int(rng.choice([1, 33, 64, 130, 255, 300, 513]))
        window = [(-1, -1), (-1, 0), (int(rng.integers(0, 80)), 0), (int(rng.integers(0, 60)), int(rng.integers(0, 60))),
                  (-1, int(rng.integers(0, 50)))][int(rng.integers(0, 5))]
        dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
        at_end = bool(rng.integers(0, 2))
        gen = torch.Generator().manual_seed(seed * 100 + it)
        G = lambda s, t=dtype: E.guarded(s, t, at_end)
        q, k, v, do = (G(s).copy_(randn(s, dtype, gen)) for s in ((b, sq, h, d), (b, sk, hk, d), (b, sk, hk, d), (b, sq, h, d)))
        scale = 1.0 / np.sqrt(d)
        case = (b, sq, sk, h, hk, d, window, dtype, at_end)
        ru = lambda x, m: -(-x // m) * m
        o, lse = E.fwd(q, k, v, scale, window, out=(G(q.shape), G((b, h, sq), torch.float32)))
        dq, dk, dv = E.bwd(do, q, k, v, o, lse, scale, window,
                           out=(G(q.shape), G(k.shape), G(v.shape), G((b, h, ru(sq, 128)), torch.float32),
                                G((b, ru(sq, 128), h, ru(d, 32)), torch.float32)))
        o_ref, lse_ref, dq_ref, dk_ref, dv_ref = reference(q, k, v, do, scale, window)
        ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
        for name, got, want in (("o", o, o_ref), ("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
            err = (got.float() - want).abs()
            assert bool(torch.all(err <= ATOL + 2 * ulp * want.abs())), (name, case, float(err.max()))
        seen = torch.isfinite(lse_ref)
        assert torch.equal(torch.isposinf(lse), ~seen), case
        assert not seen.any() or float((lse[seen] - lse_ref[seen]).abs().max()) <= 4e-3, case


@pytest.mark.parametrize("case", [
    # b, sq, sk (cache rows), h, h_k, d, appended rows
    (2, 1, 300, 4, 2, 128, 1),      # decode kernel, head group in one score tile
    (3, 1, 1500, 8, 2, 64, 1),      # ... with the keys split over workgroups and the merge kernel
    (2, 3, 900, 8, 2, 32, 3),
    (1, 70, 400, 2, 2, 64, 70),     # a prompt chunk: forward kernel with a per-batch key count
    (1, 1, 600, 2, 2, 80, 1),       # a head_dim without a tuned kernel
])
def test_emulated_cache_call_appends_and_attends(case):
    b, sq, sk, h, hk, d, n_new = case
    dtype = torch.float16
    gen = torch.Generator().manual_seed(sk + d)
    q = randn((b, sq, h, d), dtype, gen)
    kc, vc = randn((b, sk, hk, d), dtype, gen), randn((b, sk, hk, d), dtype, gen)
    kn, vn = randn((b, n_new, hk, d), dtype, gen), randn((b, n_new, hk, d), dtype, gen)
    lens = torch.tensor([sk - n_new - 7 * i for i in range(b)], dtype=torch.int32)
    kc0, vc0 = kc.clone(), vc.clone()
    o, lse = E.kvcache(q, kc, vc, kn, vn, lens, 1.0 / np.sqrt(d), (-1, 0))
    for bi in range(b):
        at, n = int(lens[bi]), int(lens[bi]) + n_new
        kk, vv = kc0[bi].clone(), vc0[bi].clone()
        kk[at:n], vv[at:n] = kn[bi], vn[bi]
        assert torch.equal(kc[bi], kk) and torch.equal(vc[bi], vv)  # appended in place, nothing else touched
        o_ref, lse_ref, *_ = reference(q[bi:bi + 1], kk[None, :n], vv[None, :n], None, 1.0 / np.sqrt(d), (-1, 0))
        assert float((o[bi].float() - o_ref[0]).abs().max()) <= ATOL
        assert float((lse[bi] - lse_ref[0]).abs().max()) <= 1e-3


@pytest.mark.parametrize("case", [
    (1, 300, 700, 2, 2, 64, (-1, 0), torch.bfloat16),
    (1, 300, 700, 2, 1, 128, (-1, -1), torch.float16),
    (1, 300, 500, 2, 2, 96, (-1, 0), torch.bfloat16),
])
def test_results_do_not_depend_on_how_far_the_waves_run_apart(case):
    """A missing barrier shows as a result that depends on the order in which the waves of a
    workgroup advance.  The emulator's default is round robin; here a randomly picked wave runs
    up to 7 or 400 steps in a row, which lets it get as far ahead as the kernels' barriers
    permit (several tiles of the LDS ring, if they permitted it).  Forward and backward must be
    bit-identical to the round-robin run.  (With the tile barrier of the forward kernel taken
    out, the same comparison fails with differences of 0.4-0.6 in O: the check does bite.)"""
    b, sq, sk, h, hk, d, window, dtype = case
    gen = torch.Generator().manual_seed(5)
    q, k, v, do = (randn(s, dtype, gen) for s in ((b, sq, h, d), (b, sk, hk, d), (b, sk, hk, d), (b, sq, h, d)))
    scale = 1.0 / np.sqrt(d)
    bits = lambda t: t.view(torch.int16) if t.dtype != torch.float32 else t.view(torch.int32)
    try:
        E.schedule(1, 0)
        o0, lse0 = E.fwd(q, k, v, scale, window)
        g0 = E.bwd(do, q, k, v, o0, lse0, scale, window)
        for burst, seed in ((7, 3), (400, 2)):
            E.schedule(burst, seed)
            o1, lse1 = E.fwd(q, k, v, scale, window)
            g1 = E.bwd(do, q, k, v, o1, lse1, scale, window)
            for a, c in zip((o0, lse0, *g0), (o1, lse1, *g1)):
                assert torch.equal(bits(a), bits(c)), (case, burst)
    finally:
        E.schedule(1, 0)


@pytest.mark.parametrize("d", [64, 80, 128])
def test_emulated_calls_without_keys_or_without_queries(d):
    """seqlen_k = 0: O = 0, LSE = +inf, dQ = 0 (flash_fwd_kernel.h:70-104); seqlen_q = 0: nothing
    to write forward, dK = dV = 0.  Guarded tensors: the empty side has no bytes to touch."""
    b, h, dtype = 2, 4, torch.float16
    gen = torch.Generator().manual_seed(d)
    G = lambda s, t=dtype: E.guarded(s, t)
    for sq in (3, 200):
        q, do = G((b, sq, h, d)).copy_(randn((b, sq, h, d), dtype, gen)), G((b, sq, h, d)).copy_(randn((b, sq, h, d), dtype, gen))
        k, v = G((b, 0, h, d)), G((b, 0, h, d))
        o, lse = E.fwd(q, k, v, 0.3, (-1, -1), out=(G(q.shape).fill_(7.0), G((b, h, sq), torch.float32)))
        assert bool((o == 0).all()) and bool(torch.isposinf(lse).all())
        dq, dk, dv = E.bwd(do, q, k, v, o, lse, 0.3, (-1, -1))
        assert bool((dq == 0).all()) and dk.numel() == 0 and dv.numel() == 0
    sk = 150
    q, do = G((b, 0, h, d)), G((b, 0, h, d))
    k, v = G((b, sk, h, d)).copy_(randn((b, sk, h, d), dtype, gen)), G((b, sk, h, d)).copy_(randn((b, sk, h, d), dtype, gen))
    o, lse = E.fwd(q, k, v, 0.3, (-1, 0), out=(G(q.shape), G((b, h, 0), torch.float32)))
    out = (G(q.shape), G(k.shape).fill_(7.0), G(v.shape).fill_(7.0), G((b, h, 0), torch.float32), G((b, 0, h, d), torch.float32))
    dq, dk, dv = E.bwd(do, q, k, v, o, lse, 0.3, (-1, 0), out=out)
    assert dq.numel() == 0 and bool((dk == 0).all()) and bool((dv == 0).all())


def test_scratch_in_the_callers_workspace_gives_the_same_bits():
    """The key-axis split of the forward (few query blocks, many keys) and the partial dK / dV of
    a shared-out head group, with the scratch in a guarded, poisoned workspace of exactly the
    size the *_workspace_bytes query names, against the calls that take their own scratch;
    the backward also without any dq_accum to borrow from."""
    from byteir_amd import ops
    bits = lambda t: t.view(torch.int16 if t.element_size() == 2 else torch.int32)
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(4)
    q, k, v = randn((1, 64, 2, 64), dtype, gen), randn((1, 1100, 2, 64), dtype, gen), randn((1, 1100, 2, 64), dtype, gen)
    o, lse, rng = torch.empty_like(q), torch.empty((1, 2, 64), dtype=torch.float32), torch.zeros(2, dtype=torch.int64)
    blob = ops.pack_flash_args(q, k, v, o, 0.125, (-1, 0), 0.0)
    need = E.workspace_bytes("fwd", blob, dtype)
    assert need > 0
    ws = E.guarded((need,), torch.uint8).fill_(0xFF)
    o0, l0 = E.fwd(q, k, v, 0.125, (-1, 0))
    E._call("fwd", [q, k, v, rng, o, lse, None], blob, dtype, workspace=ws)
    assert torch.equal(bits(o0), bits(o)) and torch.equal(l0, lse)
    # backward, eight query heads on two key/value heads: the group is shared out over workgroups
    b, s_, h, hk, d = 1, 300, 8, 2, 64
    q, k, v, do = randn((b, s_, h, d), dtype, gen), randn((b, s_, hk, d), dtype, gen), randn((b, s_, hk, d), dtype, gen), randn((b, s_, h, d), dtype, gen)
    o, lse = E.fwd(q, k, v, 0.125, (-1, 0))
    g0 = E.bwd(do, q, k, v, o, lse, 0.125, (-1, 0))  # partials in dq_accum
    blob = ops.pack_flash_args(q, k, v, o, 0.125, (-1, 0), 0.0)
    need = E.workspace_bytes("bwd", blob, dtype, 0)
    assert need > 0 and E.workspace_bytes("bwd", blob, dtype, 1 << 30) == 0
    like = lambda t: torch.empty_strided(t.shape, t.stride(), dtype=t.dtype)
    for ws in (E.guarded((need,), torch.uint8).fill_(0xFF), None):  # the caller's workspace; the library's own allocation
        dq, dk, dv, dsm = like(q), like(k), like(v), torch.empty((b, h, 384), dtype=torch.float32)
        E._call("bwd", [do, q, k, v, o, lse, rng, dq, dk, dv, dsm, None], blob, dtype, workspace=ws)
        for a, c in zip(g0, (dq, dk, dv)):
            assert torch.equal(bits(a), bits(c))


@pytest.mark.parametrize("layout,case", [
    ("packed_qkv", (2, 192, 192, 4, 4, 64, (-1, 0))),      # q, k, v are slices of one [b, s, 3, h, d] tensor
    ("packed_qkv", (1, 130, 130, 2, 2, 96, (-1, -1))),
    ("bhsd", (2, 160, 224, 4, 4, 128, (-1, 0))),           # [b, h, s, d] storage viewed as [b, s, h, d]
    ("bhsd", (1, 100, 300, 3, 3, 32, (20, 5))),
])
def test_emulated_calls_follow_the_strides_of_their_tensors(layout, case):
    """The blob carries batch, row and head strides: tensors that are views of larger ones."""
    b, sq, sk, h, hk, d, window = case
    dtype = torch.float16
    gen = torch.Generator().manual_seed(sq + d)
    q, k, v, do = randn((b, sq, h, d), dtype, gen), randn((b, sk, hk, d), dtype, gen), randn((b, sk, hk, d), dtype, gen), randn((b, sq, h, d), dtype, gen)
    if layout == "packed_qkv":
        pk = torch.empty((b, sq, 3, h, d), dtype=dtype)
        pk[:, :, 0], pk[:, :, 1], pk[:, :, 2] = q, k, v
        sq_, sk_, sv_ = pk[:, :, 0], pk[:, :, 1], pk[:, :, 2]
        o_buf = torch.full((b, sq, 2, h, d), 7.0, dtype=dtype)
        o_view = o_buf[:, :, 1]
    else:
        tr = lambda x: x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        sq_, sk_, sv_ = tr(q), tr(k), tr(v)
        o_buf = torch.full((b, h, sq, d), 7.0, dtype=dtype)
        o_view = o_buf.permute(0, 2, 1, 3)
    scale = 1.0 / np.sqrt(d)
    o, lse = E.fwd(sq_, sk_, sv_, scale, window, out=(o_view, torch.empty((b, h, sq), dtype=torch.float32)))
    do_s = torch.empty_strided(o.shape, o.stride(), dtype=dtype).copy_(do)  # dO is addressed with the strides of O
    dq, dk, dv = E.bwd(do_s, sq_, sk_, sv_, o, lse, scale, window)
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = reference(q, k, v, do, scale, window)
    for name, got, want in (("o", o, o_ref), ("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
        assert float((got.float() - want).abs().max()) <= ATOL, (name, case)
    if layout == "packed_qkv":
        assert bool((o_buf[:, :, 0] == 7.0).all())  # the neighbouring slice of the output's storage is untouched


@pytest.mark.parametrize("code", ["f16", "bf16"])
@pytest.mark.parametrize("case", [
    # b, sq, sk, h, h_k, d, window, p_dropout
    (2, 128, 128, 2, 2, 64, (-1, 0), 0.1),
    (1, 200, 333, 2, 2, 128, (-1, -1), 0.5),
    (1, 130, 260, 4, 2, 96, (40, 30), 0.2),    # grouped heads: dropout streams are per query head
])
def test_emulated_dropout_is_the_reference_function_of_seed_offset_and_position(case, code):
    """Dropout (Philox4x32-7 on (seed, offset, batch, head, 16 x 32 block), keep when the byte is
    at most floor(255 p_keep)) against the oracle's thread-by-thread restatement: forward and
    backward with the same rng_state."""
    import oracle
    b, sq, sk, h, hk, d, window, p_drop = case
    ocode = oracle.F16 if code == "f16" else oracle.BF16
    rng = np.random.default_rng(sum(case[:6]))
    mk = lambda shape: oracle.from_f32(rng.standard_normal(shape).astype(np.float32), ocode)
    q, k, v, do = mk((b, sq, h, d)), mk((b, sk, hk, d)), mk((b, sk, hk, d)), mk((b, sq, h, d))
    to_t = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16) if a.dtype == np.uint16 else torch.from_numpy(a.copy())
    to_np = lambda t: t.view(torch.int16).numpy().view(np.uint16) if t.dtype == torch.bfloat16 else t.numpy()
    state = (0x9E3779B97F4A7C15, 0x1_0000_0003)
    scale = 1.0 / np.sqrt(d)
    tq, tk, tv, tdo = to_t(q), to_t(k), to_t(v), to_t(do)
    o, lse = E.fwd(tq, tk, tv, scale, window, p_dropout=p_drop, rng_state=state)
    _, lse_ref, o32 = oracle.flash_fwd(q, k, v, scale, window, round_p=False, p_dropout=p_drop, rng_state=state)
    assert np.abs(o.float().numpy() - o32).max() <= ATOL
    seen = ~np.isposinf(lse_ref)
    assert np.abs(lse.numpy()[seen] - lse_ref[seen]).max() <= 4e-3
    dq, dk, dv = E.bwd(tdo, tq, tk, tv, o, lse, scale, window, p_dropout=p_drop, rng_state=state)
    rq, rk, rv, _ = oracle.flash_bwd(do, q, k, v, to_np(o), lse.numpy(), scale, window, round_p=False, p_dropout=p_drop, rng_state=state)
    for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        assert np.abs(got.float().numpy() - oracle.to_f32(want)).max() <= ATOL, name


def test_a_tensor_that_is_too_short_is_reported_with_the_workgroup_and_thread():
    """Negative controls: K one row short (a buffer load passes the descriptor's range check and
    then lies outside every tensor) and O one row short (a plain store runs into the protected
    page)."""
    from byteir_amd import ops
    b, sq, sk, h, d = 1, 256, 320, 2, 64
    gen = torch.Generator().manual_seed(1)
    mk = lambda rows, at_end=True: E.guarded((b, rows, h, d), torch.float16, at_end).copy_(randn((b, rows, h, d), torch.float16, gen))
    q, k, v = mk(sq), mk(sk), mk(sk)
    o, lse, rng = E.guarded((b, sq, h, d), torch.float16), E.guarded((b, h, sq), torch.float32), torch.zeros(2, dtype=torch.int64)
    blob = ops.pack_flash_args(q, k, v, o, 0.125, (-1, -1), 0.0)
    E._call("fwd", [q, k, v, rng, o, lse, None], blob, torch.float16)  # as declared: fine
    k_short = mk(sk - 1)
    with pytest.raises(E.EmuFault, match=r"outside every tensor.*workgroup \(\d+, 0, 0\) of \(\d+, 1, 1\), thread \d+"):
        E._call("fwd", [q, k_short, v, rng, o, lse, None], blob, torch.float16)
    o_short = E.guarded((b, sq - 1, h, d), torch.float16)
    with pytest.raises(E.EmuFault, match=r"memory access outside every tensor.*workgroup"):
        E._call("fwd", [q, k, v, rng, o_short, lse, None], blob, torch.float16)
    E._call("fwd", [q, k, v, rng, o, lse, None], blob, torch.float16)  # and the library still works afterwards


@pytest.mark.parametrize("at_end", [True, False])
@pytest.mark.parametrize("shape", [
    (4, 1100, 1100, 64, 16, 64, (-1, 0)),
    (2, 2100, 1500, 64, 64, 64, (-1, -1)),
])
def test_a_sample_of_the_workgroups_of_the_two_ragged_shapes_stays_in_bounds(shape, at_end):
    """Every launch of a forward and a backward call (forward; D, dK/dV, group sum, dQ) with one
    workgroup in 331 executed (the first of every launch, and ids 330 modulo 331), all tensors
    guarded.  The results are not looked at: with most workgroups left out the backward
    reads unwritten intermediates, which cannot change an address."""
    b, sq, sk, h, hk, d, window = shape
    gen = torch.Generator().manual_seed(3)
    dt = torch.bfloat16
    g = lambda s, t=dt: E.guarded(s, t, at_end)
    q, k, v, do = (g(s).copy_(randn(s, dt, gen)) for s in ((b, sq, h, d), (b, sk, hk, d), (b, sk, hk, d), (b, sq, h, d)))
    o, lse = g((b, sq, h, d)).zero_(), g((b, h, sq), torch.float32).fill_(12.0)
    ru = lambda x, m: -(-x // m) * m
    out = (g(q.shape), g(k.shape), g(v.shape), g((b, h, ru(sq, 128)), torch.float32).zero_(), g((b, ru(sq, 128), h, ru(d, 32)), torch.float32))
    L = E.lib()
    try:
        for stride in (331,):
            for phase in (0, stride - 1):
                E.select(stride, phase)
                L.fa_emu_reset()
                E.fwd(q, k, v, 1.0 / np.sqrt(d), window, out=(o, lse))
                n_fwd = L.fa_emu_blocks_run()
                E.bwd(do, q, k, v, o, lse, 1.0 / np.sqrt(d), window, out=out)
                assert n_fwd >= 1 and L.fa_emu_blocks_run() - n_fwd >= 10
    finally:
        E.select(1, 0)
