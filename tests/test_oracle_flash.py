"""Pins the flash-attention part of the CPU oracle: reference golden vectors, torch's CPU
scaled_dot_product_attention + autograd, scipy logsumexp, finite differences, blob bytes."""
import os
import struct

import numpy as np
import pytest
import torch
from scipy.special import logsumexp

import oracle


def load_golden(golden_dir):
    return {n: np.load(os.path.join(golden_dir, f"fa_{n}.npy")) for n in
            ("q", "k", "v", "dout", "out", "dq", "dk", "dv")}


def ulp_diff_f16(a, b):
    """distance in fp16 units-in-the-last-place (monotone integer mapping of the bits)"""
    def key(x):
        u = x.view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(a) - key(b))


def test_golden_inputs_are_the_documented_closed_form(golden_dir):
    # generate_flash_attn_ground_truth.py:23-25: arange(n, fp16)/30000, /40000, /50000
    g = load_golden(golden_dir)
    n = 128 * 3 * 32
    ar = torch.arange(n, dtype=torch.float16)
    for name, div in (("q", 30000), ("k", 40000), ("v", 50000)):
        want = (ar / div).numpy().reshape(1, 128, 3, 32)
        assert np.array_equal(g[name], want), name
    assert np.all(g["dout"] == np.float16(1 / 32))


def test_forward_against_reference_golden_vectors(golden_dir):
    g = load_golden(golden_dir)
    o, lse, _ = oracle.flash_fwd(g["q"], g["k"], g["v"], 0.5, window=(-1, 0))
    d = ulp_diff_f16(o, g["out"])
    # the reference test demands bit equality of its own kernel (flash_attn_fwd_test.cc:137-147);
    # summation order inside the CUDA kernel is not reproducible on a CPU, so allow one fp16 ulp
    assert d.max() <= 1, d.max()
    assert (d == 0).mean() > 0.97
    assert np.all(np.isfinite(lse))


def test_backward_against_reference_golden_vectors(golden_dir):
    g = load_golden(golden_dir)
    o, lse, _ = oracle.flash_fwd(g["q"], g["k"], g["v"], 0.5, window=(-1, 0))
    dq, dk, dv, _ = oracle.flash_bwd(g["dout"], g["q"], g["k"], g["v"], g["out"], lse, 0.5, window=(-1, 0))
    for name, got in (("dq", dq), ("dk", dk), ("dv", dv)):
        want = g[name].astype(np.float32)
        err = np.abs(got.astype(np.float32) - want)
        # <= 2 fp16 ulp of the value with an absolute floor for the exact zeros in dq's first row
        tol = 2 * 2.0 ** -10 * np.abs(want) + 2e-6
        assert np.all(err <= tol), (name, float((err / tol).max()))
    # the first query row attends to one key only, so dS = P*(dP - D) = 0 there exactly
    assert np.all(g["dq"][0, 0] == 0) and np.all(dq[0, 0] == 0)


def torch_sdpa(q, k, v, scale, causal):
    tq, tk, tv = (torch.tensor(t.astype(np.float32)).permute(0, 2, 1, 3).requires_grad_() for t in (q, k, v))
    sq, sk = q.shape[1], k.shape[1]
    mask = None
    if causal:  # bottom-right aligned, col <= row + sk - sq (lib/mask.h:171-172)
        i = torch.arange(sq)[:, None]
        j = torch.arange(sk)[None, :]
        mask = j <= i + sk - sq
    out = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=scale)
    return out, (tq, tk, tv)


@pytest.mark.parametrize("causal,sq,sk", [(False, 40, 72), (True, 64, 64), (True, 33, 80)])
def test_forward_matches_torch_sdpa_and_logsumexp(causal, sq, sk):
    rng = np.random.default_rng(8)
    b, h, d = 2, 3, 32
    q = rng.standard_normal((b, sq, h, d)).astype(np.float16)
    k = rng.standard_normal((b, sk, h, d)).astype(np.float16)
    v = rng.standard_normal((b, sk, h, d)).astype(np.float16)
    scale = 1 / np.sqrt(d)
    window = (-1, 0) if causal else (-1, -1)
    o, lse, o32 = oracle.flash_fwd(q, k, v, scale, window, round_p=False)
    want, _ = torch_sdpa(q, k, v, scale, causal)
    want = want.detach().permute(0, 2, 1, 3).numpy()
    np.testing.assert_allclose(o32, want, atol=2e-5, rtol=1e-4)
    # LSE: natural log of the sum over kept keys of exp(scale * q.k) (softmax.h:172)
    s = np.einsum("bihd,bjhd->bhij", q.astype(np.float64), k.astype(np.float64)) * scale
    if causal:
        i = np.arange(sq)[:, None]
        j = np.arange(sk)[None, :]
        s = np.where(j <= i + sk - sq, s, -np.inf)
    np.testing.assert_allclose(lse, logsumexp(s, axis=-1), atol=1e-4, rtol=1e-5)
    # reconstruct O from LSE: o_i = sum_j exp(s_ij - lse_i) v_j
    p = np.exp(s - lse[..., None].astype(np.float64))
    rec = np.einsum("bhij,bjhd->bihd", p, v.astype(np.float64))
    np.testing.assert_allclose(o32, rec, atol=1e-4)
    # rounding P to fp16 (the reference's arithmetic) stays within 2e-2 of plain float attention
    o_r, _, _ = oracle.flash_fwd(q, k, v, scale, window, round_p=True)
    assert np.abs(o_r.astype(np.float32) - want).max() < 2e-2


def test_fully_masked_rows_give_zero_and_inf():
    # causal with sq > sk: rows i < sq - sk keep no key -> O = 0, LSE = +inf
    # (flash_fwd_kernel.h:70-104, softmax.h:171-172)
    rng = np.random.default_rng(9)
    q = rng.standard_normal((1, 8, 1, 32)).astype(np.float16)
    k = rng.standard_normal((1, 5, 1, 32)).astype(np.float16)
    o, lse, _ = oracle.flash_fwd(q, k, k, 0.3, (-1, 0))
    assert np.all(o[0, :3] == 0) and np.all(np.isposinf(lse[0, 0, :3]))
    assert np.all(np.isfinite(lse[0, 0, 3:]))
    # row 3 keeps exactly key 0 -> O = v_0
    assert np.array_equal(o[0, 3, 0], k[0, 0, 0])


@pytest.mark.parametrize("causal", [False, True])
def test_backward_matches_torch_autograd(causal):
    rng = np.random.default_rng(10)
    b, h, d, sq, sk = 1, 2, 32, 48, 64
    q = rng.standard_normal((b, sq, h, d)).astype(np.float32)
    k = rng.standard_normal((b, sk, h, d)).astype(np.float32)
    v = rng.standard_normal((b, sk, h, d)).astype(np.float32)
    do = rng.standard_normal((b, sq, h, d)).astype(np.float32)
    scale = 0.2
    window = (-1, 0) if causal else (-1, -1)
    o, lse, _ = oracle.flash_fwd(q, k, v, scale, window, round_p=False)
    dq, dk, dv, D = oracle.flash_bwd(do, q, k, v, o, lse, scale, window, round_p=False)
    out, (tq, tk, tv) = torch_sdpa(q, k, v, scale, causal)
    out.backward(torch.tensor(do).permute(0, 2, 1, 3))
    for got, t in ((dq, tq), (dk, tk), (dv, tv)):
        np.testing.assert_allclose(got, t.grad.permute(0, 2, 1, 3).numpy(), atol=3e-5, rtol=1e-4)
    np.testing.assert_allclose(D, np.einsum("bihd,bihd->bhi", do, o), atol=1e-5)


def test_backward_finite_difference():
    rng = np.random.default_rng(11)
    q = rng.standard_normal((1, 6, 1, 32)).astype(np.float32)
    k = rng.standard_normal((1, 7, 1, 32)).astype(np.float32)
    v = rng.standard_normal((1, 7, 1, 32)).astype(np.float32)
    do = rng.standard_normal((1, 6, 1, 32)).astype(np.float32)
    scale = 0.25

    def loss(qq, kk, vv):  # float64 loss through plain numpy
        s = np.einsum("bihd,bjhd->bhij", qq, kk) * scale
        i = np.arange(6)[:, None]; j = np.arange(7)[None, :]
        s = np.where(j <= i + 1, s, -np.inf)
        p = np.exp(s - logsumexp(s, axis=-1, keepdims=True))
        return float((np.einsum("bhij,bjhd->bihd", p, vv) * do).sum())

    o, lse, _ = oracle.flash_fwd(q, k, v, scale, (-1, 0), round_p=False)
    dq, dk, dv, _ = oracle.flash_bwd(do, q, k, v, o, lse, scale, (-1, 0), round_p=False)
    q64, k64, v64 = (t.astype(np.float64) for t in (q, k, v))
    eps = 1e-5
    for arr, grad, which in ((q64, dq, 0), (k64, dk, 1), (v64, dv, 2)):
        for idx in [(0, 0, 0, 0), (0, 3, 0, 5), (0, 5, 0, 31)]:
            hi = [q64.copy(), k64.copy(), v64.copy()]; lo = [q64.copy(), k64.copy(), v64.copy()]
            hi[which][idx] += eps; lo[which][idx] -= eps
            fd = (loss(*hi) - loss(*lo)) / (2 * eps)
            assert abs(fd - grad[idx]) < 1e-4, (which, idx, fd, grad[idx])


def test_bf16_storage_path():
    rng = np.random.default_rng(12)
    b, s, h, d = 1, 64, 2, 64
    q32, k32, v32 = (rng.standard_normal((b, s, h, d)).astype(np.float32) for _ in range(3))
    q, k, v = (oracle.to_bf16_bits(t) for t in (q32, k32, v32))
    o, lse, o32 = oracle.flash_fwd(q, k, v, 0.125)
    want, _ = torch_sdpa(oracle.from_bf16_bits(q), oracle.from_bf16_bits(k), oracle.from_bf16_bits(v), 0.125, False)
    want = want.detach().permute(0, 2, 1, 3).numpy()
    assert np.abs(oracle.from_bf16_bits(o) - want).max() < 2e-2


def test_extra_args_blob_known_answer():
    # runtime/test/test_files/flash_attn_fwd.mlir:9 extra_args, packed as
    # OpAccessor::GetAttrAsVoidPtr does (op_accessor.cc:212-242): i64 -> 8 B, f32 -> 4 B
    fields = [12288] * 4 + [96] * 4 + [32] * 4 + [1, 3, 3, 32, 32, 0.5, 128, 128, 128, 128, 0.0, -1, 0]
    want = b"".join(struct.pack("<f", f) if isinstance(f, float) else struct.pack("<q", f) for f in fields)
    assert len(want) == 192
    a = oracle.fa_args(1, 128, 128, 3, 3, 32, 0.5, window=(-1, 0))
    blob = oracle.fa_pack_args(a)
    assert blob.tobytes() == want
    back = oracle.fa_unpack_args(blob)
    assert (back.seqlen_q, back.window_size_left, back.window_size_right, back.softmax_scale) == (128, -1, 0, 0.5)
    # strides of the causal fp16 benchmark configuration
    c4 = oracle.fa_args(4, 2048, 2048, 32, 32, 128, 1 / np.sqrt(128), window=(-1, 0))
    assert (c4.q_batch_stride, c4.q_row_stride, c4.q_head_stride) == (8388608, 4096, 128)


# ---- key/value cache (run_flash_attn_kvcache) -------------------------------------------------
def load_kv_golden(golden_dir):
    g = {n: np.load(os.path.join(golden_dir, f"fa_kv_{n}.npy")) for n in
         ("q", "knew", "vnew", "kcache", "vcache", "out", "kcache_out", "vcache_out", "seqlens")}
    return g


def test_kvcache_golden_inputs_are_the_documented_closed_form(golden_dir):
    # generate_flash_attn_ground_truth.py:56-74: arange/30000, /40000, /50000; 64 valid rows
    g = load_kv_golden(golden_dir)
    small, cache = torch.arange(2 * 1 * 3 * 32, dtype=torch.float16), torch.arange(2 * 128 * 3 * 32, dtype=torch.float16)
    assert np.array_equal(g["q"], (small / 30000).numpy().reshape(2, 1, 3, 32))
    assert np.array_equal(g["knew"], (small / 40000).numpy().reshape(2, 1, 3, 32))
    assert np.array_equal(g["vnew"], (small / 50000).numpy().reshape(2, 1, 3, 32))
    assert np.array_equal(g["kcache"], (cache / 40000).numpy().reshape(2, 128, 3, 32))
    assert np.array_equal(g["vcache"], (cache / 50000).numpy().reshape(2, 128, 3, 32))
    assert g["seqlens"].tolist() == [64, 64]


def test_kvcache_against_reference_golden_vectors(golden_dir):
    """SM80CUDATestFlashAttnKVCache.Basic (flash_attn_fwd_test.cc:183-330): output and both
    updated caches.  The caches must match exactly (a copy); the output within one fp16 ulp."""
    g = load_kv_golden(golden_dir)
    o, lse, kc, vc = oracle.flash_kvcache(g["q"], g["kcache"], g["vcache"], g["knew"], g["vnew"], g["seqlens"], 0.5)
    assert np.array_equal(kc, g["kcache_out"])
    assert np.array_equal(vc, g["vcache_out"])
    # only row 64 of each batch changed, and it now holds the new key / value
    assert np.array_equal(kc[:, 64], g["knew"][:, 0]) and np.array_equal(kc[:, :64], g["kcache"][:, :64])
    assert np.array_equal(kc[:, 65:], g["kcache"][:, 65:])
    d = ulp_diff_f16(o, g["out"])
    assert d.max() <= 1, d.max()
    assert np.all(np.isfinite(lse))


def test_kvcache_equals_plain_attention_over_the_valid_rows():
    """Closed form: decoding against a cache is plain attention over the concatenation of the
    valid cache rows and the new rows, per batch, causal aligned to the end."""
    rng = np.random.default_rng(5)
    b, sq, h, h_k, d, cap, n_new = 3, 4, 4, 2, 32, 96, 4
    q = rng.standard_normal((b, sq, h, d)).astype(np.float16)
    kc = rng.standard_normal((b, cap, h_k, d)).astype(np.float16)
    vc = rng.standard_normal((b, cap, h_k, d)).astype(np.float16)
    kn = rng.standard_normal((b, n_new, h_k, d)).astype(np.float16)
    vn = rng.standard_normal((b, n_new, h_k, d)).astype(np.float16)
    lens = np.array([0, 17, 92], dtype=np.int32)
    o, lse, kc2, vc2 = oracle.flash_kvcache(q, kc, vc, kn, vn, lens, 0.3, window=(-1, 0))
    for bi in range(b):
        n = int(lens[bi])
        kk = np.concatenate([kc[bi, :n], kn[bi]])[None]
        vv = np.concatenate([vc[bi, :n], vn[bi]])[None]
        ob, lb, _ = oracle.flash_fwd(q[bi:bi + 1], kk, vv, 0.3, window=(-1, 0))
        assert np.array_equal(o[bi], ob[0]) and np.array_equal(lse[bi], lb[0])
        assert np.array_equal(kc2[bi, :n + n_new], kk[0]) and np.array_equal(kc2[bi, n + n_new:], kc[bi, n + n_new:])
    # the inputs are left alone
    assert not np.array_equal(kc2, kc)


def test_kvcache_extra_args_blob_known_answer():
    # runtime/test/test_files/flash_attn_kvcache.mlir:11 extra_args, packed as
    # OpAccessor::GetAttrAsVoidPtr does (op_accessor.cc:212-242)
    fields = [96, 12288, 12288, 96, 96, 96] + [96] * 6 + [32] * 6 + [2, 3, 3, 32, 32, 1, 0.5, 1, 128, 128, 128, -1, -1]
    want = b"".join(struct.pack("<f", f) if isinstance(f, float) else struct.pack("<q", f) for f in fields)
    assert len(want) == 244
    assert oracle.fa_kvcache_pack_args(2, 1, 128, 3, 3, 32, 1, 0.5, (-1, -1)).tobytes() == want


# ---- dropout ---------------------------------------------------------------------------------
def _philox_words(ctr, key, rounds):
    off, sub, seed = ctr[0] | (ctr[1] << 32), ctr[2] | (ctr[3] << 32), key[0] | (key[1] << 32)
    return [int(x) for x in oracle.philox4x32(seed, sub, off, rounds)]


def test_philox4x32_known_answer_vectors():
    """The published known-answer vectors of Philox4x32 (Random123 kat_vectors: counter words,
    key words -> output words), for the standard 10 rounds and for 7 rounds, the count the
    reference library runs (lib/philox.cuh:43-50)."""
    zero, ones = [0] * 4, [0xFFFFFFFF] * 4
    pi_ctr, pi_key = [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]
    assert _philox_words(zero, [0, 0], 10) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert _philox_words(ones, ones[:2], 10) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert _philox_words(pi_ctr, pi_key, 10) == [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]
    assert _philox_words(zero, [0, 0], 7) == [0x5F6FB709, 0x0D893F64, 0x4F121F81, 0x4F730A48]
    assert _philox_words(ones, ones[:2], 7) == [0x5207DDC2, 0x45165E59, 0x4D8EE751, 0x8C52F662]


def test_dropout_mask_structure():
    """One Philox value serves one lane of one 16 x 32 block: the 16 elements that share
    (row % 8, (col % 8) / 2) inside a block are exactly the 16 bytes of that value, and
    different (batch, head) pairs use offsets 32 apart."""
    rs = np.array([0x1234567, 1000], dtype=np.uint64)
    b, h, sq, sk = 1, 2, 32, 64
    for thr_p in (0.0, 0.37, 0.9):
        m = oracle.dropout_keep_mask(rs, b, h, sq, sk, thr_p)
        thr = oracle.dropout_threshold(thr_p)
        for hi, rb, cb, lane in ((0, 0, 0, 0), (1, 1, 1, 13), (0, 1, 0, 31)):
            r = oracle.philox4x32(rs[0], rb | (cb << 32), int(rs[1]) + hi * 32 + lane)
            by = r.view(np.uint8)
            for tile in range(4):
                for half in range(2):
                    for e in range(2):
                        row = rb * 16 + lane // 4 + 8 * half
                        col = cb * 32 + tile * 8 + 2 * (lane % 4) + e
                        assert m[0, hi, row, col] == (by[4 * tile + 2 * half + e] <= thr)
    # p_dropout = 0 keeps everything (threshold 255)
    assert oracle.dropout_threshold(0.0) == 255 and oracle.dropout_keep_mask(rs, 1, 1, 16, 32, 0.0).all()


def test_dropout_keep_rate_matches_the_8_bit_threshold():
    rs = np.array([42, 7], dtype=np.uint64)
    for p in (0.1, 0.5):
        m = oracle.dropout_keep_mask(rs, 1, 2, 64, 128, p)
        want = (oracle.dropout_threshold(p) + 1) / 256.0
        assert abs(m.mean() - want) < 4 * np.sqrt(want * (1 - want) / m.size)


def _dropout_reference(q, k, v, keep, p_drop, scale, causal):
    """float64 attention with an explicit keep-mask: O = ((keep * softmax(S)) / p_keep) V"""
    b, sq, h, d = q.shape
    sk = k.shape[1]
    q64, k64, v64 = (t.astype(np.float64) for t in (q, k, v))
    s = np.einsum("bihd,bjhd->bhij", q64, k64) * scale
    if causal:
        i, j = np.arange(sq)[:, None], np.arange(sk)[None, :]
        s = np.where(j > i + sk - sq, -np.inf, s)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    z = np.where(keep, p, 0.0) / np.float64(np.float32(1.0) - np.float32(p_drop))
    return np.einsum("bhij,bjhd->bihd", z, v64), z, p


@pytest.mark.parametrize("causal", [False, True])
def test_dropout_forward_is_attention_with_the_explicit_mask(causal):
    rng = np.random.default_rng(5)
    b, sq, sk, h, d, p_drop = 2, 40, 72, 2, 16, 0.25
    q, k, v = (rng.standard_normal((b, s, h, d)).astype(np.float32) for s in (sq, sk, sk))
    rs = np.array([0xDEADBEEFCAFE, 12345], dtype=np.uint64)
    keep = oracle.dropout_keep_mask(rs, b, h, sq, sk, p_drop)
    window = (-1, 0) if causal else (-1, -1)
    o, lse, o32 = oracle.flash_fwd(q, k, v, 0.3, window, round_p=False, p_dropout=p_drop, rng_state=rs)
    want, _, _ = _dropout_reference(q, k, v, keep, p_drop, 0.3, causal)
    np.testing.assert_allclose(o32, want, atol=2e-5, rtol=1e-4)
    # LSE is that of the undropped scores
    _, lse0, _ = oracle.flash_fwd(q, k, v, 0.3, window, round_p=False)
    assert np.array_equal(lse, lse0)


def test_dropout_backward_is_the_gradient_with_the_mask_held_fixed():
    rng = np.random.default_rng(6)
    b, sq, sk, h, d, p_drop, scale = 1, 24, 40, 2, 8, 0.4, 0.35
    q, k, v, do = (rng.standard_normal((b, s, h, d)).astype(np.float32) for s in (sq, sk, sk, sq))
    rs = np.array([99, 4], dtype=np.uint64)
    keep = torch.from_numpy(oracle.dropout_keep_mask(rs, b, h, sq, sk, p_drop))
    p_keep = float(np.float32(1.0) - np.float32(p_drop))
    tq, tk, tv = (torch.from_numpy(t).double().requires_grad_(True) for t in (q, k, v))
    s = torch.einsum("bihd,bjhd->bhij", tq, tk) * scale
    z = torch.where(keep, torch.softmax(s, -1), torch.zeros((), dtype=torch.float64)) / p_keep
    out = torch.einsum("bhij,bjhd->bihd", z, tv)
    out.backward(torch.from_numpy(do).double())
    o, lse, o32 = oracle.flash_fwd(q, k, v, scale, round_p=False, p_dropout=p_drop, rng_state=rs)
    dq, dk, dv, dsm = oracle.flash_bwd(do, q, k, v, o32, lse, scale, round_p=False, p_dropout=p_drop, rng_state=rs)
    for got, want in ((dq, tq.grad), (dk, tk.grad), (dv, tv.grad)):
        np.testing.assert_allclose(got, want.numpy(), atol=3e-5, rtol=1e-4)
    # D is kept scaled by p_keep (flash_bwd_preprocess_kernel.h:124-128)
    np.testing.assert_allclose(dsm, np.einsum("bihd,bihd->bhi", do, o32) * p_keep, atol=1e-5, rtol=1e-5)


def test_backward_with_grouped_heads_is_the_gradient():
    """h_k < h: dK and dV of a key/value head are the sums over its query heads (torch autograd
    through attention with repeated K / V heads)."""
    rng = np.random.default_rng(8)
    b, sq, sk, h, h_k, d, scale = 2, 20, 28, 6, 2, 8, 0.3
    q, do = (rng.standard_normal((b, sq, h, d)).astype(np.float32) for _ in range(2))
    k, v = (rng.standard_normal((b, sk, h_k, d)).astype(np.float32) for _ in range(2))
    tq, tk, tv = (torch.from_numpy(t).double().requires_grad_(True) for t in (q, k, v))
    ke, ve = (t.repeat_interleave(h // h_k, dim=2) for t in (tk, tv))
    s = torch.einsum("bihd,bjhd->bhij", tq, ke) * scale
    i, j = torch.arange(sq)[:, None], torch.arange(sk)[None, :]
    s = s.masked_fill(j > i + sk - sq, float("-inf"))
    torch.einsum("bhij,bjhd->bihd", torch.softmax(s, -1), ve).backward(torch.from_numpy(do).double())
    o, lse, o32 = oracle.flash_fwd(q, k, v, scale, (-1, 0), round_p=False)
    dq, dk, dv, _ = oracle.flash_bwd(do, q, k, v, o32, lse, scale, (-1, 0), round_p=False)
    for got, want in ((dq, tq.grad), (dk, tk.grad), (dv, tv.grad)):
        np.testing.assert_allclose(got, want.numpy(), atol=3e-5, rtol=1e-4)
