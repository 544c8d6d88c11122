"""ctypes/numpy front end of the CPU oracle (oracle/oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, as the checker.  The product package never imports it.

Storage dtypes are numpy float32, float16 and, for bfloat16, uint16 bit patterns
(numpy has no bf16); helpers convert between float32 and bf16 bits with
round-to-nearest-even.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32, F16, BF16 = 0, 1, 2
SUM, MAX, MIN, PROD, MEAN, SUMSQR = range(6)


def build(force=False):
    """Compile oracle.c with gcc (used by __graft_entry__.build and lazily by tests)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c"))
    ):
        subprocess.check_call(["make", "-B", "-C", _HERE, "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class FaArgs(ctypes.Structure):
    """The 25 extra_args fields of the flash-attention custom op, in blob order
    (compiler/lib/Conversion/HloToByreTensor/HloToByreCustom.cpp:149-176)."""

    _fields_ = (
        [(n, ctypes.c_int64) for n in (
            "q_batch_stride", "k_batch_stride", "v_batch_stride", "o_batch_stride",
            "q_row_stride", "k_row_stride", "v_row_stride", "o_row_stride",
            "q_head_stride", "k_head_stride", "v_head_stride", "o_head_stride",
            "b", "h", "h_k", "d", "d_rounded")]
        + [("softmax_scale", ctypes.c_float)]
        + [(n, ctypes.c_int64) for n in (
            "seqlen_q", "seqlen_k", "seqlen_q_rounded", "seqlen_k_rounded")]
        + [("p_dropout", ctypes.c_float)]
        + [(n, ctypes.c_int64) for n in ("window_size_left", "window_size_right")]
    )


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u64, i32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int
        L.oracle_set_threads.argtypes = [i32]
        L.oracle_get_threads.restype = i32
        L.oracle_h2f.argtypes = [ctypes.c_uint16]; L.oracle_h2f.restype = ctypes.c_float
        L.oracle_f2h.argtypes = [ctypes.c_float]; L.oracle_f2h.restype = ctypes.c_uint16
        L.oracle_bf2f.argtypes = [ctypes.c_uint16]; L.oracle_bf2f.restype = ctypes.c_float
        L.oracle_f2bf.argtypes = [ctypes.c_float]; L.oracle_f2bf.restype = ctypes.c_uint16
        L.oracle_convert_from_f32.argtypes = [vp, vp, ctypes.c_size_t, i32]
        L.oracle_convert_to_f32.argtypes = [vp, vp, ctypes.c_size_t, i32]
        L.oracle_deduce_output_shape.argtypes = [vp, i32, vp, i32, vp]
        L.oracle_deduce_output_shape.restype = i32
        L.oracle_reduce_canonicalize.argtypes = [vp, i32, vp, i32, vp, i32, vp, vp, vp]
        L.oracle_reduce_canonicalize.restype = i32
        L.oracle_use_reduce_column.argtypes = [u64, u64, u64]
        L.oracle_use_reduce_column.restype = i32
        L.oracle_reference_workspace_bytes.argtypes = [u64, u64, u64, u64]
        L.oracle_reference_workspace_bytes.restype = u64
        L.oracle_reduce.argtypes = [i32, i32, vp, vp, u64, u64, u64]
        L.oracle_reduce_sum_f64.argtypes = [i32, vp, vp, vp, u64, u64, u64]
        L.oracle_softmax.argtypes = [i32, vp, vp, u64, u64]
        L.oracle_fa_pack_args.argtypes = [ctypes.POINTER(FaArgs), vp]
        L.oracle_fa_pack_args.restype = ctypes.c_size_t
        L.oracle_fa_unpack_args.argtypes = [vp, ctypes.POINTER(FaArgs)]
        L.oracle_fa_unpack_args.restype = ctypes.c_size_t
        L.oracle_flash_fwd.argtypes = [ctypes.POINTER(FaArgs), i32, i32, vp, vp, vp, vp, vp, vp]
        L.oracle_flash_bwd.argtypes = [ctypes.POINTER(FaArgs), i32, i32] + [vp] * 10
        L.oracle_flash_fwd_rng.argtypes = [ctypes.POINTER(FaArgs), i32, i32] + [vp] * 7
        L.oracle_flash_bwd_rng.argtypes = [ctypes.POINTER(FaArgs), i32, i32] + [vp] * 11
        L.oracle_splitmix64_at.argtypes = [u64, u64]
        L.oracle_splitmix64_at.restype = u64
        L.oracle_fill.argtypes = [i32, i32, u64, u64, u64, ctypes.c_float, ctypes.c_float, vp]
        L.oracle_philox4x32.argtypes = [u64, u64, u64, i32, vp]
        L.oracle_dropout_keep.argtypes = [vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_uint8]
        L.oracle_dropout_keep.restype = i32
        _lib = L
    return _lib


def set_threads(n):
    lib().oracle_set_threads(int(n))


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _code(arr, bf16=False):
    if arr.dtype == np.float32:
        return F32
    if arr.dtype == np.float16:
        return F16
    if arr.dtype == np.uint16:
        return BF16
    raise TypeError(f"unsupported storage dtype {arr.dtype}")


# ---- 16-bit conversions -------------------------------------------------------------
def to_bf16_bits(x):
    """float32 array -> uint16 array of bfloat16 bit patterns (round to nearest even)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_convert_from_f32(_p(x), _p(out), x.size, BF16)
    return out


def from_bf16_bits(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, dtype=np.float32)
    lib().oracle_convert_to_f32(_p(b), _p(out), b.size, BF16)
    return out


def to_f32(x):
    """Any storage array (f32 / f16 / bf16 bits) -> float32 values."""
    if x.dtype == np.uint16:
        return from_bf16_bits(x)
    return x.astype(np.float32)


def from_f32(x, code):
    if code == F32:
        return np.ascontiguousarray(x, dtype=np.float32)
    if code == F16:
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape, dtype=np.float16)
        lib().oracle_convert_from_f32(_p(x), _p(out), x.size, F16)
        return out
    return to_bf16_bits(x)


# ---- reductions ---------------------------------------------------------------------
def deduce_output_shape(shape, dims):
    s = np.asarray(shape, dtype=np.int64)
    d = np.asarray(dims, dtype=np.int64)
    out = np.zeros(max(len(s), 1), dtype=np.int64)
    r = lib().oracle_deduce_output_shape(_p(s), len(s), _p(d), len(d), _p(out))
    if r < 0:
        raise ValueError("invalid dimension")
    return [int(v) for v in out[:r]]


def reduce_canonicalize(in_shape, out_shape, dims):
    """-> (status, A, B, C); status 0 ok, 1 output-shape mismatch, 2 non-consecutive, 3 bad dim."""
    s = np.asarray(in_shape, dtype=np.int64)
    o = np.asarray(out_shape, dtype=np.int64)
    d = np.asarray(dims, dtype=np.int64)
    A, B, C = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
    st = lib().oracle_reduce_canonicalize(_p(s), len(s), _p(o), len(o), _p(d), len(d),
                                          ctypes.byref(A), ctypes.byref(B), ctypes.byref(C))
    return st, A.value, B.value, C.value


def use_reduce_column(A, B, C):
    return bool(lib().oracle_use_reduce_column(A, B, C))


UNIFORM, NORMAL = 0, 1


def fill(dtype_code, dist, seed, count, a=0.0, b=1.0, first=0):
    """Elements first .. first + count - 1 of the counter-based sequence brt_rocm_fill writes:
    float32 array for dtype_code 0, uint16 storage bits for 1 (f16) and 2 (bf16)."""
    out = np.empty(int(count), dtype=np.float32 if dtype_code == 0 else np.uint16)
    lib().oracle_fill(dtype_code, dist, int(seed), int(first), int(count), a, b, _p(out))
    return out


def reference_workspace_bytes(A, B, C, elem_size=4):
    return int(lib().oracle_reference_workspace_bytes(A, B, C, elem_size))


def reduce_abc(op, x, A, B, C):
    """Fold the middle axis of x viewed as [A,B,C]; sequential float chain per output."""
    x = np.ascontiguousarray(x)
    n_out = C if (A == 0 and B == 0) else A * C
    out = np.empty(n_out, dtype=x.dtype)
    lib().oracle_reduce(op, _code(x), _p(x), _p(out), A, B, C)
    return out


def reduce_op(op, x, dims):
    """Reduce an N-d array over `dims` the way the reference op kernel does."""
    x = np.ascontiguousarray(x)
    out_shape = deduce_output_shape(x.shape, dims)
    st, A, B, C = reduce_canonicalize(x.shape, out_shape, dims)
    if st != 0:
        raise ValueError(f"reduce_canonicalize status {st}")
    return reduce_abc(op, x, A, B, C).reshape(out_shape)


def reduce_sum_f64(x, A, B, C):
    """-> (sum in double, sum of |x| in double) per output of the [A,B,C] fold."""
    x = np.ascontiguousarray(x)
    out = np.empty(A * C, dtype=np.float64)
    out_abs = np.empty(A * C, dtype=np.float64)
    lib().oracle_reduce_sum_f64(_code(x), _p(x), _p(out), _p(out_abs), A, B, C)
    return out, out_abs


# ---- softmax ------------------------------------------------------------------------
def softmax(x, axis=-1):
    """Softmax over `axis` (the last one by default); x is f32 / f16 / bf16-bits; same storage
    out.  Another axis is moved last, reduced by the same C routine and moved back."""
    if axis % x.ndim != x.ndim - 1:
        return np.ascontiguousarray(np.moveaxis(softmax(np.moveaxis(x, axis, -1)), -1, axis))
    x = np.ascontiguousarray(x)
    cols = x.shape[-1]
    rows = x.size // cols if cols else 0
    out = np.empty_like(x)
    lib().oracle_softmax(_code(x), _p(x), _p(out), rows, cols)
    return out


# ---- flash attention ----------------------------------------------------------------
def round_up(x, m):
    return (x + m - 1) // m * m


def fa_args(b, sq, sk, h, h_k, d, scale, window=(-1, -1), p_dropout=0.0):
    """extra_args for dense [b, s, h, d] tensors, as the compiler computes them
    (compiler/lib/Conversion/HloToByreTensor/HloToByreCustom.cpp:111-147)."""
    a = FaArgs()
    a.q_batch_stride = sq * h * d; a.k_batch_stride = sk * h_k * d
    a.v_batch_stride = sk * h_k * d; a.o_batch_stride = sq * h * d
    a.q_row_stride = h * d; a.k_row_stride = h_k * d; a.v_row_stride = h_k * d; a.o_row_stride = h * d
    a.q_head_stride = d; a.k_head_stride = d; a.v_head_stride = d; a.o_head_stride = d
    a.b, a.h, a.h_k, a.d, a.d_rounded = b, h, h_k, d, round_up(d, 32)
    a.softmax_scale = scale
    a.seqlen_q, a.seqlen_k = sq, sk
    a.seqlen_q_rounded, a.seqlen_k_rounded = round_up(sq, 128), round_up(sk, 128)
    a.p_dropout = p_dropout
    a.window_size_left, a.window_size_right = window
    return a


def fa_pack_args(a):
    blob = np.zeros(192, dtype=np.uint8)
    n = lib().oracle_fa_pack_args(ctypes.byref(a), _p(blob))
    assert n == 192
    return blob


def fa_unpack_args(blob):
    blob = np.ascontiguousarray(blob, dtype=np.uint8)
    a = FaArgs()
    n = lib().oracle_fa_unpack_args(_p(blob), ctypes.byref(a))
    assert n == 192
    return a


def philox4x32(seed, subsequence, offset, rounds=7):
    """-> the 4 output words (uint32) of Philox4x32-`rounds` with key = seed and
    counter = (offset, subsequence)."""
    out = np.zeros(4, dtype=np.uint32)
    lib().oracle_philox4x32(int(seed), int(subsequence), int(offset), int(rounds), _p(out))
    return out


def dropout_threshold(p_dropout):
    """floor(p_keep * 255) with p_keep = 1 - p_dropout in float32 (flash_api.cu:291-292)."""
    return int(np.floor(np.float64(np.float32(1.0) - np.float32(p_dropout)) * 255.0))


def dropout_keep_mask(rng_state, b, h, sq, sk, p_dropout):
    """-> bool [b, h, sq, sk]: which attention entries survive dropout for rng_state = (seed, offset)."""
    rs = np.asarray(rng_state, dtype=np.uint64)
    thr = dropout_threshold(p_dropout)
    m = np.empty((b, h, sq, sk), dtype=bool)
    L = lib()
    for bi in range(b):
        for hi in range(h):
            for i in range(sq):
                for j in range(sk):
                    m[bi, hi, i, j] = L.oracle_dropout_keep(_p(rs), bi * h + hi, i, j, thr)
    return m


def flash_fwd(q, k, v, scale, window=(-1, -1), round_p=True, p_dropout=0.0, rng_state=None):
    """q [b,sq,h,d], k/v [b,sk,h_k,d] in one storage dtype; rng_state = (seed, offset) when
    p_dropout > 0.
    -> (o storage dtype [b,sq,h,d], lse f32 [b,h,sq], o unrounded f32 [b,sq,h,d])."""
    q, k, v = (np.ascontiguousarray(t) for t in (q, k, v))
    b, sq, h, d = q.shape
    sk, h_k = k.shape[1], k.shape[2]
    a = fa_args(b, sq, sk, h, h_k, d, scale, window, p_dropout)
    o = np.empty_like(q)
    lse = np.empty((b, h, sq), dtype=np.float32)
    o32 = np.empty((b, sq, h, d), dtype=np.float32)
    rs = np.asarray(rng_state, dtype=np.uint64) if p_dropout > 0 else None
    lib().oracle_flash_fwd_rng(ctypes.byref(a), _code(q), int(round_p), _p(q), _p(k), _p(v),
                               _p(rs) if rs is not None else None, _p(o), _p(lse), _p(o32))
    return o, lse, o32


def flash_bwd(dout, q, k, v, o, lse, scale, window=(-1, -1), round_p=True, p_dropout=0.0, rng_state=None):
    """-> (dq, dk, dv in storage dtype, D = rowsum(dout*o) f32 [b,h,sq], times p_keep under dropout)."""
    dout, q, k, v, o = (np.ascontiguousarray(t) for t in (dout, q, k, v, o))
    lse = np.ascontiguousarray(lse, dtype=np.float32)
    b, sq, h, d = q.shape
    sk, h_k = k.shape[1], k.shape[2]
    assert h % h_k == 0
    a = fa_args(b, sq, sk, h, h_k, d, scale, window, p_dropout)
    dq, dk, dv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    dsm = np.empty((b, h, sq), dtype=np.float32)
    rs = np.asarray(rng_state, dtype=np.uint64) if p_dropout > 0 else None
    lib().oracle_flash_bwd_rng(ctypes.byref(a), _code(q), int(round_p), _p(dout), _p(q), _p(k), _p(v),
                               _p(o), _p(lse), _p(rs) if rs is not None else None,
                               _p(dq), _p(dk), _p(dv), _p(dsm))
    return dq, dk, dv, dsm


def fa_kvcache_pack_args(b, sq, sk, h, h_k, d, seqlen_knew, scale, window=(-1, -1)):
    """The 244-byte extra_args blob of run_flash_attn_kvcache for dense [b, s, h, d] tensors:
    18 strides (q, k, v, knew, vnew, o: batch, then row, then head), b, h, h_k, d, d_rounded,
    seqlen_knew as i64, the scale as f32, seqlen_q, seqlen_k, their roundings to 128 and the
    two window sizes as i64, no padding
    (external_libs/runtime/flash_attn/lib/flash_api.cu:727-773)."""
    import struct
    qb, kb, nb = sq * h * d, sk * h_k * d, seqlen_knew * h_k * d
    ints1 = [qb, kb, kb, nb, nb, qb,
             h * d, h_k * d, h_k * d, h_k * d, h_k * d, h * d,
             d, d, d, d, d, d,
             b, h, h_k, d, round_up(d, 32), seqlen_knew]
    ints2 = [sq, sk, round_up(sq, 128), round_up(sk, 128), window[0], window[1]]
    return np.frombuffer(struct.pack("<24q", *ints1) + struct.pack("<f", scale) + struct.pack("<6q", *ints2),
                         dtype=np.uint8).copy()


def flash_kvcache(q, kcache, vcache, knew, vnew, seqlens_k, scale, window=(-1, -1), round_p=True):
    """Decoding against a key/value cache as run_mha_fwd_with_kvcache does it
    (flash_api.cu:434-567; BlockInfo, block_info.h:27-37; the Append_KV branch,
    flash_fwd_kernel.h:660-740, with rotary_dim = 0): per batch, rows
    [seqlens_k[b], seqlens_k[b] + seqlen_knew) of the caches are overwritten with knew / vnew,
    then q attends to rows [0, seqlens_k[b] + seqlen_knew) with the window aligned to the end
    of that range.  Restated on top of flash_fwd, one batch at a time.
    -> (o, lse [b,h,sq] f32, kcache_out, vcache_out); the inputs are not modified."""
    kc, vc = np.array(kcache, copy=True), np.array(vcache, copy=True)
    b, sq, h, d = q.shape
    n_new = 0 if knew is None else knew.shape[1]
    o = np.empty_like(q)
    lse = np.empty((b, h, sq), dtype=np.float32)
    for bi in range(b):
        n0 = int(seqlens_k[bi]) if seqlens_k is not None else kc.shape[1]
        if knew is not None:
            top = min(n0 + n_new, kc.shape[1])
            kc[bi, n0:top] = knew[bi, :top - n0]
            vc[bi, n0:top] = vnew[bi, :top - n0]
        n = min(n0 + n_new, kc.shape[1])
        ob, lb, _ = flash_fwd(q[bi:bi + 1], kc[bi:bi + 1, :n], vc[bi:bi + 1, :n], scale, window, round_p)
        o[bi], lse[bi] = ob[0], lb[0]
    return o, lse, kc, vc
