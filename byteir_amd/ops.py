"""Direct calls into the kernel C ABI with torch tensors as device memory.

torch is used for allocation and streams only; every computation below is a hand-written
HIP kernel reached through libbrt_rocm_kernels.so / libflash_attn.so.  Shapes follow the
reference's op kernels: reductions take the canonical [A, B, C] view computed by
`canonicalize_reduce` (ReduceImpl, runtime/lib/backends/cuda/providers/default/reduction/reduce_impl.h:28-59).
"""
import ctypes
import struct

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def _stream(stream=None):
    s = stream if stream is not None else torch.cuda.current_stream()
    return ctypes.c_void_p(s.cuda_stream)


def _dev(t):
    if not t.is_cuda:
        raise ValueError("device tensor required: the ROCm provider has no host path")
    if not t.is_contiguous():
        raise ValueError("dense row-major tensor required")
    return ctypes.c_void_p(t.data_ptr())


def fill(t, dist, seed, a=0.0, b=1.0, stream=None):
    """Counter-based synthetic data in place (brt_rocm_fill): element i is a function of
    (seed, i) only; dist = _lib.FILL_UNIFORM ([a, b)) or _lib.FILL_NORMAL (mean 0, sigma b)."""
    _lib.check(_lib.kernels().brt_rocm_fill(_DT[t.dtype], dist, seed, _dev(t), t.numel(), a, b, _stream(stream)),
               "brt_rocm_fill")
    return t


def deduce_output_shape(shape, dims):
    """reduction::DeduceOutputShape, runtime/lib/core/common/utils/math_helper.cc:145-159."""
    for d in dims:
        if not 0 <= d < len(shape):
            raise ValueError("invalid dimension")
    return [s for i, s in enumerate(shape) if i not in dims]


def canonicalize_reduce(in_shape, out_shape, dims):
    """ReduceImpl's constructor: -> (A, B, C); raises ValueError where the reference throws."""
    if list(out_shape) != deduce_output_shape(in_shape, dims):
        raise ValueError("output shape does not match the deduced shape")
    live = sorted(d for d in dims if in_shape[d] != 1)
    if not live:
        n = 1
        for s in in_shape:
            n *= s
        return 0, 0, n
    if any(b - a != 1 for a, b in zip(live, live[1:])):
        raise ValueError("Only consecutive dimensions reduction is supported")
    A = B = C = 1
    for s in in_shape[:live[0]]:
        A *= s
    for d in live:
        B *= in_shape[d]
    for s in in_shape[live[-1] + 1:]:
        C *= s
    return A, B, C


def reduce_workspace_bytes(dtype, A, B, C):
    return _lib.kernels().brt_rocm_reduce_workspace_bytes(_DT[dtype], A, B, C)


def reduce_abc(op, x, out, A, B, C, workspace=None, stream=None):
    """Enqueue out[a,c] = fold_b x[a,b,c]; `workspace` is a uint8 device tensor of at least
    reduce_workspace_bytes(...) bytes (allocated here when omitted)."""
    K = _lib.kernels()
    need = K.brt_rocm_reduce_workspace_bytes(_DT[x.dtype], A, B, C)
    if need and workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    ws_ptr = ctypes.c_void_p(workspace.data_ptr()) if workspace is not None else None
    ws_len = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _lib.check(K.brt_rocm_reduce(op, _DT[x.dtype], _dev(x), _dev(out), A, B, C, ws_ptr, ws_len,
                                 _stream(stream)), "brt_rocm_reduce")
    return out


def reduce_abc_static(op, x, out, A, B, C, stream=None):
    """The same fold through brt_rocm_reduce_static: split partials in the library's own device
    array, no allocation of any kind; raises when the fold needs more than that array holds."""
    _lib.check(_lib.kernels().brt_rocm_reduce_static(op, _DT[x.dtype], _dev(x), _dev(out), A, B, C,
                                                     _stream(stream)), "brt_rocm_reduce_static")
    return out


def reduce(op, x, dims, stream=None):
    """Reduce<Op>Op over `dims` of a dense tensor (op: _lib.REDUCE_SUM / MAX / MIN / PROD / MEAN /
    SUMSQR)."""
    out_shape = deduce_output_shape(list(x.shape), list(dims))
    A, B, C = canonicalize_reduce(list(x.shape), out_shape, list(dims))
    out = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    return reduce_abc(op, x, out, A, B, C, stream=stream)


def softmax_workspace_bytes(x, axis=-1):
    """brt_rocm_softmax_workspace_bytes for softmax(x, axis=axis)."""
    axis = axis % x.dim()
    a, b, c = 1, x.shape[axis], 1
    for n in x.shape[:axis]:
        a *= n
    for n in x.shape[axis + 1:]:
        c *= n
    return _lib.kernels().brt_rocm_softmax_workspace_bytes(_DT[x.dtype], a, b, c)


def softmax(x, out=None, stream=None, axis=-1, workspace=None):
    """byteir.softmax over `axis` of a dense tensor (the last one by default).  workspace: the
    caller's scratch (uint8 device tensor of softmax_workspace_bytes) for the inner-axis split."""
    if out is None:
        out = torch.empty_like(x)
    axis = axis % x.dim()
    a, b, c = 1, x.shape[axis], 1
    for n in x.shape[:axis]:
        a *= n
    for n in x.shape[axis + 1:]:
        c *= n
    if workspace is not None:
        _lib.check(_lib.kernels().brt_rocm_softmax_axis_ws(_DT[x.dtype], _dev(x), _dev(out), a, b, c, _dev(workspace),
                                                           workspace.numel() * workspace.element_size(), _stream(stream)),
                   "brt_rocm_softmax_axis_ws")
        return out
    _lib.check(_lib.kernels().brt_rocm_softmax_axis(_DT[x.dtype], _dev(x), _dev(out), a, b, c,
                                                    _stream(stream)), "brt_rocm_softmax_axis")
    return out


# ---- flash attention through the custom-library ABI ---------------------------------------
def round_up(x, m):
    return (x + m - 1) // m * m


def pack_flash_args(q, k, v, o, scale, window, p_dropout=0.0):
    """The 192-byte extra_args blob for [b, s, h, d] tensors: 17 i64, f32, 4 i64, f32, 2 i64,
    unpadded (OpAccessor::GetAttrAsVoidPtr, runtime/lib/core/framework/op_accessor.cc:212-242;
    field order compiler/lib/Conversion/HloToByreTensor/HloToByreCustom.cpp:149-176)."""
    b, sq, h, d = q.shape
    sk, h_k = k.shape[1], k.shape[2]
    ints1 = [q.stride(0), k.stride(0), v.stride(0), o.stride(0),
             q.stride(1), k.stride(1), v.stride(1), o.stride(1),
             q.stride(2), k.stride(2), v.stride(2), o.stride(2),
             b, h, h_k, d, round_up(d, 32)]
    ints2 = [sq, sk, round_up(sq, 128), round_up(sk, 128)]
    return (struct.pack("<17q", *ints1) + struct.pack("<f", scale) + struct.pack("<4q", *ints2)
            + struct.pack("<f", p_dropout) + struct.pack("<2q", *window))


def _call_custom(fn, tensors, blob, stream):
    arr = (ctypes.c_void_p * len(tensors))(*[t.data_ptr() if t is not None else None for t in tensors])
    buf = ctypes.create_string_buffer(blob, len(blob))
    fn(arr, ctypes.cast(buf, ctypes.c_void_p), _stream(stream))


def _call_custom_ws(kind, dtype, tensors, blob, workspace, stream):
    """flash_attn_<kind>_ws: the error-returning entry point with the caller's scratch
    (`workspace`: a uint8 device tensor, or None)."""
    L = _lib.flash_attn()
    arr = (ctypes.c_void_p * len(tensors))(*[t.data_ptr() if t is not None else None for t in tensors])
    buf = ctypes.create_string_buffer(blob, len(blob))
    ws = ctypes.c_void_p(workspace.data_ptr()) if workspace is not None else None
    n = workspace.numel() * workspace.element_size() if workspace is not None else 0
    rc = getattr(L, f"flash_attn_{kind}_ws")(arr, ctypes.cast(buf, ctypes.c_void_p), 1 if dtype == torch.float16 else 2, ws, n, _stream(stream))
    if rc < 0:
        raise ValueError(L.flash_attn_last_error().decode())
    _lib.check(rc, f"flash_attn_{kind}_ws")


def flash_attn_workspace_bytes(kind, dtype, blob, dq_accum_bytes=0):
    """flash_attn_{fwd,bwd,kvcache}_workspace_bytes for an extra_args blob."""
    L = _lib.flash_attn()
    buf = ctypes.create_string_buffer(blob, len(blob))
    code = 1 if dtype == torch.float16 else 2
    if kind == "bwd":
        return L.flash_attn_bwd_workspace_bytes(ctypes.cast(buf, ctypes.c_void_p), code, dq_accum_bytes)
    return getattr(L, f"flash_attn_{kind}_workspace_bytes")(ctypes.cast(buf, ctypes.c_void_p), code)


def rng_state_tensor(seed, offset, device):
    """The rng_state operand of the attention calls: {seed, offset} as two 64-bit words."""
    to_i64 = lambda x: int(x) - (1 << 64) if int(x) >= (1 << 63) else int(x)
    return torch.tensor([to_i64(seed), to_i64(offset)], dtype=torch.int64, device=device)


def flash_attn_fwd(q, k, v, scale, window=(-1, -1), stream=None, out=None, p_dropout=0.0, rng_state=None, workspace=None):
    """run_flash_attn_fwd: tensors {q, k, v, rng_state, o, softmax_lse, softmax_P}
    (external_libs/runtime/flash_attn/lib/flash_api.cu:586-654). -> (o, lse[b,h,sq] f32).
    out: optional (o, lse, rng_state) to write into instead of allocating.
    p_dropout > 0 reads {seed, offset} from rng_state (an int64[2] device tensor, see
    rng_state_tensor), as the reference's kernel does (flash_fwd_kernel.h:46-47)."""
    L = _lib.flash_attn()
    b, sq, h, d = q.shape
    if out is not None:
        o, lse, rng = out
    else:
        o = torch.empty_like(q)
        lse = torch.empty((b, h, sq), dtype=torch.float32, device=q.device)
        rng = rng_state if rng_state is not None else torch.zeros(2, dtype=torch.int64, device=q.device)
    blob = pack_flash_args(q, k, v, o, scale, window, p_dropout)
    if workspace is not None:  # the caller's scratch for the key-axis split (flash_attn_fwd_ws)
        _call_custom_ws("fwd", q.dtype, [q, k, v, rng, o, lse, None], blob, workspace, stream)
        return o, lse
    fn = L.run_flash_attn_fwd if q.dtype == torch.float16 else L.run_flash_attn_fwd_bf16
    _call_custom(fn, [q, k, v, rng, o, lse, None], blob, stream)
    return o, lse


def flash_attn_bwd_buffers(q, k, v):
    """The output and scratch tensors of run_flash_attn_bwd for these shapes:
    (dq, dk, dv, d_softmax, dq_accum, rng_state)."""
    b, sq, h, d = q.shape
    sq_r, d_r = round_up(sq, 128), round_up(d, 32)
    like = lambda t: torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device=t.device)
    # dq, dk, dv are addressed with the strides of q, k, v (flash_api.cu:377-389)
    return (like(q), like(k), like(v),
            torch.empty((b, h, sq_r), dtype=torch.float32, device=q.device),
            torch.empty((b, sq_r, h, d_r), dtype=torch.float32, device=q.device),
            torch.zeros(2, dtype=torch.int64, device=q.device))


def flash_attn_bwd(dout, q, k, v, o, lse, scale, window=(-1, -1), stream=None, out=None, p_dropout=0.0,
                   rng_state=None, workspace=None):
    """run_flash_attn_bwd: tensors {dout, q, k, v, out, softmax_lse, rng_state, dq, dk, dv,
    d_softmax, dq_accum} (flash_api.cu:656-725). -> (dq, dk, dv).
    out: optional result of flash_attn_bwd_buffers to write into instead of allocating.
    p_dropout > 0 needs the rng_state the forward call used."""
    L = _lib.flash_attn()
    dq, dk, dv, dsm, dq_accum, rng = out if out is not None else flash_attn_bwd_buffers(q, k, v)
    if rng_state is not None:
        rng = rng_state
    blob = pack_flash_args(q, k, v, o, scale, window, p_dropout)
    if workspace is not None:  # the caller's scratch for partial dK / dV (flash_attn_bwd_ws)
        _call_custom_ws("bwd", q.dtype, [dout, q, k, v, o, lse, rng, dq, dk, dv, dsm, dq_accum], blob, workspace, stream)
        return dq, dk, dv
    fn = L.run_flash_attn_bwd if q.dtype == torch.float16 else L.run_flash_attn_bwd_bf16
    _call_custom(fn, [dout, q, k, v, o, lse, rng, dq, dk, dv, dsm, dq_accum], blob, stream)
    return dq, dk, dv


def pack_flash_kvcache_args(q, kcache, vcache, knew, vnew, o, scale, window):
    """The 244-byte extra_args blob of run_flash_attn_kvcache: 24 i64, f32, 6 i64, unpadded
    (field order external_libs/runtime/flash_attn/lib/flash_api.cu:727-773).  knew / vnew may
    be None: their strides and seqlen_knew are then 0."""
    b, sq, h, d = q.shape
    sk, h_k = kcache.shape[1], kcache.shape[2]
    kn = knew if knew is not None else None
    st = lambda t, i: t.stride(i) if t is not None else 0
    ints1 = [q.stride(0), kcache.stride(0), vcache.stride(0), st(kn, 0), st(vnew, 0), o.stride(0),
             q.stride(1), kcache.stride(1), vcache.stride(1), st(kn, 1), st(vnew, 1), o.stride(1),
             q.stride(2), kcache.stride(2), vcache.stride(2), st(kn, 2), st(vnew, 2), o.stride(2),
             b, h, h_k, d, round_up(d, 32), knew.shape[1] if knew is not None else 0]
    ints2 = [sq, sk, round_up(sq, 128), round_up(sk, 128), window[0], window[1]]
    return struct.pack("<24q", *ints1) + struct.pack("<f", scale) + struct.pack("<6q", *ints2)


def flash_attn_kvcache(q, kcache, vcache, knew, vnew, seqlens_k, scale, window=(-1, -1), stream=None, workspace=None):
    """run_flash_attn_kvcache: tensors {q, k_cache, v_cache, k_new, v_new, seqlens_k, o,
    softmax_lse} (flash_api.cu:727-811).  Appends knew / vnew to the caches IN PLACE at row
    seqlens_k[b], then attends to the first seqlens_k[b] + seqlen_knew rows of each batch.
    seqlens_k: int32 [b] device tensor. -> (o, lse[b,h,sq] f32)."""
    L = _lib.flash_attn()
    b, sq, h, d = q.shape
    o = torch.empty_like(q)
    lse = torch.empty((b, h, sq), dtype=torch.float32, device=q.device)
    blob = pack_flash_kvcache_args(q, kcache, vcache, knew, vnew, o, scale, window)
    if workspace is not None:
        _call_custom_ws("kvcache", q.dtype, [q, kcache, vcache, knew, vnew, seqlens_k, o, lse], blob, workspace, stream)
        return o, lse
    fn = L.run_flash_attn_kvcache if q.dtype == torch.float16 else L.run_flash_attn_kvcache_bf16
    _call_custom(fn, [q, kcache, vcache, knew, vnew, seqlens_k, o, lse], blob, stream)
    return o, lse
