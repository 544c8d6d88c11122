"""The flash-attention library executed on the host (tests/emu/lib/libflash_attn.so: the HIP
sources compiled against tests/emu/wave_emu.h, every lane a fiber): the same C ABI as the GPU
library of that name, on CPU tensors.  Tensors are registered with the emulator for the duration of
a call, so that buffer loads that pass their descriptor's range check are also checked against
the tensors' extents; `guarded` tensors end at (or start behind) a protected page, which turns
any stray access of a plain load or store into a reported fault."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU_LIB_DIR = os.path.join(ROOT, "tests", "emu", "lib")
LIB = os.path.join(EMU_LIB_DIR, "libflash_attn.so")
_vp = ctypes.c_void_p
_L = None


class EmuFault(RuntimeError):
    pass


def lib():
    global _L
    if _L is None:
        if not os.path.exists(LIB):
            subprocess.check_call([sys.executable, "-m", "byteir_amd.build", "emu"], cwd=ROOT)
        L = ctypes.CDLL(LIB)
        for n in ("fwd", "bwd", "kvcache"):
            f = getattr(L, f"flash_attn_{n}_checked")
            f.argtypes = [ctypes.POINTER(_vp), _vp, ctypes.c_int, _vp]
            f.restype = ctypes.c_int
        for n in ("fwd", "bwd", "kvcache"):
            getattr(L, f"flash_attn_{n}_ws").argtypes = [ctypes.POINTER(_vp), _vp, ctypes.c_int, _vp, ctypes.c_size_t, _vp]
            getattr(L, f"flash_attn_{n}_workspace_bytes").restype = ctypes.c_size_t
        L.flash_attn_fwd_workspace_bytes.argtypes = [_vp, ctypes.c_int]
        L.flash_attn_kvcache_workspace_bytes.argtypes = [_vp, ctypes.c_int]
        L.flash_attn_bwd_workspace_bytes.argtypes = [_vp, ctypes.c_int, ctypes.c_size_t]
        L.fa_emu_last_error.restype = ctypes.c_char_p
        L.flash_attn_last_error.restype = ctypes.c_char_p
        L.fa_emu_alloc.restype = _vp
        L.fa_emu_alloc.argtypes = [ctypes.c_size_t, ctypes.c_int]
        L.fa_emu_free.argtypes = [_vp]
        L.fa_emu_register.argtypes = [_vp, ctypes.c_size_t]
        L.fa_emu_unregister.argtypes = [_vp]
        L.fa_emu_select.argtypes = [ctypes.c_longlong, ctypes.c_longlong]
        L.fa_emu_blocks_run.restype = ctypes.c_longlong
        L.fa_emu_schedule.argtypes = [ctypes.c_int, ctypes.c_ulonglong]
        _L = L
    return _L


def select(stride=1, phase=0):
    """Run only the workgroups of every launch whose linear id is `phase` modulo `stride`."""
    lib().fa_emu_select(stride, phase)


def schedule(burst=1, seed=0):
    """burst <= 1: the waves of a workgroup advance round robin.  burst > 1: a wave picked at random
    runs up to `burst` steps in a row before the next pick, i.e. as far ahead of the others as
    the kernel's own barriers allow."""
    lib().fa_emu_schedule(burst, seed)


def guarded(shape, dtype, at_end=True):
    """A tensor whose last byte is the last byte before a protected page (at_end) or whose first
    byte is the first behind one.  Lives until the process ends."""
    L = lib()
    n = int(np.prod(shape))
    if n == 0:
        return torch.empty(shape, dtype=dtype)  # no bytes: nothing to guard (its data pointer is null)
    nbytes = n * torch.empty(0, dtype=dtype).element_size()
    p = L.fa_emu_alloc(max(nbytes, 16), 1 if at_end else 0)
    if not p:
        raise MemoryError("fa_emu_alloc")
    buf = (ctypes.c_char * max(nbytes, 16)).from_address(p)
    return torch.frombuffer(buf, dtype=dtype, count=n).reshape(shape)


def workspace_bytes(kind, blob, dtype, dq_accum_bytes=0):
    """flash_attn_{fwd,bwd,kvcache}_workspace_bytes for an extra_args blob."""
    L = lib()
    buf = ctypes.create_string_buffer(blob, len(blob))
    code = 1 if dtype == torch.float16 else 2
    if kind == "bwd":
        return L.flash_attn_bwd_workspace_bytes(ctypes.cast(buf, _vp), code, dq_accum_bytes)
    return getattr(L, f"flash_attn_{kind}_workspace_bytes")(ctypes.cast(buf, _vp), code)


def _call(kind, tensors, blob, dtype, workspace=None):
    L = lib()
    # the storage behind each tensor (a strided view addresses more than numel elements of it)
    live = {t.untyped_storage().data_ptr(): t.untyped_storage().nbytes() for t in list(tensors) + [workspace] if t is not None}
    for p, n in live.items():
        L.fa_emu_register(_vp(p), max(16, n))
    arr = (_vp * len(tensors))(*[t.data_ptr() if t is not None else None for t in tensors])
    buf = ctypes.create_string_buffer(blob, len(blob))
    try:
        code = 1 if dtype == torch.float16 else 2
        if workspace is not None:  # the caller's scratch (flash_attn_<kind>_ws)
            rc = getattr(L, f"flash_attn_{kind}_ws")(arr, ctypes.cast(buf, _vp), code, workspace.data_ptr(), workspace.numel() * workspace.element_size(), None)
        else:
            rc = getattr(L, f"flash_attn_{kind}_checked")(arr, ctypes.cast(buf, _vp), code, None)
    finally:
        for p in live:
            L.fa_emu_unregister(_vp(p))
    if rc:
        msg = L.fa_emu_last_error().decode() if L.fa_emu_faulted() else L.flash_attn_last_error().decode()
        L.fa_emu_reset()
        raise EmuFault(f"flash_attn_{kind}: rc {rc}: {msg}")


def _rng(rng_state):
    """{seed, offset} as the two 64-bit words the calls read."""
    to_i64 = lambda x: int(x) - (1 << 64) if int(x) >= (1 << 63) else int(x)
    return torch.tensor([to_i64(rng_state[0]), to_i64(rng_state[1])] if rng_state else [0, 0], dtype=torch.int64)


def fwd(q, k, v, scale, window=(-1, -1), out=None, p_dropout=0.0, rng_state=None):
    from byteir_amd import ops
    b, sq, h, d = q.shape
    o, lse = out if out is not None else (torch.empty_like(q), torch.empty((b, h, sq), dtype=torch.float32))
    _call("fwd", [q, k, v, _rng(rng_state), o, lse, None], ops.pack_flash_args(q, k, v, o, scale, window, p_dropout), q.dtype)
    return o, lse


def bwd(do, q, k, v, o, lse, scale, window=(-1, -1), out=None, p_dropout=0.0, rng_state=None):
    from byteir_amd import ops
    b, sq, h, d = q.shape
    ru = lambda x, m: -(-x // m) * m
    if out is None:
        # dq, dk, dv are addressed with the strides of q, k, v (flash_api.cu:377-389)
        like = lambda t: torch.empty_strided(t.shape, t.stride(), dtype=t.dtype)
        out = (like(q), like(k), like(v),
               torch.empty((b, h, ru(sq, 128)), dtype=torch.float32), torch.empty((b, ru(sq, 128), h, ru(d, 32)), dtype=torch.float32))
    dq, dk, dv, dsm, acc = out
    _call("bwd", [do, q, k, v, o, lse, _rng(rng_state), dq, dk, dv, dsm, acc], ops.pack_flash_args(q, k, v, o, scale, window, p_dropout), q.dtype)
    return dq, dk, dv


def kvcache(q, kcache, vcache, knew, vnew, seqlens_k, scale, window=(-1, -1)):
    from byteir_amd import ops
    b, sq, h, d = q.shape
    o, lse = torch.empty_like(q), torch.empty((b, h, sq), dtype=torch.float32)
    _call("kvcache", [q, kcache, vcache, knew, vnew, seqlens_k, o, lse],
          ops.pack_flash_kvcache_args(q, kcache, vcache, knew, vnew, o, scale, window), q.dtype)
    return o, lse


# ---- the reductions, the softmax and the input generator on the host ------------------------
KLIB = os.path.join(EMU_LIB_DIR, "libbrt_rocm_kernels.so")
_K = None


def klib():
    """tests/emu/lib/libbrt_rocm_kernels.so: reduce.hip, softmax.hip and fill.hip compiled for the
    host plus a host stand-in for the device layer (the C ABI of include/brt_rocm_kernels.h on
    host memory)."""
    global _K
    if _K is None:
        if not os.path.exists(KLIB):
            subprocess.check_call([sys.executable, "-m", "byteir_amd.build", "emu"], cwd=ROOT)
        K = ctypes.CDLL(KLIB)
        sz, i32 = ctypes.c_size_t, ctypes.c_int
        K.brt_rocm_reduce_workspace_bytes.argtypes = [i32, sz, sz, sz]
        K.brt_rocm_reduce_workspace_bytes.restype = sz
        K.brt_rocm_reduce.argtypes = [i32, i32, _vp, _vp, sz, sz, sz, _vp, sz, _vp]
        K.brt_rocm_reduce_static.argtypes = [i32, i32, _vp, _vp, sz, sz, sz, _vp]
        K.brt_rocm_softmax.argtypes = [i32, _vp, _vp, sz, sz, _vp]
        K.brt_rocm_softmax_axis.argtypes = [i32, _vp, _vp, sz, sz, sz, _vp]
        K.brt_rocm_fill.argtypes = [i32, i32, ctypes.c_uint64, _vp, sz, ctypes.c_float, ctypes.c_float, _vp]
        K.fa_emu_last_error.restype = ctypes.c_char_p
        K.fa_emu_alloc.restype = _vp
        K.fa_emu_alloc.argtypes = [sz, i32]
        K.fa_emu_register.argtypes = [_vp, sz]
        K.fa_emu_unregister.argtypes = [_vp]
        _K = K
    return _K


_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def kguarded(shape, dtype, at_end=True, offset_elems=0):
    """Like guarded(), from the kernels library's own table; `offset_elems` shifts the tensor's
    start off the 16-byte grid (at_end: the end stays against the protected page)."""
    K = klib()
    n = int(np.prod(shape))
    es = torch.empty(0, dtype=dtype).element_size()
    nbytes = (n + offset_elems) * es
    p = K.fa_emu_alloc(max(nbytes, 16), 1 if at_end else 0)
    if not p:
        raise MemoryError("fa_emu_alloc")
    if at_end:  # fa_emu_alloc rounds the size up to 16 bytes: push the tensor against the page's end
        p += (-nbytes) % 16 if nbytes >= 16 else 0
    buf = (ctypes.c_char * max(nbytes, 16)).from_address(p)
    return torch.frombuffer(buf, dtype=dtype, count=n, offset=offset_elems * es).reshape(shape)


def _kcheck(rc, what):
    K = klib()
    if rc:
        msg = K.fa_emu_last_error().decode()
        K.fa_emu_reset()
        raise EmuFault(f"{what}: rc {rc}: {msg}")


def reduce(op, x, A, B, C, out=None, static=False):
    """brt_rocm_reduce (or brt_rocm_reduce_static) of x viewed as [A, B, C] over B -> [A * C]."""
    K = klib()
    code = _CODE[x.dtype]
    out = out if out is not None else torch.empty(A * C, dtype=x.dtype)
    if static:
        rc = K.brt_rocm_reduce_static(op, code, x.data_ptr(), out.data_ptr(), A, B, C, None)
    else:
        nws = K.brt_rocm_reduce_workspace_bytes(code, A, B, C)
        ws = kguarded((max(nws, 16),), torch.uint8) if nws else None
        rc = K.brt_rocm_reduce(op, code, x.data_ptr(), out.data_ptr(), A, B, C, ws.data_ptr() if ws is not None else None, nws, None)
    _kcheck(rc, "brt_rocm_reduce")
    return out


def softmax(x, out=None, axis_abc=None):
    K = klib()
    out = out if out is not None else torch.empty_like(x)
    if axis_abc is None:
        rows, cols = x.shape
        rc = K.brt_rocm_softmax(_CODE[x.dtype], x.data_ptr(), out.data_ptr(), rows, cols, None)
    else:
        rc = K.brt_rocm_softmax_axis(_CODE[x.dtype], x.data_ptr(), out.data_ptr(), *axis_abc, None)
    _kcheck(rc, "brt_rocm_softmax")
    return out


def fill(t, dist, seed, a=0.0, b=1.0):
    _kcheck(klib().brt_rocm_fill(_CODE[t.dtype], dist, seed, t.data_ptr(), t.numel(), a, b, None), "brt_rocm_fill")
    return t
