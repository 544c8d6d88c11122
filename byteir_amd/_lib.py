"""ctypes loaders for the in-tree shared libraries.  Loading fails loudly: there is no
fallback path of any kind."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")

F32, F16, BF16 = 0, 1, 2
REDUCE_SUM, REDUCE_MAX, REDUCE_MIN, REDUCE_PROD, REDUCE_MEAN, REDUCE_SUMSQR = range(6)
FILL_UNIFORM, FILL_NORMAL = 0, 1
REDUCE_STATIC_SCRATCH_BYTES = 8 << 20
ERROR_STATIC_SCRATCH_TOO_SMALL = 20001


class LibraryMissing(RuntimeError):
    pass


def lib_path(name):
    return os.path.join(LIB_DIR, name)


def _load(name, mode=ctypes.DEFAULT_MODE):
    path = lib_path(name)
    if not os.path.exists(path):
        raise LibraryMissing(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation.")
    return ctypes.CDLL(path, mode=mode)


_kernels = None


def kernels():
    """libbrt_rocm_kernels.so with argtypes set from include/brt_rocm_kernels.h."""
    global _kernels
    if _kernels is None:
        L = _load("libbrt_rocm_kernels.so", ctypes.RTLD_GLOBAL)
        vp, sz, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
        pvp = ctypes.POINTER(ctypes.c_void_p)
        L.brt_rocm_version.restype = ctypes.c_char_p
        L.brt_rocm_error_string.argtypes = [i32]
        L.brt_rocm_error_string.restype = ctypes.c_char_p
        L.brt_rocm_device_count.argtypes = [ctypes.POINTER(i32)]
        L.brt_rocm_set_device.argtypes = [i32]
        L.brt_rocm_malloc.argtypes = [pvp, sz]
        L.brt_rocm_free.argtypes = [vp]
        L.brt_rocm_host_malloc.argtypes = [pvp, sz]
        L.brt_rocm_host_free.argtypes = [vp]
        for n in ("h2d", "d2h", "d2d"):
            getattr(L, f"brt_rocm_memcpy_{n}").argtypes = [vp, vp, sz, vp]
        L.brt_rocm_memset.argtypes = [vp, i32, sz, vp]
        L.brt_rocm_copy_kernel.argtypes = [vp, vp, sz, vp]
        L.brt_rocm_mfma_rate_probe.argtypes = [i32, vp, sz, vp, sz, i32, i32, vp]
        L.brt_rocm_stream_create.argtypes = [pvp]
        L.brt_rocm_stream_destroy.argtypes = [vp]
        L.brt_rocm_stream_synchronize.argtypes = [vp]
        L.brt_rocm_event_create.argtypes = [pvp]
        L.brt_rocm_event_destroy.argtypes = [vp]
        L.brt_rocm_event_record.argtypes = [vp, vp]
        L.brt_rocm_event_synchronize.argtypes = [vp]
        L.brt_rocm_event_elapsed_ms.argtypes = [ctypes.POINTER(ctypes.c_float), vp, vp]
        L.brt_rocm_fill.argtypes = [i32, i32, ctypes.c_uint64, vp, sz, ctypes.c_float, ctypes.c_float, vp]
        L.brt_rocm_reduce_workspace_bytes.argtypes = [i32, sz, sz, sz]
        L.brt_rocm_reduce_workspace_bytes.restype = sz
        L.brt_rocm_reduce.argtypes = [i32, i32, vp, vp, sz, sz, sz, vp, sz, vp]
        L.brt_rocm_reduce_ex.argtypes = [i32, i32, vp, vp, sz, sz, sz, vp, sz, vp, vp]
        L.brt_rocm_reduce_plan_describe.argtypes = [i32, sz, sz, sz, ctypes.c_char_p, sz]
        L.brt_rocm_reduce_static.argtypes = [i32, i32, vp, vp, sz, sz, sz, vp]
        L.brt_rocm_softmax.argtypes = [i32, vp, vp, sz, sz, vp]
        L.brt_rocm_softmax_axis.argtypes = [i32, vp, vp, sz, sz, sz, vp]
        L.brt_rocm_softmax_axis_ws.argtypes = [i32, vp, vp, sz, sz, sz, vp, sz, vp]
        L.brt_rocm_softmax_workspace_bytes.argtypes = [i32, sz, sz, sz]
        L.brt_rocm_softmax_workspace_bytes.restype = sz
        _kernels = L
    return _kernels


def check(err, what=""):
    if err != 0:
        msg = kernels().brt_rocm_error_string(err).decode()
        raise RuntimeError(f"{what}: HIP error {err} ({msg})")


_flash = None


def flash_attn():
    """libflash_attn.so: VERSION + run_flash_attn_{fwd,bwd}[_bf16] (include/flash_api.h)."""
    global _flash
    if _flash is None:
        L = _load("libflash_attn.so", ctypes.RTLD_GLOBAL)
        vp = ctypes.c_void_p
        for n in ("run_flash_attn_fwd", "run_flash_attn_bwd", "run_flash_attn_fwd_bf16", "run_flash_attn_bwd_bf16",
                  "run_flash_attn_kvcache", "run_flash_attn_kvcache_bf16"):
            f = getattr(L, n)
            f.argtypes = [ctypes.POINTER(vp), vp, vp]
            f.restype = None
        sz, i32 = ctypes.c_size_t, ctypes.c_int
        for n in ("fwd", "bwd", "kvcache"):
            getattr(L, f"flash_attn_{n}_checked").argtypes = [ctypes.POINTER(vp), vp, i32, vp]
            getattr(L, f"flash_attn_{n}_ws").argtypes = [ctypes.POINTER(vp), vp, i32, vp, sz, vp]
            getattr(L, f"flash_attn_{n}_workspace_bytes").restype = sz
        L.flash_attn_fwd_workspace_bytes.argtypes = [vp, i32]
        L.flash_attn_kvcache_workspace_bytes.argtypes = [vp, i32]
        L.flash_attn_bwd_workspace_bytes.argtypes = [vp, i32, sz]
        L.flash_attn_last_error.restype = ctypes.c_char_p
        _flash = L
    return _flash


ALLOC_FN = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_size_t)
FREE_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p)
OP_LISTENER = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int)

_brt = None


def brt():
    """libbrt.so with argtypes set from include/brt_c_api.h."""
    global _brt
    if _brt is None:
        kernels()  # libbrt.so links against the kernel library
        L = _load("libbrt.so", ctypes.RTLD_GLOBAL)
        vp, sz, i32, cp = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_char_p
        L.brt_last_error.restype = cp
        L.brt_session_create.argtypes = [i32, ALLOC_FN, FREE_FN]
        L.brt_session_create.restype = vp
        L.brt_session_destroy.argtypes = [vp]
        L.brt_session_destroy.restype = None
        L.brt_session_load.argtypes = [vp, cp]
        L.brt_session_load_text.argtypes = [vp, cp]
        L.brt_register_kernels_from_dynlib.argtypes = [cp]
        L.brt_session_has_kernel.argtypes = [vp, cp]
        L.brt_session_intermediate_bytes.argtypes = [vp, cp]
        L.brt_session_intermediate_bytes.restype = ctypes.c_size_t
        L.brt_session_arg_num.argtypes = [vp]
        L.brt_session_arg_num.restype = sz
        L.brt_session_arg_offset.argtypes = [vp, cp]
        L.brt_session_arg_name.argtypes = [vp, sz]
        L.brt_session_arg_name.restype = cp
        L.brt_session_arg_kind.argtypes = [vp, sz]
        L.brt_session_arg_rank.argtypes = [vp, sz]
        L.brt_session_arg_rank.restype = sz
        L.brt_session_arg_shape.argtypes = [vp, sz, ctypes.POINTER(ctypes.c_int64)]
        L.brt_session_arg_shape.restype = None
        L.brt_session_arg_dtype.argtypes = [vp, sz]
        L.brt_session_arg_dtype.restype = cp
        L.brt_session_arg_space.argtypes = [vp, sz]
        L.brt_session_arg_space.restype = cp
        L.brt_session_op_num.argtypes = [vp]
        L.brt_session_op_num.restype = sz
        L.brt_session_op_key.argtypes = [vp, sz]
        L.brt_session_op_key.restype = cp
        L.brt_session_op_attr_blob.argtypes = [vp, sz, cp, vp, sz]
        L.brt_session_op_attr_blob.restype = ctypes.c_long
        L.brt_request_create.argtypes = [vp, vp, i32]
        L.brt_request_create.restype = vp
        L.brt_request_destroy.argtypes = [vp]
        L.brt_request_destroy.restype = None
        L.brt_request_bind_arg.argtypes = [vp, sz, vp]
        L.brt_request_get_arg.argtypes = [vp, sz]
        L.brt_request_get_arg.restype = vp
        L.brt_request_finish_io_binding.argtypes = [vp]
        L.brt_request_sync.argtypes = [vp]
        L.brt_session_run.argtypes = [vp, vp]
        L.brt_request_add_op_listener.argtypes = [vp, OP_LISTENER, vp]
        L.brt_request_add_op_listener.restype = None
        _brt = L
    return _brt
