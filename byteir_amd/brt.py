"""Python face of the host runtime, shaped like the reference's `brt` module
(runtime/python/src/module.cc:252-423) and its torch wrapper `BRTBackend`
(runtime/python/brt/backend.py:8-141), over the C ABI of libbrt.so.

    session = Session(device="ROCM")                 # brt.Session(device="CUDA", ...)
    session.load(path)                               # ByRE text
    req = session.new_request_context(stream)        # external HIP stream, e.g. torch's
    req.bind_arg(offset, tensor.data_ptr()); req.finish_io_binding(); req.run(); req.sync()
"""
import ctypes

from . import _lib

_DTYPES = {"f32": "float32", "f16": "float16", "bf16": "bfloat16", "f64": "float64", "i64": "int64",
           "i32": "int32", "i16": "int16", "i8": "int8", "ui8": "uint8", "i1": "bool"}


def _brt():
    return _lib.brt()


def _check(rc):
    if rc != 0:
        raise RuntimeError(_brt().brt_last_error().decode())


class Session:
    def __init__(self, device="ROCM", device_id=0, alloc_func=None, free_func=None):
        """device "ROCM" (alias "CUDA": modules written for the CUDA provider run unchanged);
        device_id < 0 gives a plan-only session for hosts without a GPU.  alloc_func/free_func:
        optional Python callables (size -> address, address -> None), e.g. torch's
        caching_allocator_alloc / caching_allocator_delete as in the reference's BRTBackend."""
        if device.upper() not in ("ROCM", "CUDA"):
            raise ValueError(f"unsupported device {device}")
        B = _brt()
        self._alloc_cb, self._free_cb = _lib.ALLOC_FN(0), _lib.FREE_FN(0)  # NULL: hipMalloc / hipFree
        if alloc_func is not None and free_func is not None:
            self._alloc_cb = _lib.ALLOC_FN(lambda n: alloc_func(n))
            self._free_cb = _lib.FREE_FN(lambda p: free_func(p))
        self._h = B.brt_session_create(device_id, self._alloc_cb, self._free_cb)
        if not self._h:
            raise RuntimeError(B.brt_last_error().decode())
        self._requests = []

    def close(self):
        if getattr(self, "_h", None):
            for r in list(self._requests):
                r.close()
            _brt().brt_session_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def load(self, path):
        _check(_brt().brt_session_load(self._h, str(path).encode()))

    def load_from_memory(self, text):
        _check(_brt().brt_session_load_text(self._h, text.encode()))

    def has_kernel(self, key):
        return bool(_brt().brt_session_has_kernel(self._h, key.encode()))

    # ---- graph introspection (module.cc:407-423) ------------------------------------------
    def get_arg_num(self):
        return _brt().brt_session_arg_num(self._h)

    def get_graph_arg_offset(self, name):
        return _brt().brt_session_arg_offset(self._h, name.encode())

    def get_arg_name(self, offset):
        return _brt().brt_session_arg_name(self._h, offset).decode()

    def _offsets(self, bit):
        return [i for i in range(self.get_arg_num()) if _brt().brt_session_arg_kind(self._h, i) & bit]

    def get_input_arg_offsets(self):
        return self._offsets(1)

    def get_output_arg_offsets(self):
        return self._offsets(2)

    def get_weight_arg_offsets(self):
        return self._offsets(4)

    def get_static_shape(self, offset):
        B = _brt()
        rank = B.brt_session_arg_rank(self._h, offset)
        buf = (ctypes.c_int64 * max(rank, 1))()
        B.brt_session_arg_shape(self._h, offset, buf)
        return [int(buf[i]) for i in range(rank)]

    def get_data_type(self, offset):
        return _DTYPES[_brt().brt_session_arg_dtype(self._h, offset).decode()]

    def get_space(self, offset):
        return _brt().brt_session_arg_space(self._h, offset).decode()

    def get_intermediate_bytes(self, space):
        """size of the per-frame arena for the memref.alloc intermediates of a memory space"""
        return _brt().brt_session_intermediate_bytes(self._h, space.encode())

    def get_op_keys(self):
        B = _brt()
        return [B.brt_session_op_key(self._h, i).decode() for i in range(B.brt_session_op_num(self._h))]

    def get_op_attr_blob(self, op_index, name):
        """the packed bytes OpAccessor::GetAttrAsVoidPtr hands to a custom library"""
        buf = ctypes.create_string_buffer(4096)
        n = _brt().brt_session_op_attr_blob(self._h, op_index, name.encode(), buf, 4096)
        if n < 0:
            raise RuntimeError(_brt().brt_last_error().decode())
        return buf.raw[:n]

    def new_request_context(self, stream=None):
        """stream: an integer hipStream_t (e.g. torch.cuda.current_stream().cuda_stream) used as
        the compute stream; None lets the request own a stream."""
        r = RequestContext(self, stream)
        self._requests.append(r)
        return r


class RequestContext:
    def __init__(self, session, stream):
        self._s = session
        self._listeners = []
        self._h = _brt().brt_request_create(session._h, ctypes.c_void_p(stream or 0), 0 if stream is None else 1)
        if not self._h:
            raise RuntimeError(_brt().brt_last_error().decode())

    def close(self):
        if getattr(self, "_h", None):
            _brt().brt_request_destroy(self._h)
            self._h = None
            if self in self._s._requests:
                self._s._requests.remove(self)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def bind_arg(self, offset, data_ptr):
        _check(_brt().brt_request_bind_arg(self._h, offset, ctypes.c_void_p(data_ptr)))

    def get_arg(self, offset):
        p = _brt().brt_request_get_arg(self._h, offset)
        if not p:
            raise RuntimeError(_brt().brt_last_error().decode())
        return p

    def finish_io_binding(self):
        _check(_brt().brt_request_finish_io_binding(self._h))

    def run(self):
        _check(_brt().brt_session_run(self._s._h, self._h))

    def sync(self):
        _check(_brt().brt_request_sync(self._h))

    def add_op_listener(self, fn):
        """fn(op_key: str, op_index: int, after: bool) around every op kernel run."""
        cb = _lib.OP_LISTENER(lambda user, key, idx, after: fn(key.decode(), idx, bool(after)))
        self._listeners.append(cb)
        _brt().brt_request_add_op_listener(self._h, cb, None)


class BRTBackend:
    """Runs a ByRE module on torch tensors, like the reference's BRTBackend
    (runtime/python/brt/backend.py): torch's caching allocator backs the session, the request
    runs on torch's current stream."""

    def __init__(self, device, brt_file_path):
        import torch
        self.torch = torch
        self.device = device
        self.session = Session(device="ROCM", alloc_func=torch.cuda.caching_allocator_alloc,
                               free_func=torch.cuda.caching_allocator_delete)
        self.session.load(brt_file_path)
        self.req = self.session.new_request_context(torch.cuda.current_stream().cuda_stream)

    def _check_arg(self, offset, t):
        if list(t.shape) != self.session.get_static_shape(offset):
            raise ValueError(f"argument {offset}: shape {list(t.shape)} != {self.session.get_static_shape(offset)}")
        if str(t.dtype).replace("torch.", "") != self.session.get_data_type(offset):
            raise ValueError(f"argument {offset}: dtype {t.dtype} != {self.session.get_data_type(offset)}")
        if not t.is_cuda or not t.is_contiguous():
            raise ValueError(f"argument {offset}: a contiguous device tensor is required")

    def run_with_outputs(self, inputs, outputs):
        ins, outs = self.session.get_input_arg_offsets(), self.session.get_output_arg_offsets()
        assert len(ins) == len(inputs) and len(outs) == len(outputs)
        for off, t in list(zip(ins, inputs)) + list(zip(outs, outputs)):
            self._check_arg(off, t)
            self.req.bind_arg(off, t.data_ptr())
        self.req.finish_io_binding()
        self.req.run()
        self.req.sync()

    def run(self, inputs):
        torch = self.torch
        outs = [torch.empty(self.session.get_static_shape(o), dtype=getattr(torch, self.session.get_data_type(o)), device="cuda")
                for o in self.session.get_output_arg_offsets()]
        self.run_with_outputs(inputs, outs)
        return outs

    def profile_with_outputs(self, inputs, outputs, warmup=10, iters=50):
        """average milliseconds of run()+sync() on the host clock (backend.py:81-141)."""
        import time
        self.run_with_outputs(inputs, outputs)
        for _ in range(warmup):
            self.req.run(); self.req.sync()
        t = time.time()
        for _ in range(iters):
            self.req.run(); self.req.sync()
        return (time.time() - t) / iters * 1e3
