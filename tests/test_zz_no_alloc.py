"""brt_rocm_reduce_static, the fold that allocates nothing (split partials in a device array that
belongs to the library), against brt_rocm_reduce with a caller workspace: the two share their
kernels, so the results must be bit-identical.  Two calls in a row on the same GPU, the second on
a smaller input, so that partials left over from the first call would show."""
import ctypes

import numpy as np
import pytest
import torch

from byteir_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _both(op, x, A, B, C):
    want = torch.empty(A * C, dtype=x.dtype, device="cuda")
    got = torch.full((A * C,), 7.0, dtype=x.dtype, device="cuda")
    ops.reduce_abc(op, x, want, A, B, C)
    ops.reduce_abc_static(op, x, got, A, B, C)
    torch.cuda.synchronize()
    return got, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_static_scratch_fold_equals_workspace_fold_on_two_calls_in_a_row(dtype):
    g = torch.Generator(device="cuda").manual_seed(5)
    # first call: a tall column fold that splits (partials in the scratch), sum and max
    A, B, C = 1, 16384, 2048
    assert ops.reduce_workspace_bytes(dtype, A, B, C) > 0
    x = (torch.rand(A * B * C, generator=g, device="cuda") * 2 - 1).to(dtype)
    for op in (_lib.REDUCE_SUM, _lib.REDUCE_MAX):
        got, want = _both(op, x, A, B, C)
        assert torch.equal(got.view(torch.int16 if dtype == torch.float16 else torch.int32),
                           want.view(torch.int16 if dtype == torch.float16 else torch.int32))
    # second call: smaller, still split, different A so the partial layout differs
    A2, B2, C2 = 3, 1000, 257
    assert ops.reduce_workspace_bytes(dtype, A2, B2, C2) > 0
    x2 = (torch.rand(A2 * B2 * C2, generator=g, device="cuda") * 2 - 1).to(dtype)
    for op in (_lib.REDUCE_SUM, _lib.REDUCE_MAX, _lib.REDUCE_MEAN):
        got, want = _both(op, x2, A2, B2, C2)
        assert torch.equal(got.view(torch.int16 if dtype == torch.float16 else torch.int32),
                           want.view(torch.int16 if dtype == torch.float16 else torch.int32))
    # and against the arithmetic itself, in float64 on the host
    want64 = x2.double().view(A2, B2, C2).sum(1).reshape(-1).cpu().numpy()
    got, _ = _both(_lib.REDUCE_SUM, x2, A2, B2, C2)
    tol = 1e-5 if dtype == torch.float32 else 2e-3
    sabs = x2.double().abs().view(A2, B2, C2).sum(1).reshape(-1).cpu().numpy()
    assert np.all(np.abs(got.double().cpu().numpy() - want64) <= tol * np.maximum(np.abs(want64), 1e-2 * sabs))
    # a row fold without split (no scratch at all) goes through the same entry point
    got, want = _both(_lib.REDUCE_SUM, x2, A2 * B2, C2, 1)
    assert torch.equal(got, want)


def test_static_scratch_fold_allocates_no_device_memory():
    """Free device memory as the driver reports it (hipMemGetInfo) and the caching allocator's
    counters are the same before and after the calls: a hipMalloc inside the entry point would
    lower the first, an allocation through torch would raise the second."""
    K = _lib.kernels()
    A, B, C = 1, 16384, 2048
    x = torch.ones(A * B * C, dtype=torch.float32, device="cuda")
    out = torch.empty(A * C, dtype=torch.float32, device="cuda")
    call = lambda op: K.brt_rocm_reduce_static(op, _lib.F32, ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                                               A, B, C, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert call(_lib.REDUCE_SUM) == 0  # first call on this device: the scratch address is looked up here
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    stats0 = {k: torch.cuda.memory_stats()[k] for k in ("allocation.all.allocated", "segment.all.allocated", "reserved_bytes.all.current")}
    for op in (_lib.REDUCE_SUM, _lib.REDUCE_MAX, _lib.REDUCE_SUM):
        assert call(op) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    stats1 = {k: torch.cuda.memory_stats()[k] for k in stats0}
    assert free1 == free0 and stats1 == stats0
    assert bool((out == float(B)).all())


def test_static_scratch_refuses_a_fold_that_does_not_fit():
    K = _lib.kernels()
    limit = _lib.REDUCE_STATIC_SCRATCH_BYTES
    # widest f16 tile count that still splits in two: the partials just exceed the array
    shape = next(((1, 64, c) for c in range(300 * 4096, 512 * 4096, 4096)
                  if K.brt_rocm_reduce_workspace_bytes(_lib.F16, 1, 64, c) > limit), None)
    if shape is None:
        pytest.skip("no fold of the current plan needs more than the static scratch")
    A, B, C = shape
    x = torch.zeros(A * B * C, dtype=torch.float16, device="cuda")
    out = torch.full((A * C,), 3.0, dtype=torch.float16, device="cuda")
    err = K.brt_rocm_reduce_static(_lib.REDUCE_SUM, _lib.F16, ctypes.c_void_p(x.data_ptr()),
                                   ctypes.c_void_p(out.data_ptr()), A, B, C, None)
    assert err == _lib.ERROR_STATIC_SCRATCH_TOO_SMALL
    assert b"static scratch" in K.brt_rocm_error_string(err)
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())  # nothing was enqueued
