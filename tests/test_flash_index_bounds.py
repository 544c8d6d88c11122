"""Host-side bounds check of the flash-attention kernels' index arithmetic (no GPU).

`byteir_amd/csrc/flash_attn/flash_index.h` holds the integer functions with which the tuned
forward, dK/dV and dQ kernels decode a workgroup id, pick their tile ranges and form global and
LDS offsets; `index_check.cc` (g++) runs the same functions for every workgroup, thread and tile
of a launch and verifies that every address stays inside its tensor, buffer descriptor or LDS
array, that no 32-bit offset wraps and that every decoded index is inside its extent.  The
shapes are the benchmark configurations, the shape list of the GPU tests, and the two ragged
shapes that ran in a session which ended in a GPU memory fault (also with 64 query rows per
wave in the forward, the variant that was being introduced then)."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "byteir_amd", "lib", "libfa_index_check.so")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        subprocess.check_call([sys.executable, "-m", "byteir_amd.build", "index_check"], cwd=ROOT)
    L = ctypes.CDLL(LIB)
    L.fa_index_check.restype = ctypes.c_longlong
    L.fa_index_check.argtypes = [ctypes.POINTER(ctypes.c_longlong), ctypes.c_longlong,
                                 ctypes.POINTER(ctypes.c_longlong), ctypes.c_char_p, ctypes.c_int]
    L.fa_fwd_stream_span_bytes.restype = ctypes.c_longlong
    L.fa_fwd_stream_span_bytes.argtypes = [ctypes.c_longlong, ctypes.c_longlong]
    L.fa_bwd_stream_span_bytes.restype = ctypes.c_longlong
    L.fa_bwd_stream_span_bytes.argtypes = [ctypes.c_longlong, ctypes.c_longlong]
    return L


def check(L, b, h, h_k, sq, sk, d, win, qb=1, which=3, rs_scale=1):
    """-> (failed checks, checks made, first failure)."""
    shape = (ctypes.c_longlong * 11)(b, h, h_k, sq, sk, d, win[0], win[1], qb, which, rs_scale)
    sq_r, d_r = -(-sq // 128) * 128, -(-d // 32) * 32
    n, msg = ctypes.c_longlong(0), ctypes.create_string_buffer(512)
    bad = L.fa_index_check(shape, b * sq_r * h * d_r * 4, ctypes.byref(n), msg, 512)
    return bad, n.value, msg.value.decode()


# b, sq, sk, h, h_k, d, window: the tuned head dimensions of tests/test_gpu_flash_attn.py::CASES
GPU_TEST_SHAPES = [
    (1, 128, 128, 3, 3, 32, (-1, 0)), (2, 256, 256, 4, 4, 64, (-1, -1)), (2, 256, 256, 4, 4, 128, (-1, 0)),
    (1, 200, 333, 2, 2, 64, (-1, -1)), (1, 333, 200, 2, 2, 128, (-1, 0)), (1, 77, 500, 8, 8, 32, (-1, 0)),
    (1, 513, 513, 8, 2, 64, (-1, 0)), (1, 300, 300, 2, 2, 64, (64, 0)), (1, 300, 260, 2, 2, 128, (40, 30)),
    (3, 1, 50, 1, 1, 32, (-1, -1)), (2, 260, 260, 8, 2, 128, (-1, 0)), (1, 190, 300, 6, 1, 32, (50, 20)),
    (1, 1000, 1000, 4, 2, 64, (100, 60)), (1, 900, 1100, 2, 2, 128, (70, 0)), (1, 700, 700, 2, 1, 32, (0, 90)),
    (1, 2100, 2100, 2, 2, 64, (-1, 0)), (1, 2304, 2304, 4, 2, 128, (-1, -1)),
    (1, 4096, 4096, 16, 4, 128, (-1, 0)), (1, 4096, 4096, 8, 8, 128, (-1, 0)), (2, 3000, 3000, 8, 8, 64, (-1, -1)),
]


@pytest.mark.parametrize("shape", GPU_TEST_SHAPES)
def test_every_address_of_the_gpu_test_shapes_is_in_bounds(lib, shape):
    b, sq, sk, h, h_k, d, win = shape
    bad, n, msg = check(lib, b, h, h_k, sq, sk, d, win)
    assert n > 1000 and bad == 0, (shape, msg)


@pytest.mark.parametrize("qb", [1, 2])
@pytest.mark.parametrize("shape", [
    (4, 1100, 1100, 64, 16, 64, (-1, 0)),    # grouped heads, causal: the backward shares a group out over two workgroups
    (2, 2100, 1500, 64, 64, 64, (-1, -1)),   # more queries than keys
])
def test_the_two_shapes_of_the_faulting_session_are_in_bounds_on_the_host(lib, shape, qb):
    """Forward with 32 and with 64 query rows per wave, D kernel, dK/dV (with its partial buffers
    in dq_accum), group sum, dQ.  Nothing here runs on a GPU."""
    b, sq, sk, h, h_k, d, win = shape
    bad, n, msg = check(lib, b, h, h_k, sq, sk, d, win, qb=qb, which=3 if qb == 1 else 1)
    assert n > 10 ** 6 and bad == 0, (shape, qb, msg)


def test_benchmark_configurations_are_in_bounds(lib):
    for shape in ((4, 2048, 2048, 32, 32, 128, (-1, 0)), (2, 8192, 8192, 16, 16, 64, (-1, -1))):
        b, sq, sk, h, h_k, d, win = shape
        bad, n, msg = check(lib, b, h, h_k, sq, sk, d, win)
        assert n > 10 ** 6 and bad == 0, (shape, msg)


def test_the_check_reports_a_wrapping_offset_and_the_launch_guard_excludes_it(lib):
    """Negative control: key rows 1 MiB apart make a 5000-row head slice 5 GB long; the 32-bit
    tile offsets wrap, the check says so, and the launchers' guard sends such a call to the
    generic kernels."""
    b, sq, sk, h, d, scale = 1, 256, 5000, 1, 128, 4096
    bad, n, msg = check(lib, b, h, h, sq, sk, d, (-1, -1), which=1, rs_scale=scale)
    assert bad > 0 and "wraps" in msg, msg
    assert lib.fa_fwd_stream_span_bytes(sk, h * d * scale) >= 2 ** 31
    bad, n, msg = check(lib, b, h, h, sq, sk, d, (-1, -1), which=2, rs_scale=scale)
    assert bad > 0 and "wraps" in msg, msg
    assert lib.fa_bwd_stream_span_bytes(max(sq, sk), h * d * scale) >= 2 ** 31


def test_whatever_the_guards_let_through_does_not_wrap(lib):
    """Row strides just below the guard's limit, short and long sequences, sq != sk, windows: the
    tuned kernels take these calls (span < 2^31), so no offset may wrap and every access the
    hardware range check lets through must lie inside the tensor."""
    rng = np.random.default_rng(5)
    tried = 0
    for _ in range(200):
        d = int(rng.choice([32, 64, 128]))
        sk = int(rng.integers(1, 3000)); sq = int(rng.integers(1, 600))
        limit = (2 ** 31 // 2 - 256) // (max(sq, sk) + 4 * 64 + 128)   # largest row stride the forward guard accepts
        scale = max(1, limit // d - int(rng.integers(0, 3)))
        rs = d * scale
        win = [(-1, -1), (-1, 0), (40, 0), (17, 33)][int(rng.integers(0, 4))]
        fwd_ok = lib.fa_fwd_stream_span_bytes(sk, rs) < 2 ** 31
        bwd_ok = lib.fa_bwd_stream_span_bytes(max(sq, sk), rs) < 2 ** 31
        which = (1 if fwd_ok else 0) | (2 if bwd_ok else 0)
        if not which:
            continue
        bad, n, msg = check(lib, 1, 1, 1, sq, sk, d, win, which=which, rs_scale=scale)
        assert bad == 0, ((sq, sk, d, scale, win), msg)
        tried += 1
    assert tried > 100


def test_a_shifted_block_decode_would_be_caught(lib):
    """The check is not vacuous for the decode either: it is given more workgroups than the launch
    has (batch * heads overstated by the caller's own arithmetic below) and must object."""
    # 3 heads, causal -> order 3; pretending there are 4 heads makes bh reach 3: out of [0, 3)
    bad, n, msg = check(lib, 1, 3, 3, 300, 300, 64, (-1, 0))
    assert bad == 0
    # a key/value head count that does not divide the heads breaks hk = hi / (h / h_k)
    bad, n, msg = check(lib, 1, 6, 4, 300, 300, 64, (-1, 0), which=1)
    assert bad > 0, "6 query heads on 4 key/value heads must address a head beyond the K tensor"
