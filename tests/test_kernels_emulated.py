"""The reduction, softmax and input-generator kernels executed on the host, lane by lane (no GPU):
reduce.hip, softmax.hip and fill.hip compiled unchanged against tests/emu/wave_emu.h, as
tests/test_flash_emulated.py does for the attention kernels.  Every tensor ends at a protected
page or begins behind one, also when it starts off the 16-byte grid, so the vector loads of the
row, column and softmax kernels -- peeled heads and tails, clamped addresses, spans of 16-byte
words that cover an unaligned row -- cannot read or write a byte outside their tensors without
the run ending in a reported fault.  (On the GPU such an access inside an allocation's padding
would go unnoticed.)"""
import os

import numpy as np
import pytest
import torch

import emu_util as E
import oracle

pytestmark = pytest.mark.skipif(not (os.path.exists(E.KLIB) or os.path.exists("/opt/rocm/llvm/bin/clang++")),
                                reason="no host clang to build the emulated library with")

SUM, MAX, MIN, PROD, MEAN, SUMSQR = range(6)

REDUCE_CASES = [
    # A, B, C, dtype, elements the tensor starts off the 16-byte grid
    (1, 16, 32, torch.float32, 0), (16, 32, 1, torch.float32, 0), (1, 128 * 128, 1, torch.float32, 0),   # the reference's shape list,
    (2, 128, 256, torch.float32, 0), (2, 16 * 8, 64, torch.float32, 0),                                    # canonicalised
    (512, 1024, 1, torch.float32, 0),          # rows: 64 lanes per row
    (1, 3000, 520, torch.float32, 0),          # columns, split in two passes
    (1, 1100, 8192, torch.float32, 0),         # wide columns (the headline kernel), split
    (37, 5025, 1, torch.float32, 1),           # rows of odd length on an unaligned tensor: peeled head and tail
    (7, 333, 33, torch.float32, 3),            # columns that are no multiple of the vector
    (3, 50257, 1, torch.float16, 0), (5, 4099, 1, torch.float16, 3),
    (16, 2049, 260, torch.float16, 0), (1, 700, 1026, torch.float16, 1),
    (1, 1, 77, torch.float32, 0), (9, 1, 1, torch.float32, 1),   # nothing to fold
]


@pytest.mark.parametrize("at_end", [True, False])
@pytest.mark.parametrize("case", REDUCE_CASES)
def test_emulated_reductions_match_float64_and_stay_inside_their_tensors(case, at_end):
    A, B, C, dtype, off = case
    gen = torch.Generator().manual_seed(A + B + C)
    x = E.kguarded((A, B, C), dtype, at_end, off)
    x.copy_(torch.rand((A, B, C), generator=gen) * 2 - 1)
    out = E.kguarded((A * C,), dtype, at_end, off)
    x64 = x.double()
    for op in (SUM, MAX, MIN, MEAN, SUMSQR):
        out.fill_(-7.0)
        got = E.reduce(op, x, A, B, C, out=out).double().reshape(A, C)
        if op in (MAX, MIN):
            want = x64.max(1).values if op == MAX else x64.min(1).values
            assert torch.equal(got, want), (case, op)
            continue
        terms = x64 * x64 if op == SUMSQR else x64
        want, mag = terms.sum(1), terms.abs().sum(1)
        if op == MEAN:
            want, mag = want / B, mag / B
        tol = 1e-5 if dtype == torch.float32 else 2.0 ** -10
        assert bool(torch.all((got - want).abs() <= tol * torch.maximum(want.abs(), 1e-2 * mag) + 1e-30)), (case, op, float((got - want).abs().max()))
    # the fold whose split partials live in the library's own array gives the same bits
    a = E.reduce(SUM, x, A, B, C)
    b = E.reduce(SUM, x, A, B, C, static=True)
    assert torch.equal(a.view(torch.int16 if dtype == torch.float16 else torch.int32), b.view(torch.int16 if dtype == torch.float16 else torch.int32))


def test_emulated_reduction_propagates_nan_from_any_position():
    for A, B, C in ((1, 1024, 1), (1, 3000, 520), (4, 100, 4096)):
        for pos in (0, B // 2, B - 1):
            x = E.kguarded((A, B, C), torch.float32)
            x.copy_(torch.rand((A, B, C)))
            x[0, pos, 0] = float("nan")
            for op in (SUM, MAX):
                got = E.reduce(op, x, A, B, C).reshape(A, C)
                assert bool(torch.isnan(got[0, 0])) and int(torch.isnan(got).sum()) == 1, (A, B, C, pos, op)


SOFTMAX_CASES = [
    # rows, cols, dtype, offset
    (5, 1, torch.float32, 0), (9, 7, torch.float32, 1), (33, 64, torch.bfloat16, 0), (17, 1000, torch.float16, 0),   # a wave per row
    (12, 4096, torch.bfloat16, 0),            # the benchmark's row length: four waves per row
    (6, 2048, torch.float32, 0), (5, 8192, torch.bfloat16, 0), (7, 3000, torch.bfloat16, 0),
    (3, 16384, torch.bfloat16, 0), (2, 32000, torch.float32, 0),       # a workgroup per row, row in registers
    (3, 50257, torch.bfloat16, 0), (2, 50257, torch.float32, 3),       # odd length: every row starts off the 16-byte grid
    (2, 151936, torch.bfloat16, 1),                                     # two passes over the row
    (4, 1023, torch.float16, 5),
]


@pytest.mark.parametrize("at_end", [True, False])
@pytest.mark.parametrize("case", SOFTMAX_CASES)
def test_emulated_softmax_matches_float64_and_stays_inside_its_tensors(case, at_end):
    rows, cols, dtype, off = case
    gen = torch.Generator().manual_seed(rows + cols)
    x = E.kguarded((rows, cols), dtype, at_end, off)
    x.copy_(torch.randn((rows, cols), generator=gen) * 2.0)
    y = E.kguarded((rows, cols), dtype, at_end, off)
    y.fill_(-7.0)
    E.softmax(x, out=y)
    want = torch.softmax(x.double(), -1)
    ulp = {torch.float32: 2.0 ** -23, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    err = (y.double() - want).abs()
    # storage types: one rounding of the float result; f32: the float arithmetic itself (exp2, two multiplies)
    rel = 16 * ulp if dtype == torch.float32 else 2 * ulp
    assert bool(torch.all(err <= rel * want + 1e-30 + (2.0 ** -24 if dtype == torch.float16 else 0))), (case, float(err.max()))
    assert float((y.double().sum(-1) - 1).abs().max()) <= cols * ulp


@pytest.mark.parametrize("abc,dtype", [((3, 50, 128), torch.float32), ((2, 333, 17), torch.bfloat16), ((1, 4000, 100), torch.float32),
                                        ((16, 7, 1), torch.float16), ((1, 20000, 8), torch.float32)])
def test_emulated_softmax_over_an_inner_axis(abc, dtype):
    A, B, C = abc
    gen = torch.Generator().manual_seed(B)
    x = E.kguarded((A, B, C), dtype)
    x.copy_(torch.randn((A, B, C), generator=gen) * 2.0)
    y = E.kguarded((A, B, C), dtype, at_end=False)
    E.softmax(x, out=y, axis_abc=(A, B, C))
    want = torch.softmax(x.double(), 1)
    ulp = {torch.float32: 2.0 ** -23, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    err = (y.double() - want).abs()
    rel = 16 * ulp if dtype == torch.float32 else 2 * ulp
    assert bool(torch.all(err <= rel * want + 1e-30 + (2.0 ** -24 if dtype == torch.float16 else 0))), (abc, float(err.max()))


@pytest.mark.parametrize("dtype,code", [(torch.float32, oracle.F32), (torch.float16, oracle.F16), (torch.bfloat16, oracle.BF16)])
def test_emulated_generator_equals_its_host_twin_bit_for_bit(dtype, code):
    """brt_rocm_fill's kernel against oracle_fill: the same bits from (seed, index), for element
    counts around the kernel's per-thread span."""
    for n in (1, 7, 4096, 100003):
        for dist, a, b in ((0, -1.0, 1.0), (1, 0.0, 2.0)):
            t = E.kguarded((n,), dtype)
            E.fill(t, dist, 0xC2 + n, a, b)
            want = oracle.fill(code, dist, 0xC2 + n, n, a, b)
            got = t.view(torch.int16).numpy().view(np.uint16) if dtype != torch.float32 else t.numpy()
            assert np.array_equal(got.view(want.dtype), want), (dtype, n, dist)


def test_a_short_output_is_reported():
    """Negative control: the column kernel writing one element past a guarded output."""
    x = E.kguarded((1, 64, 520), torch.float32)
    x.copy_(torch.rand((1, 64, 520)))
    short = E.kguarded((519,), torch.float32)
    with pytest.raises(E.EmuFault, match="memory access outside every tensor"):
        E.reduce(SUM, x, 1, 64, 520, out=short)
    assert torch.isfinite(E.reduce(SUM, x, 1, 64, 520)).all()  # and the library still works afterwards
