"""GPU parity of the fused row softmax against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch
from scipy.special import softmax as sp_softmax

import oracle
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

# storage-type tolerances: |got - oracle| <= TOL_REL * |oracle| + TOL_ABS
#   f32 : the kernel's exp is v_exp_f32 on a pre-scaled argument (about 2e-6 relative for
#         |x - max| <= 30), sums are wave trees instead of one chain
#   f16 / bf16 : one storage ulp (2^-10 / 2^-7 relative) from the single rounding at the store
TOL = {oracle.F32: (1e-5, 1e-10), oracle.F16: (2.0 ** -10, 6e-8), oracle.BF16: (2.0 ** -7, 1e-38)}


def run_case(shape, code, seed=0, sigma=2.0):
    from byteir_amd import ops
    x32 = (np.random.default_rng(seed).standard_normal(shape) * sigma).astype(np.float32)
    xs = oracle.from_f32(x32, code)
    got = oracle.to_f32(host(ops.softmax(dev(xs))))
    want = oracle.to_f32(oracle.softmax(xs))
    if code == oracle.F32 and shape[-1] > 8192:
        # the oracle's single float chain over >8192 exponentials drifts past 1e-5 from the
        # exact value; for such rows the yardstick is the fp64 closed form that pins the oracle
        want = sp_softmax(x32.astype(np.float64), axis=-1).astype(np.float32)
    rel, ab = TOL[code]
    assert np.all(np.abs(got - want) <= rel * np.abs(want) + ab), float(np.abs(got - want).max())
    return got, want


@pytest.mark.parametrize("code", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("shape", [(10, 128), (8 * 12, 256, 256), (3, 1), (5, 4097), (7, 8), (33, 4096), (2, 8192),
                                   (2, 20000), (1, 100003), (129, 520),
                                   # rows held in LDS (odd lengths shift every row off 16-byte alignment),
                                   # the longest that fit, and rows streamed twice
                                   (6, 50257), (3, 32000), (2, 39900), (3, 40000), (2, 79800), (2, 80100), (5, 8200)])
def test_softmax_matches_oracle(shape, code):
    run_case(shape, code)


@pytest.mark.parametrize("code", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("shape,axis", [((4, 33, 70), 1), ((2, 3, 5, 7), 2), ((129, 1000), 0), ((3, 260, 2), 1),
                                        ((2, 1, 300), 1), ((5, 64, 64), -2),
                                        # few columns, long axis: the axis is cut into segments over workgroups
                                        ((1, 5000, 100), 1), ((2, 3000, 24), 1), ((3, 2000, 7), 1), ((40000, 16), 0),
                                        # wide: 128-bit column groups, one workgroup per column tile
                                        ((3, 300, 2048), 1), ((600, 4100), 0)])
def test_softmax_over_an_inner_axis(shape, axis, code):
    from byteir_amd import ops
    x32 = (np.random.default_rng(sum(shape)).standard_normal(shape) * 2.0).astype(np.float32)
    xs = oracle.from_f32(x32, code)
    got = oracle.to_f32(host(ops.softmax(dev(xs), axis=axis)))
    want = oracle.to_f32(oracle.softmax(xs, axis=axis))
    if code == oracle.F32 and shape[axis] > 2048:  # the oracle's float chain drifts; fp64 closed form instead
        want = sp_softmax(x32.astype(np.float64), axis=axis).astype(np.float32)
    rel, ab = TOL[code]
    assert np.all(np.abs(got - want) <= rel * np.abs(want) + ab), float(np.abs(got - want).max())
    np.testing.assert_allclose(got.sum(axis=axis), 1.0, atol=2e-2 if code != oracle.F32 else 1e-5)


@pytest.mark.parametrize("rows", [6, 4000])
def test_softmax_inner_axis_with_infinities(rows):
    from byteir_amd import ops
    x = torch.randn((2, rows, 130), device="cuda")
    x[0, :3, 5] = -float("inf")          # the column starts with -inf values
    x[1, :, 7] = -float("inf")           # a column of -inf only: NaN, as exp(-inf - -inf) / 0 in the reference lowering
    x[1, 2, 9] = float("nan")
    y = host(ops.softmax(x, axis=1))
    want = oracle.softmax(host(x), axis=1)
    assert np.array_equal(np.isnan(y), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.abs(y[ok] - want[ok]).max() <= 1e-5
    assert np.all(y[0, :3, 5] == 0)


@pytest.mark.parametrize("code", [oracle.F32, oracle.BF16])
@pytest.mark.parametrize("cols", [9001, 30000, 90000])
def test_long_rows_from_an_unaligned_view_leave_their_neighbours_alone(cols, code):
    """Input and output start 1 element (f32: 4 bytes, bf16: 2 bytes) into a 16-byte granule: the
    kernels read whole granules around the rows and must write the rows only."""
    from byteir_amd import ops
    rows = 3
    x32 = (np.random.default_rng(cols).standard_normal((rows, cols)) * 2.0).astype(np.float32)
    xs = oracle.from_f32(x32, code)
    tdt = torch.float32 if code == oracle.F32 else torch.bfloat16
    buf_in = torch.zeros(rows * cols + 16, dtype=tdt, device="cuda")
    buf_out = torch.full((rows * cols + 16,), 7.0, dtype=tdt, device="cuda")
    xin = buf_in[1:1 + rows * cols].view(rows, cols)
    xin.copy_(dev(xs))
    yout = buf_out[1:1 + rows * cols].view(rows, cols)
    ops.softmax(xin, yout)
    got = oracle.to_f32(host(yout))
    want = sp_softmax(oracle.to_f32(xs).astype(np.float64), axis=-1).astype(np.float32)
    rel, ab = TOL[code]
    assert np.all(np.abs(got - want) <= rel * np.abs(want) + ab)
    assert float(buf_out[0]) == 7.0 and torch.all(buf_out[1 + rows * cols:] == 7.0)


@pytest.mark.parametrize("cols", [20000, 120000])
def test_long_rows_in_place_nan_and_infinities(cols):
    from byteir_amd import ops
    x = torch.randn((4, cols), device="cuda")
    x[1, cols // 3] = float("nan")
    x[2, :] = -float("inf")
    x[3, : cols - 5] = -float("inf")   # every lane but a few sees only -inf
    x = torch.cat([x, x[3:4].clone()])
    x[4, 8:16] = float("nan")          # a lane that sees nothing but -inf and NaN must still pass the NaN on
    want = oracle.softmax(host(x))
    y = host(ops.softmax(x, x))        # in place
    assert np.all(np.isnan(y[1])) and np.all(np.isnan(y[2])) and np.all(np.isnan(y[4]))
    assert np.array_equal(np.isnan(y), np.isnan(want))
    assert np.abs(y[0] - want[0]).max() <= 1e-5 * want[0].max() + 1e-10
    assert np.all(y[3, : cols - 5] == 0) and abs(float(y[3].sum()) - 1.0) < 1e-5


def test_softmax_properties_f32():
    from byteir_amd import ops
    x = dev((np.random.default_rng(3).standard_normal((256, 4096)) * 2).astype(np.float32))
    y = ops.softmax(x)
    assert torch.allclose(y.sum(dim=-1, dtype=torch.float64), torch.ones(256, dtype=torch.float64, device="cuda"), atol=1e-5)
    xc = torch.round(x * 64) / 64
    assert torch.equal(ops.softmax(xc), ops.softmax(xc + 8.0))  # shift invariance, exact for coarse values
    hot = torch.zeros((2, 1000), device="cuda")
    hot[0, 7] = 200.0
    hot[1, :] = -1e30
    hot[1, 3] = 1e30
    out = ops.softmax(hot)
    assert out[0, 7] == 1 and out[0].sum() == 1 and out[1, 3] == 1 and out[1].sum() == 1


def test_softmax_in_place_and_nan_row():
    from byteir_amd import ops
    x = (np.random.default_rng(4).standard_normal((9, 512))).astype(np.float32)
    x[4, 17] = np.nan
    d = dev(x)
    want = host(ops.softmax(d))
    ops.softmax(d, out=d)
    got = host(d)
    assert np.array_equal(got, want, equal_nan=True)
    assert np.isnan(got[4]).all() and not np.isnan(np.delete(got, 4, axis=0)).any()


def test_baseline_config3_full_size():
    """[32768, 4096] bf16 ~ N(0, 4): compare 2048 sampled rows with the oracle, and check every
    row sums to one within bf16 rounding of 4096 terms."""
    from byteir_amd import ops
    rng = np.random.default_rng(0xC3)
    x32 = (rng.standard_normal((32768, 4096), dtype=np.float32) * 2)
    xs = oracle.to_bf16_bits(x32)
    y = ops.softmax(dev(xs))
    rows = rng.choice(32768, 2048, replace=False)
    got = oracle.to_f32(host(y[torch.from_numpy(rows).cuda()]))
    want = oracle.to_f32(oracle.softmax(xs[rows]))
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + 1e-38)
    assert (got == want).mean() > 0.98
    sums = y.float().sum(dim=-1, dtype=torch.float64)
    assert float((sums - 1).abs().max()) < 4096 * 2.0 ** -9 * 0.05 + 1e-2


def test_random_shapes_sweep():
    """Thirty seeded random [A, B, C] softmaxes over B (C = 1: rows of any length and alignment;
    C > 1: an inner axis), all storage types, against the fp64 closed form."""
    from byteir_amd import ops
    rng = np.random.default_rng(77)
    for case in range(30):
        A = int(rng.choice([1, 2, 5, 40]))
        B = int(rng.choice([1, 3, 17, 130, 1000, 4097, 9001, 33000, 70003]))
        C = int(rng.choice([1, 1, 1, 2, 7, 24, 128, 1030]))
        while A * B * C > 2_000_000:
            if A > 1: A //= 2
            elif C > 1: C //= 2
            else: B //= 2
        code = [oracle.F32, oracle.F16, oracle.BF16][case % 3]
        x32 = (rng.standard_normal((A, B, C)) * 2.0).astype(np.float32)
        xs = oracle.from_f32(x32, code)
        got = oracle.to_f32(host(ops.softmax(dev(xs), axis=1)))
        want = sp_softmax(oracle.to_f32(xs).astype(np.float64), axis=1).astype(np.float32)
        rel, ab = TOL[code]
        assert np.all(np.abs(got - want) <= rel * np.abs(want) + ab), (case, A, B, C, code)
