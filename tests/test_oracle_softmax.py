"""Pins the softmax part of the CPU oracle against scipy and closed forms."""
import numpy as np
import pytest
from scipy.special import softmax as sp_softmax

import oracle


@pytest.mark.parametrize("shape", [(10, 128), (8 * 12 * 4, 256), (3, 1), (5, 4097)])
def test_f32_against_scipy_f64(shape):
    # 10x128 and ...x256x256 are the reference's own softmax test shapes
    # (tests/numerical_test/mlir_tests/cpu_ops/custom_call_byteir_softmax.mlir, .../ops/softmax.mlir)
    x = (np.random.default_rng(5).standard_normal(shape) * 2).astype(np.float32)
    got = oracle.softmax(x)
    want = sp_softmax(x.astype(np.float64), axis=-1)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-9)  # float chain over <=4097 terms
    np.testing.assert_allclose(got.sum(axis=-1, dtype=np.float64), 1.0, atol=1e-5)


def test_shift_invariance_and_one_hot():
    x = np.random.default_rng(6).standard_normal((16, 512)).astype(np.float32)
    # softmax(x + c) == softmax(x); a power-of-two shift of already-coarse values is exact
    xc = (np.round(x * 64) / 64).astype(np.float32)
    assert np.array_equal(oracle.softmax(xc), oracle.softmax(xc + np.float32(8.0)))
    # one-hot limit: a dominant entry takes all the mass, without overflow
    y = np.zeros((2, 100), np.float32)
    y[0, 7] = 200.0
    y[1, :] = -1e30
    y[1, 3] = 1e30
    out = oracle.softmax(y)
    assert out[0, 7] == 1.0 and out[0].sum() == 1.0
    assert out[1, 3] == 1.0 and out[1].sum() == 1.0
    # uniform row
    assert np.allclose(oracle.softmax(np.zeros((1, 64), np.float32)), 1 / 64)


@pytest.mark.parametrize("code", [oracle.F16, oracle.BF16])
def test_16bit_storage_rounds_once(code):
    x32 = (np.random.default_rng(7).standard_normal((64, 4096)) * 2).astype(np.float32)
    xs = oracle.from_f32(x32, code)
    got = oracle.to_f32(oracle.softmax(xs))
    want64 = sp_softmax(oracle.to_f32(xs).astype(np.float64), axis=-1)
    want = oracle.to_f32(oracle.from_f32(want64.astype(np.float32), code))
    ulp = 2.0 ** -7 if code == oracle.BF16 else 2.0 ** -10  # spacing / value upper bound
    # float internals, one rounding at the store: within one storage ulp of the fp64 result
    assert np.all(np.abs(got - want) <= ulp * np.abs(want) + 6e-8)  # 6e-8: fp16 subnormal spacing
    # and almost everywhere identical
    assert (got == want).mean() > 0.99
    np.testing.assert_allclose(got.sum(axis=-1, dtype=np.float64), 1.0, atol=4096 * 2.0 ** -9 * 1e-2 + 1e-2)
