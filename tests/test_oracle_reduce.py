"""Pins the reduction part of the CPU oracle (shape rule, workspace rule, values)."""
import itertools

import numpy as np
import pytest

import oracle

# shape list of the reference's own test,
# runtime/test/backends/cuda/providers/default/kernel/reduction_test.cc:171-180
REF_CASES = [
    ((1, 16, 32), (0,)), ((1, 16, 32), (1,)), ((1, 16, 32), (2,)), ((1, 16, 32), (0, 1)),
    ((1, 16, 32), (0, 2)), ((1, 128, 128), (0, 1)), ((2, 128, 256), (0, 1)), ((2, 16, 8, 64), (1, 2)),
]


def brute_force(x, dims, fold, init):
    """Index-decode fold, the shape of GoldenReduction (reduction_test.cc:39-92):
    walk the input linearly, route every element to its output by dropping reduced axes."""
    out_shape = [s for i, s in enumerate(x.shape) if i not in dims]
    out = np.full(int(np.prod(out_shape)) if out_shape else 1, init, dtype=x.dtype)
    for lin, val in enumerate(x.reshape(-1)):
        idx = np.unravel_index(lin, x.shape)
        o = 0
        for i, s in enumerate(x.shape):
            if i not in dims:
                o = o * s + idx[i]
        out[o] = fold(out[o], val)
    return out.reshape(out_shape)


@pytest.mark.parametrize("shape,dims", REF_CASES)
def test_reference_shape_list_abc_and_values(shape, dims):
    rng = np.random.default_rng(1)
    x = rng.random(shape, dtype=np.float32)  # [0,1) like the reference's RandCUDABuffer
    out_shape = oracle.deduce_output_shape(shape, dims)
    assert out_shape == [s for i, s in enumerate(shape) if i not in dims]
    st, A, B, C = oracle.reduce_canonicalize(shape, out_shape, dims)
    assert st == 0
    # closed form: with size-1 dims stripped, A/B/C are the products before / over / after
    live = sorted(d for d in dims if shape[d] != 1)
    if live:
        assert A == int(np.prod(shape[:live[0]])) and C == int(np.prod(shape[live[-1] + 1:]))
        assert B == int(np.prod([shape[d] for d in live]))
    else:  # {1,16,32} over {0}: nothing left to reduce -> copy of all elements
        assert (A, B, C) == (0, 0, int(np.prod(shape)))
    got_sum = oracle.reduce_op(oracle.SUM, x, dims)
    got_max = oracle.reduce_op(oracle.MAX, x, dims)
    if x.size <= 8192:
        bf_sum = brute_force(x, dims, lambda a, b: np.float32(a + b), np.float32(0))
        assert np.array_equal(got_sum, bf_sum)  # same sequential float chain -> bit equal
        bf_max = brute_force(x, dims, max, np.float32(-np.inf))
        assert np.array_equal(got_max, bf_max)
    np.testing.assert_allclose(got_sum, x.astype(np.float64).sum(axis=dims), rtol=1e-5, atol=1e-4)
    assert np.array_equal(got_max, x.max(axis=dims))


def test_canonicalize_rules():
    # unsorted dims are sorted (resnet18_fw_bw_host_cuda.mlir:178 has dense<[3, 2]>)
    assert oracle.reduce_canonicalize((4, 8, 3, 5), (4, 8), (3, 2)) == (0, 32, 15, 1)
    # size-1 dims are dropped before the consecutive check: {0,2} over [1,16,32] is fine
    assert oracle.reduce_canonicalize((1, 16, 32), (16,), (0, 2)) == (0, 16, 32, 1)
    # genuinely non-consecutive -> rejected (reduce_impl.h:41-42)
    assert oracle.reduce_canonicalize((2, 16, 32), (16,), (0, 2))[0] == 2
    # keep-dims style output shape is rejected (reduce_impl.h:35)
    assert oracle.reduce_canonicalize((4, 8), (4, 1), (1,))[0] == 1
    # nothing left to reduce -> A=B=0, C=numel (plain copy)
    assert oracle.reduce_canonicalize((1, 7, 1), (7,), (0, 2)) == (0, 0, 0, 7)
    # out-of-range dimension
    assert oracle.reduce_canonicalize((4, 8), (4,), (2,))[0] == 3
    # benchmark shapes
    assert oracle.reduce_canonicalize((4096, 1024), (4096,), (1,)) == (0, 4096, 1024, 1)
    assert oracle.reduce_canonicalize((16384, 8192), (8192,), (0,)) == (0, 1, 16384, 8192)
    assert oracle.reduce_canonicalize((16384, 8192), (16384,), (1,)) == (0, 16384, 8192, 1)


def test_copy_case_values():
    x = np.arange(7, dtype=np.float32).reshape(1, 7, 1)
    assert np.array_equal(oracle.reduce_op(oracle.SUM, x, (0, 2)), x.reshape(7))


def test_path_and_workspace_rule():
    # .../reduction/kernels/reduction.cu:411-413
    assert oracle.use_reduce_column(4096, 1024, 1)
    assert oracle.use_reduce_column(16384, 8192, 1)
    assert not oracle.use_reduce_column(1, 16384, 8192)
    assert oracle.use_reduce_column(1, 32, 1) and not oracle.use_reduce_column(1, 33, 1)
    # closed form for the tall case: BX=32, BY=16, f=64: 16384 -> 256 -> 4 -> 1 (3 passes),
    # workspace 4 * (256 + 4) * 8192 bytes
    assert oracle.reference_workspace_bytes(1, 16384, 8192, 4) == 4 * (256 + 4) * 8192 == 8519680
    assert oracle.reference_workspace_bytes(4096, 1024, 1, 4) == 0
    # one pass when B <= f
    assert oracle.reference_workspace_bytes(2, 64, 32, 4) == 0
    # two passes: C=1 -> BX=1, BY=512, f=2048; B=4096 -> 2 -> 1
    assert oracle.reference_workspace_bytes(1, 4096, 1, 4) == 4 * 1 * 2 * 1
    # the f16 quirk: sized with sizeof(T)=2 although used as float
    assert oracle.reference_workspace_bytes(1, 16384, 8192, 2) == 2 * (256 + 4) * 8192


@pytest.mark.parametrize("op", [oracle.SUM, oracle.MAX])
@pytest.mark.parametrize("pos", [0, 511, 1023])
def test_nan_propagation(op, pos):
    # reduction_test.cc:182-215 puts the NaN first; also last and middle here
    x = np.random.default_rng(2).random(1024, dtype=np.float32)
    x[pos] = np.nan
    assert np.isnan(oracle.reduce_op(op, x, (0,)))


def test_max_identity_and_infinities():
    x = np.full((3, 5), -np.inf, dtype=np.float32)
    assert np.array_equal(oracle.reduce_op(oracle.MAX, x, (1,)), np.full(3, -np.inf, np.float32))
    x[1, 2] = np.inf
    assert oracle.reduce_op(oracle.MAX, x, (1,))[1] == np.inf


def test_sum_f64_and_f16():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((64, 300, 5)).astype(np.float32)
    s64, sabs = oracle.reduce_sum_f64(x, 64, 300, 5)
    np.testing.assert_allclose(s64.reshape(64, 5), x.astype(np.float64).sum(axis=1), rtol=1e-12)
    np.testing.assert_allclose(sabs.reshape(64, 5), np.abs(x.astype(np.float64)).sum(axis=1), rtol=1e-12)
    # f16 storage accumulates in float and rounds once (reduce_impl.h:64-69)
    xh = x.astype(np.float16)
    got = oracle.reduce_op(oracle.SUM, xh, (1,))
    want = xh.astype(np.float32).sum(axis=1, dtype=np.float64)
    assert got.dtype == np.float16
    np.testing.assert_allclose(got.astype(np.float64), want, rtol=2e-3, atol=2e-3)
    assert np.array_equal(oracle.reduce_op(oracle.MAX, xh, (1,)), xh.max(axis=1))


def test_half_conversions_exhaustive():
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    as_f16 = bits.view(np.float16)
    f = np.array([L.oracle_h2f(int(b)) for b in bits[::7]], dtype=np.float32)
    assert np.array_equal(f, as_f16[::7].astype(np.float32), equal_nan=True)
    rng = np.random.default_rng(4)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0, -0.0, 65504, 65519.99, 65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, np.inf, -np.inf], np.float32),
    ])
    got = np.empty(vals.shape, np.float16)
    L.oracle_convert_from_f32(vals.ctypes.data, got.ctypes.data, vals.size, oracle.F16)
    assert np.array_equal(got.view(np.uint16), vals.astype(np.float16).view(np.uint16))
    # bf16: RNE on the top 16 bits; check against an integer closed form
    u = vals.view(np.uint32).astype(np.uint64)
    want = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    finite = np.isfinite(vals)
    assert np.array_equal(oracle.to_bf16_bits(vals)[finite], want[finite])
    assert np.array_equal(oracle.from_bf16_bits(want), (want.astype(np.uint32) << 16).view(np.float32))


# ---- the operators the reference defines but never registers (reduction_helper.h:37-137) -------
def test_min_prod_mean_sumsqr_against_closed_forms():
    """Pins chosen so that a swapped init, a missing division, a square of the sum instead of a
    sum of squares or a min that behaves like max each fail: integers small enough that every
    float operation is exact, so numpy's integer arithmetic is the expected value bit for bit."""
    rng = np.random.default_rng(11)
    xi = rng.integers(-9, 10, size=(6, 64, 5))
    x = xi.astype(np.float32)
    assert np.array_equal(oracle.reduce_op(oracle.MIN, x, (1,)), xi.min(axis=1).astype(np.float32))
    assert np.array_equal(oracle.reduce_op(oracle.SUMSQR, x, (1,)), (xi * xi).sum(axis=1).astype(np.float32))
    # 64 is a power of two: sum / 64 is exact
    assert np.array_equal(oracle.reduce_op(oracle.MEAN, x, (1,)), (xi.sum(axis=1) / 64.0).astype(np.float32))
    # products of +-1 and +-2 stay exact powers of two
    pi = rng.choice(np.array([-2, -1, 1, 2]), size=(4, 40, 3))
    assert np.array_equal(oracle.reduce_op(oracle.PROD, pi.astype(np.float32), (1,)),
                          pi.astype(np.float64).prod(axis=1).astype(np.float32))
    # a fold length that is no power of two: one float division of the float sum by float(B)
    y = rng.integers(-50, 50, size=(3, 7)).astype(np.float32)
    want = (y.sum(axis=1, dtype=np.float32) / np.float32(7)).astype(np.float32)
    assert np.array_equal(oracle.reduce_op(oracle.MEAN, y, (1,)), want)


def test_min_identity_nan_and_empty_product():
    x = np.full((2, 9), np.inf, dtype=np.float32)
    assert np.array_equal(oracle.reduce_op(oracle.MIN, x, (1,)), np.full(2, np.inf, np.float32))
    x[1, 4] = -np.inf
    assert oracle.reduce_op(oracle.MIN, x, (1,))[1] == -np.inf
    for pos in (0, 4, 8):  # NaN from either side of apply wins
        z = np.arange(9, dtype=np.float32)
        z[pos] = np.nan
        assert np.isnan(oracle.reduce_op(oracle.MIN, z, (0,)))
        assert np.isnan(oracle.reduce_op(oracle.PROD, z, (0,)))
    # f16 storage: squares and the chain are float, one rounding at the store
    h = np.array([[255.0, 3.0, 0.5]], dtype=np.float16)  # 255^2 = 65025 rounds to 65024 in f16
    got = oracle.reduce_op(oracle.SUMSQR, h, (1,))
    assert got.dtype == np.float16 and got[0] == np.float16(65025.0 + 9.0 + 0.25)


def test_tensors_without_elements():
    """An empty fold axis gives the operator's identity; no output element, nothing written."""
    x = np.empty((4, 0, 8), dtype=np.float32)
    want = {oracle.SUM: 0.0, oracle.MAX: -np.inf, oracle.MIN: np.inf, oracle.PROD: 1.0, oracle.SUMSQR: 0.0}
    for op, v in want.items():
        assert np.array_equal(oracle.reduce_op(op, x, (1,)), np.full((4, 8), v, np.float32))
    assert np.all(np.isnan(oracle.reduce_op(oracle.MEAN, x, (1,))))
    assert oracle.reduce_op(oracle.SUM, np.empty((0, 5), np.float32), (1,)).shape == (0,)
    assert oracle.reduce_op(oracle.SUM, np.empty((3, 5, 0), np.float32), (1,)).shape == (3, 0)


@pytest.mark.parametrize("shape,dims", [((7, 13), (1,)), ((5, 333, 7), (1,)), ((4096, 64), (0,)), ((300, 2600), (0,)), ((16, 2049, 260), (1,))])
@pytest.mark.parametrize("op", [oracle.MIN, oracle.PROD, oracle.MEAN, oracle.SUMSQR])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_integer_arithmetic_fold_agrees_with_the_oracle(shape, dims, op, dtype):
    """exact_fold (numpy integer arithmetic) is what the GPU tests compare the large f16 shapes
    with, where the scalar oracle would take minutes: on the shapes the oracle does finish, the
    two must agree bit for bit."""
    from reduce_exact import exact_fold, exact_input
    rng = np.random.default_rng(abs(hash((shape, dims, op))) % (2 ** 32))
    x = exact_input(op, shape, dims, rng).astype(dtype)
    assert np.array_equal(exact_fold(op, x, dims), oracle.reduce_op(op, x, dims))
