"""GPU parity of the HIP reductions against the CPU oracle, through the C ABI.

Mirrors the reference's CUDATestReductionOp tests
(runtime/test/backends/cuda/providers/default/kernel/reduction_test.cc:94-230): the same shape
list, two runs on the same buffers, NaN propagation; plus the full-size benchmark shapes."""
import numpy as np
import pytest
import torch

import oracle
from reduce_exact import exact_fold, exact_input
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

REF_CASES = [
    ((1, 16, 32), (0,)), ((1, 16, 32), (1,)), ((1, 16, 32), (2,)), ((1, 16, 32), (0, 1)),
    ((1, 16, 32), (0, 2)), ((1, 128, 128), (0, 1)), ((2, 128, 256), (0, 1)), ((2, 16, 8, 64), (1, 2)),
]
# ragged / odd shapes: scalar-load paths, tails, tiny and long fold axes, split passes
EXTRA_CASES = [
    ((7, 13), (1,)), ((7, 13), (0,)), ((3, 1000003), (1,)), ((1000003, 3), (0,)), ((5, 333, 7), (1,)),
    ((1, 1 << 20), (1,)), ((1 << 20,), (0,)), ((64, 4096), (1,)), ((4096, 64), (0,)), ((2, 5000, 36), (1,)),
    ((129, 1024), (1,)), ((1, 70000, 8), (1,)), ((300, 40), (1,)), ((16, 2049, 260), (1,)),
    # wide rows (8 KiB of a row per block): whole tiles, a ragged last tile, few rows
    ((4096, 8192), (0,)), ((300, 2600), (0,)), ((5, 40, 4104), (1,)), ((3, 2048), (0,)),
]


def check_sum(got, x, A, B, C):
    """north_star tolerance: 1e-5 relative against the fp64 fold, measured on the scale of
    sum|x| (a sum of signed values can be arbitrarily close to zero), plus the reference
    test's own atol 1e-4 / rtol 1e-5 against the sequential float oracle."""
    s64, sabs = oracle.reduce_sum_f64(x, A, B, C)
    got64 = got.reshape(-1).astype(np.float64)
    assert np.all(np.abs(got64 - s64) <= 1e-5 * np.maximum(np.abs(s64), 1e-2 * sabs) + 1e-30)
    if B <= 4096:  # a longer float chain drifts further from the fp64 fold than the tolerance
        seq = oracle.reduce_abc(oracle.SUM, x, A, B, C).astype(np.float64)
        assert np.all(np.abs(got64 - seq) <= 1e-4 + 1e-5 * np.maximum(np.abs(seq), sabs * 1e-1))


@pytest.mark.parametrize("shape,dims", REF_CASES + EXTRA_CASES)
@pytest.mark.parametrize("op", [oracle.SUM, oracle.MAX])
def test_reduce_f32_matches_oracle_twice(shape, dims, op):
    from byteir_amd import ops
    rng = np.random.default_rng(abs(hash((shape, dims))) % (2 ** 32))
    out_shape = oracle.deduce_output_shape(shape, dims)
    st, A, B, C = oracle.reduce_canonicalize(shape, out_shape, dims)
    assert st == 0
    assert ops.canonicalize_reduce(list(shape), out_shape, list(dims)) == (A, B, C)
    need = ops.reduce_workspace_bytes(torch.float32, A, B, C)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    out = torch.empty(out_shape, dtype=torch.float32, device="cuda")
    for run in range(2):  # second run on the same buffers and workspace (reduction_test.cc:147-164)
        x = (rng.random(shape, dtype=np.float32) if run == 0
             else rng.standard_normal(shape).astype(np.float32))
        dx = dev(x)
        ops.reduce_abc(op, dx, out, A, B, C, workspace=ws)
        got = host(out)
        if op == oracle.MAX or not (A and B and C):
            assert np.array_equal(got, oracle.reduce_op(op, x, dims))
        else:
            check_sum(got, x, A, B, C)


@pytest.mark.parametrize("op", [oracle.SUM, oracle.MAX])
@pytest.mark.parametrize("shape,dims,pos", [((1024,), (0,), 0), ((1024,), (0,), 1023), ((4, 1 << 18), (1,), 77777),
                                            ((1 << 16, 16), (0,), 12345)])
def test_nan_propagation(op, shape, dims, pos):
    from byteir_amd import ops
    x = np.random.default_rng(1).random(shape, dtype=np.float32)
    x.reshape(-1)[pos] = np.nan
    got = host(ops.reduce(op, dev(x), dims))
    want = oracle.reduce_op(op, x, dims)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(got).any()
    ok = ~np.isnan(want)
    if op == oracle.MAX:
        assert np.array_equal(got[ok], want[ok])


def test_max_of_all_minus_inf_and_inf():
    from byteir_amd import ops
    x = np.full((33, 777), -np.inf, np.float32)
    x[5, 100] = np.inf
    got = host(ops.reduce(oracle.MAX, dev(x), (1,)))
    assert np.array_equal(got, x.max(axis=1))


@pytest.mark.parametrize("shape,dims", [((64, 4096), (1,)), ((4096, 64), (0,)), ((3, 1001, 5), (1,)), ((1, 200000), (1,)),
                                        ((2, 16, 8, 64), (1, 2)), ((2000, 4104), (0,)), ((7, 8192), (0,))])
@pytest.mark.parametrize("op", [oracle.SUM, oracle.MAX])
def test_reduce_f16(shape, dims, op):
    from byteir_amd import ops
    x = np.random.default_rng(2).standard_normal(shape).astype(np.float16)
    got = host(ops.reduce(op, dev(x), dims))
    assert got.dtype == np.float16
    if op == oracle.MAX:
        assert np.array_equal(got, oracle.reduce_op(op, x, dims))
    else:  # folded in float, rounded once: within one fp16 ulp of the fp64 fold
        want = x.astype(np.float64).sum(axis=dims)
        sabs = np.abs(x.astype(np.float64)).sum(axis=dims)
        assert np.all(np.abs(got.astype(np.float64) - want) <= 2.0 ** -10 * np.abs(want) + 1e-6 * sabs + 1e-7)


# ---- MinOp, ProdOp, MeanOp, SumSqrOp (reduction_helper.h:37-137) ------------------------------
OTHER_OPS = [oracle.MIN, oracle.PROD, oracle.MEAN, oracle.SUMSQR]
OTHER_SHAPES = REF_CASES + [
    ((7, 13), (1,)), ((7, 13), (0,)), ((3, 1000003), (1,)), ((1000003, 3), (0,)), ((5, 333, 7), (1,)),
    ((1 << 20,), (0,)), ((4096, 64), (0,)), ((16, 2049, 260), (1,)), ((4096, 8192), (0,)), ((300, 2600), (0,)),
]


@pytest.mark.parametrize("shape,dims", OTHER_SHAPES)
@pytest.mark.parametrize("op", OTHER_OPS)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_other_operators_bit_exact_on_exact_inputs(shape, dims, op, dtype):
    from byteir_amd import ops
    rng = np.random.default_rng(abs(hash((shape, dims, op))) % (2 ** 32))
    x = exact_input(op, shape, dims, rng).astype(dtype)
    got = host(ops.reduce(op, dev(x), dims))
    if dtype == np.float16 and int(np.prod(shape)) > (1 << 22):
        want = exact_fold(op, x, dims)  # the scalar f16 oracle takes minutes at this size
    else:
        want = oracle.reduce_op(op, x, dims)
    assert got.dtype == dtype and got.shape == want.shape
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape,dims", [((64, 4096), (1,)), ((4096, 64), (0,)), ((3, 100003), (1,)), ((5000, 2600), (0,))])
def test_other_operators_on_real_values(shape, dims):
    """1e-5 relative against the fp64 fold (the bar of the registered sum)."""
    from byteir_amd import ops
    rng = np.random.default_rng(5)
    x = rng.standard_normal(shape).astype(np.float32)
    x64 = x.astype(np.float64)
    n = int(np.prod([shape[d] for d in dims]))
    got = host(ops.reduce(oracle.SUMSQR, dev(x), dims)).astype(np.float64)
    np.testing.assert_allclose(got, (x64 * x64).sum(axis=dims), rtol=1e-5)
    got = host(ops.reduce(oracle.MEAN, dev(x), dims)).astype(np.float64)
    assert np.all(np.abs(got - x64.mean(axis=dims)) <= 1e-5 * 1e-2 * np.abs(x64).sum(axis=dims) / n)
    assert np.array_equal(host(ops.reduce(oracle.MIN, dev(x), dims)), x.min(axis=dims))
    # factors near one: the product stays in range and its rounding error is that of a
    # chain of n multiplications in any order, at most n * 2^-24 relative
    y = (1.0 + 1e-3 * rng.standard_normal(shape)).astype(np.float32)
    got = host(ops.reduce(oracle.PROD, dev(y), dims)).astype(np.float64)
    np.testing.assert_allclose(got, y.astype(np.float64).prod(axis=dims), rtol=max(1e-5, n * 2.0 ** -24))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_tensors_without_elements(dtype):
    """An empty fold axis writes the operator's identity to every output; a tensor with no
    output element writes nothing (the reference would copy from an input without elements)."""
    from byteir_amd import ops
    x = np.empty((4, 0, 8), dtype=dtype)
    for op in (oracle.SUM, oracle.MAX, oracle.MIN, oracle.PROD, oracle.SUMSQR):
        assert np.array_equal(host(ops.reduce(op, dev(x), (1,))), oracle.reduce_op(op, x, (1,)))
    assert np.all(np.isnan(host(ops.reduce(oracle.MEAN, dev(x), (1,)))))
    assert ops.reduce(oracle.SUM, dev(np.empty((0, 5), dtype)), (1,)).shape == (0,)
    assert ops.reduce(oracle.MAX, dev(np.empty((3, 5, 0), dtype)), (1,)).shape == (3, 0)
    assert ops.reduce(oracle.SUM, dev(np.empty((0, 1, 5), dtype)), (1,)).shape == (0, 5)  # the copy branch, no element


def test_min_nan_and_infinities():
    from byteir_amd import ops
    x = np.full((3, 70000), np.inf, dtype=np.float32)
    assert np.array_equal(host(ops.reduce(oracle.MIN, dev(x), (1,))), np.full(3, np.inf, np.float32))
    x[1, 69999] = -np.inf
    x[2, 12345] = np.nan
    got = host(ops.reduce(oracle.MIN, dev(x), (1,)))
    assert got[0] == np.inf and got[1] == -np.inf and np.isnan(got[2])
    got = host(ops.reduce(oracle.MIN, dev(x), (0,)))
    assert np.isnan(got[12345]) and got[69999] == -np.inf and got[0] == np.inf


@pytest.mark.parametrize("shape,dims", [((1000, 4096), (0,)), ((1000, 4096), (1,)), ((3000, 64), (0,)), ((2, 500, 2048), (1,)),
                                        ((40000, 8), (0,))])
@pytest.mark.parametrize("op", [oracle.SUM, oracle.MAX])
def test_input_that_is_not_16_byte_aligned(shape, dims, op):
    """Extents that allow 128-bit loads but a pointer that does not: the launch falls back to
    scalar loads and must still cover every column."""
    from byteir_amd import ops
    n = int(np.prod(shape))
    x = np.random.default_rng(9).standard_normal(n).astype(np.float32)
    buf = torch.zeros(n + 1, device="cuda")
    buf[1:] = dev(x)
    view = buf[1:].view(shape)
    assert view.data_ptr() % 16 == 4
    got = host(ops.reduce(op, view, dims))
    xs = x.reshape(shape)
    if op == oracle.MAX:
        assert np.array_equal(got, xs.max(axis=dims[0]))
    else:
        out_shape = oracle.deduce_output_shape(shape, dims)
        st, A, B, C = oracle.reduce_canonicalize(shape, out_shape, dims)
        check_sum(got, xs, A, B, C)


def test_workspace_too_small_is_an_error():
    from byteir_amd import _lib, ops
    A, B, C = 1, 16384, 8192
    need = ops.reduce_workspace_bytes(torch.float32, A, B, C)
    assert need > 0
    x = torch.zeros((B, C), device="cuda")
    out = torch.zeros(C, device="cuda")
    with pytest.raises(RuntimeError):
        ops.reduce_abc(oracle.SUM, x, out, A, B, C, workspace=torch.empty(need - 1, dtype=torch.uint8, device="cuda"))
    torch.cuda.synchronize()


def test_baseline_config1_row_sum():
    """[4096, 1024] f32 ~ N(0,1), reduce axis 1 (the first benchmark configuration)."""
    from byteir_amd import ops
    x = np.random.default_rng(0xC1).standard_normal((4096, 1024)).astype(np.float32)
    got = host(ops.reduce(oracle.SUM, dev(x), (1,)))
    check_sum(got, x, 4096, 1024, 1)


def test_baseline_config2_full_size():
    """[16384, 8192] f32 ~ U(-1,1): Max and Sum over axis 0 (two-pass split) and over axis 1.
    Max is compared exactly with numpy at full size; Sum against the fp64 fold."""
    from byteir_amd import ops
    rng = np.random.default_rng(0xC2)
    x = rng.random((16384, 8192), dtype=np.float32) * 2 - 1
    dx = dev(x)
    for dims, (A, B, C) in (((0,), (1, 16384, 8192)), ((1,), (16384, 8192, 1))):
        assert np.array_equal(host(ops.reduce(oracle.MAX, dx, dims)), x.max(axis=dims[0]))
        got = host(ops.reduce(oracle.SUM, dx, dims)).astype(np.float64)
        want = x.sum(axis=dims[0], dtype=np.float64)
        sabs = np.abs(x).sum(axis=dims[0], dtype=np.float64)
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(np.abs(want), 1e-2 * sabs))
    # linearity (size-independent property): sum(2x) == 2 sum(x) bit for bit
    s1 = ops.reduce(oracle.SUM, dx, (0,))
    s2 = ops.reduce(oracle.SUM, dx * 2, (0,))
    assert torch.equal(s2, s1 * 2)


def test_random_shapes_sweep():
    """Forty seeded random [A, B, C] views (odd extents, tiny and long axes, both storage types,
    unaligned base pointers): sum within the documented tolerance, max and min bit-exact."""
    from byteir_amd import ops
    rng = np.random.default_rng(2024)
    for case in range(40):
        A = int(rng.choice([1, 2, 3, 7, 64, 300]))
        B = int(rng.choice([1, 2, 5, 33, 127, 1000, 4099, 70001]))
        C = int(rng.choice([1, 1, 1, 2, 3, 8, 33, 260, 1027]))
        while A * B * C > 3_000_000:
            if A > 1: A //= 2
            elif C > 1: C //= 2
            else: B //= 2
        dtype = np.float16 if case % 3 == 2 else np.float32
        off = int(rng.integers(0, 4))  # elements into the allocation: 16-byte alignment is not a given
        x = rng.standard_normal(A * B * C).astype(dtype)
        buf = torch.zeros(A * B * C + 8, dtype=torch.float16 if dtype == np.float16 else torch.float32, device="cuda")
        view = buf[off:off + A * B * C]
        view.copy_(dev(x))
        for op in (oracle.SUM, oracle.MAX, oracle.MIN):
            out = torch.empty(A * C, dtype=view.dtype, device="cuda")
            ops.reduce_abc(op, view, out, A, B, C)
            got = host(out)
            want = oracle.reduce_abc(op, x, A, B, C)
            if op == oracle.SUM:
                x64 = x.astype(np.float64).reshape(A, B, C)
                s64, sabs = x64.sum(axis=1).reshape(-1), np.abs(x64).sum(axis=1).reshape(-1)
                tol = (2.0 ** -10 * np.abs(s64) + 1e-6 * sabs + 1e-7) if dtype == np.float16 else (1e-5 * np.maximum(np.abs(s64), 1e-2 * sabs) + 1e-30)
                assert np.all(np.abs(got.astype(np.float64) - s64) <= tol), (case, A, B, C, dtype, off)
            else:
                assert np.array_equal(got, want), (case, op, A, B, C, dtype, off)
