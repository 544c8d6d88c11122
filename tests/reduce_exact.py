"""Inputs on which a float fold is exact in any order, and their folds by integer arithmetic:
shared by the GPU reduce tests and the oracle's own tests."""
import numpy as np

import oracle


def exact_input(op, shape, dims, rng):
    """Values for which every partial result of the fold is exact in float whatever the order,
    so that the sequential oracle is the expected value bit for bit: small integers for
    min / mean / sum of squares; for the product, signs and a few factors of 2 and 1/2."""
    if op != oracle.PROD:
        return rng.integers(-2, 3, size=shape).astype(np.float32)
    fold = int(np.prod([shape[d] for d in dims]))
    e = rng.integers(-1, 2, size=shape) * (rng.random(shape) < min(1.0, 24.0 / fold))
    return (np.exp2(e) * rng.choice(np.array([-1.0, 1.0]), size=shape)).astype(np.float32)


def exact_fold(op, x, dims):
    """The fold of exact_input values by integer arithmetic in numpy (every intermediate is an
    integer or a power of two, exact in float64), then the operator's one float step and one
    rounding to the storage type -- what a float fold in any order gives.  The small shapes check
    this against the oracle too (test_exact_fold_agrees_with_the_oracle)."""
    x64 = x.astype(np.float64)
    n = int(np.prod([x.shape[d] for d in dims]))
    if op == oracle.MIN:
        r = x64.min(axis=dims).astype(np.float32)
    elif op == oracle.SUMSQR:
        r = (x64 * x64).sum(axis=dims).astype(np.float32)
    elif op == oracle.MEAN:
        r = x64.sum(axis=dims).astype(np.float32) / np.float32(n)
    else:  # signs and powers of two: add the exponents, count the minus signs
        e = np.log2(np.abs(x64)).sum(axis=dims)
        neg = (x64 < 0).sum(axis=dims) % 2
        r = (np.exp2(e) * np.where(neg == 1, -1.0, 1.0)).astype(np.float32)
    return r.astype(x.dtype)
