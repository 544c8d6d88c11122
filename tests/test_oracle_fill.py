"""The counter-based generator shared by the benchmark's GPU fill (brt_rocm_fill) and the CPU
oracle (oracle_fill): splitmix64 against its published outputs, the two distributions against
their moments, and the element-index contract (a slice of the sequence is the sequence)."""
import numpy as np

import oracle


def test_splitmix64_published_outputs():
    # the customary check values of splitmix64 seeded with 1234567 (e.g. the test vectors that
    # accompany Vigna's splitmix64.c in xoshiro ports)
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    got = [int(oracle.lib().oracle_splitmix64_at(1234567, i)) for i in range(5)]
    assert got == want


def test_splitmix64_is_the_textbook_loop():
    # x += golden; z = mix(x): the sequential generator, restated in Python integers
    M = (1 << 64) - 1
    x = 0xC2
    for i in range(100):
        x = (x + 0x9E3779B97F4A7C15) & M
        z = x
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        z ^= z >> 31
        assert int(oracle.lib().oracle_splitmix64_at(0xC2, i)) == z


def test_uniform_is_24_bits_on_the_interval():
    x = oracle.fill(0, oracle.UNIFORM, 0xC2, 1 << 20, -1.0, 1.0)
    assert x.dtype == np.float32 and x.min() >= -1.0 and x.max() < 1.0
    # every value is k * 2^-23 - 1 exactly
    k = (x.astype(np.float64) + 1.0) * (1 << 23)
    assert np.array_equal(k, np.round(k))
    assert abs(x.mean()) < 3e-3 and abs(x.var() - 1.0 / 3.0) < 3e-3
    # the top 24 bits of the generator, restated
    z = np.array([int(oracle.lib().oracle_splitmix64_at(0xC2, i)) >> 40 for i in range(64)], dtype=np.float64)
    assert np.array_equal(x[:64].astype(np.float64), z * 2.0 ** -23 - 1.0)


def test_normal_moments_and_exactness():
    x = oracle.fill(0, oracle.NORMAL, 0xC1, 1 << 20, 0.0, 1.0).astype(np.float64)
    assert abs(x.mean()) < 4e-3 and abs(x.std() - 1.0) < 4e-3
    assert abs(((x - x.mean()) ** 3).mean()) < 2e-2            # symmetric
    assert abs((x ** 4).mean() - (3.0 - 0.1)) < 5e-2           # Irwin-Hall(12) kurtosis 3 - 6/(5*12)
    assert np.array_equal(x * 65536.0, np.round(x * 65536.0))  # multiples of 2^-16: no rounding anywhere
    y = oracle.fill(0, oracle.NORMAL, 0xC1, 4096, 0.0, 2.0)
    assert np.array_equal(y.astype(np.float64), 2.0 * x[:4096])


def test_storage_types_round_once_and_slices_agree():
    f = oracle.fill(0, oracle.NORMAL, 0xC3, 5000, 0.0, 2.0)
    b = oracle.fill(2, oracle.NORMAL, 0xC3, 5000, 0.0, 2.0)
    h = oracle.fill(1, oracle.NORMAL, 0xC41, 5000, 0.0, 1.0)
    assert np.array_equal(b, oracle.to_bf16_bits(f))
    assert np.array_equal(h.view(np.float16), oracle.fill(0, oracle.NORMAL, 0xC41, 5000, 0.0, 1.0).astype(np.float16))
    part = oracle.fill(2, oracle.NORMAL, 0xC3, 100, 0.0, 2.0, first=1234)
    assert np.array_equal(part, b[1234:1334])
