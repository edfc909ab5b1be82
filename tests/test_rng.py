"""The numpy generator that bench.py draws its inputs from against the C generator of the oracle
(the one the parity tests use): the same counter-based numbers."""
import numpy as np

from ctorch_amd import rng


def test_uniform_and_ints_are_the_oracles_bits(oracle):
    for seed, n in ((101, 1000), (212, (1 << 22) + 37), (2 ** 40 + 5, 4096)):
        assert np.array_equal(rng.uniform((n,), seed, -1, 1), oracle.uniform((n,), seed, -1, 1))
        assert np.array_equal(rng.uniform((n,), seed, 0.5, 2), oracle.uniform((n,), seed, 0.5, 2))
        assert np.array_equal(rng.ints((n,), seed, 256), oracle.ints((n,), seed, 256))
        assert np.array_equal(rng.ints((n,), seed, 32000), oracle.ints((n,), seed, 32000))
    assert rng.uniform((3, 5), 7, -2, 2).shape == (3, 5)


def test_normal_agrees_to_the_last_bit_of_log_and_cos(oracle):
    from support import ulp_diff
    for seed, sigma in ((201, 1.0), (401, 2.0), (503, 1.0)):
        a, b = rng.normal((200000,), seed, 0.0, sigma), oracle.normal((200000,), seed, 0.0, sigma)
        big = np.abs(b) > 1e-3
        assert ulp_diff(a[big], b[big]).max() <= 1
        assert np.abs(a - b).max() <= 1e-9 + 2e-7 * np.abs(b).max()
    x = rng.normal((1 << 20,), 9, 0.0, 1.0).astype(np.float64)
    assert abs(x.mean()) < 5e-3 and abs(x.std() - 1.0) < 5e-3
