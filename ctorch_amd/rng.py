"""Seeded inputs for benchmarks and full-size tests: a counter-based generator, the same numbers
on any machine and in any order of evaluation (the reference has no seedable one: its Tensor::rand
seeds from random_device, src/Tensor.cpp:463).

    z = mix(seed * 0x9E3779B97F4A7C15 + i)        i = flat element index, 64-bit wrap-around,
                                                  mix = the splitmix64 finaliser
    uniform[lo, hi]   float(lo + (hi - lo) * (z >> 40) * 2^-24)               (fp64 inside)
    normal(m, s)      Box-Muller in fp64 on the streams `seed` and `seed ^ 0xA5A5...`, cast to float
    ints(range)       z % range, as floats

numpy only.  uniform and ints are bit-identical to the C generator the tests' oracle uses; normal
agrees with it to the last bit of the fp64 log / cos of the two libraries (1 ulp of the float at most).
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_OTHER = np.uint64(0xA5A5A5A5A5A5A5A5)
_CHUNK = 1 << 22


def _draw(seed, start, count):
    with np.errstate(over="ignore"):
        z = np.uint64(seed) * _GOLDEN + np.arange(start, start + count, dtype=np.uint64)
        z ^= z >> np.uint64(30)
        z *= _M1
        z ^= z >> np.uint64(27)
        z *= _M2
        z ^= z >> np.uint64(31)
    return z


def _fill(shape, fn):
    n = int(np.prod(shape, dtype=np.int64)) if len(tuple(np.atleast_1d(shape))) else 1
    out = np.empty(n, dtype=np.float32)
    for start in range(0, n, _CHUNK):
        count = min(_CHUNK, n - start)
        out[start:start + count] = fn(start, count)
    return out.reshape(shape)


def uniform(shape, seed, lo, hi):
    lo, hi = float(lo), float(hi)
    return _fill(shape, lambda s, c: (lo + (hi - lo) * ((_draw(seed, s, c) >> np.uint64(40)).astype(np.float64)
                                                        * (1.0 / 16777216.0))).astype(np.float32))


def normal(shape, seed, mean=0.0, sigma=1.0):
    mean, sigma = float(mean), float(sigma)
    seed2 = int(np.uint64(seed) ^ _OTHER)

    def part(s, c):
        u1 = ((_draw(seed, s, c) >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)
        u2 = ((_draw(seed2, s, c) >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586476925 * u2)
        return (mean + sigma * z).astype(np.float32)

    return _fill(shape, part)


def ints(shape, seed, rng):
    return _fill(shape, lambda s, c: (_draw(seed, s, c) % np.uint64(rng)).astype(np.float32))
