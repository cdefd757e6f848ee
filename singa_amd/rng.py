"""The seeded generator of the benchmark's synthetic inputs: counter-based, so that the bytes depend
on no library's random stream.  The k-th output of splitmix64 seeded with ``seed`` is
``mix(seed + (k + 1) * golden)``; a uniform double is ``(out >> 11) * 2**-53``; a normal deviate is
Box-Muller in double precision on outputs ``2i`` and ``2i + 1``, rounded to float32 once; integers
are ``out % hi``.  The same arithmetic exists in C (the test-suite's CPU checker) and on the device
(``sgh_uniform_f32`` / ``sgh_gaussian_f32``); the tests hold the three to each other.
"""
import numpy as np

GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1, _M2 = np.uint64(0xBF58476D1CE4E5B9), np.uint64(0x94D049BB133111EB)
_TWO_PI = 6.283185307179586476925286766559


def raw(seed, k):
    """splitmix64 outputs number ``k`` (an integer or an array of them) of the stream ``seed``."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + (np.asarray(k, dtype=np.uint64) + np.uint64(1)) * GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _unit(r):
    return (r >> np.uint64(11)).astype(np.float64) * 2.0 ** -53


def _counters(n, offset, step=1, chunk=1 << 22):
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        yield lo, hi, np.arange(lo, hi, dtype=np.uint64) * np.uint64(step) + np.uint64(offset)


def uniform(seed, shape, low=0.0, high=1.0, offset=0):
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(n, np.float32)
    for lo, hi, k in _counters(n, offset):
        out[lo:hi] = (low + _unit(raw(seed, k)) * (high - low)).astype(np.float32)
    return out.reshape(shape)


def normal(seed, shape, mean=0.0, std=1.0, offset=0):
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(n, np.float32)
    for lo, hi, k in _counters(n, offset, step=2):
        u1, u2 = _unit(raw(seed, k)), _unit(raw(seed, k + np.uint64(1)))
        out[lo:hi] = (mean + std * (np.sqrt(-2.0 * np.log(1.0 - u1)) * np.cos(_TWO_PI * u2))).astype(np.float32)
    return out.reshape(shape)


def integers(seed, shape, hi, offset=0):
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(n, np.int32)
    for lo, hi_, k in _counters(n, offset):
        out[lo:hi_] = (raw(seed, k) % np.uint64(hi)).astype(np.int32)
    return out.reshape(shape)


class Stream(object):
    """Tensors number 0, 1, 2, ... of a configuration: each draw takes the next tensor index and
    uses the seed ``base + index`` (a drop-in for the two ``numpy.random.Generator`` methods the
    builders use)."""

    def __init__(self, base):
        self.base, self.index = int(base), 0

    def _next(self):
        s = self.base + self.index
        self.index += 1
        return s

    def standard_normal(self, shape):
        return normal(self._next(), tuple(shape) if np.ndim(shape) else (int(shape),))

    def integers(self, low, high, size):
        assert low == 0
        return integers(self._next(), (int(size),), high)
