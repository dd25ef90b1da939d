"""Seeded synthetic inputs for the matmul configurations of BASELINE.json.

Counter-based: element i of a stream is a pure function of (seed, i) through
splitmix64, so any sub-block can be regenerated on its own and the values do not
depend on the numpy version. Uniforms are (z >> 11) * 2^-53 in [0, 1); normals
are Box-Muller on counters (2i, 2i+1).
"""
import numpy as np

_G = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed, idx):
    """splitmix64 output number idx (array of uint64 counters) of the stream `seed`."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (idx.astype(np.uint64) + np.uint64(1)) * _G
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _chunks(n, chunk=1 << 22):
    for s in range(0, n, chunk):
        yield s, min(n, s + chunk)


def uniform01(seed, n, offset=0):
    out = np.empty(n, dtype=np.float64)
    for s, e in _chunks(n):
        idx = np.arange(s + offset, e + offset, dtype=np.uint64)
        out[s:e] = (splitmix64(seed, idx) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    return out


def uniform(seed, shape, lo=-1.0, hi=1.0):
    n = int(np.prod(shape))
    return (lo + (hi - lo) * uniform01(seed, n)).reshape(shape)


def normal(seed, shape, sigma=1.0):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float64)
    for s, e in _chunks(n):
        u = uniform01(seed, 2 * (e - s), offset=2 * s)
        u1 = 1.0 - u[0::2]                     # (0, 1]
        u2 = u[1::2]
        out[s:e] = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (sigma * out).reshape(shape)


def wide_range(seed, shape, emin=-30, emax=30):
    """a = u * 2^e, u ~ U[-1,1], e uniform integer in [emin, emax] (configuration 3)."""
    n = int(np.prod(shape))
    u = 2.0 * uniform01(seed, n) - 1.0
    idx = np.arange(n, dtype=np.uint64)
    e = (splitmix64(np.uint64(seed) ^ np.uint64(0xA5A5A5A5A5A5A5A5), idx) % np.uint64(emax - emin + 1))
    e = e.astype(np.int64) + emin
    return np.ldexp(u, e).reshape(shape)


def xavier_uniform(seed, fan_in, fan_out):
    """U(-sqrt(6/(fan_in+fan_out)), +) weights, shape [fan_in, fan_out] (configuration 5)."""
    lim = np.sqrt(6.0 / (fan_in + fan_out))
    return uniform(seed, (fan_in, fan_out), -lim, lim)
