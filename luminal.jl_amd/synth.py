"""Seeded synthetic inputs for the benchmark configurations: SplitMix64 -> Box-Muller normals and SplitMix64
uniform integers, specified here so that every host (this module, the test oracle's C generator, a Julia caller)
produces the same arrays from the same seed.

    element i of a stream with `seed`:  z = seed + (i + 1) * 0x9E3779B97F4A7C15   (mod 2^64)
                                        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9
                                        z = (z ^ (z >> 27)) * 0x94D049BB133111EB;  z ^= z >> 31
    normals: pair p takes a = stream[2p], b = stream[2p+1]; u1 = ((a >> 11) + 1) / 2^53 in (0, 1],
             u2 = (b >> 11) / 2^53 in [0, 1); r = sqrt(-2 ln u1); out[2p] = r cos(2 pi u2), out[2p+1] = r sin(2 pi u2),
             computed in float64, rounded to float32, then multiplied by `mul` in float32.
    integers in [lo, hi]: lo + stream[i] mod (hi - lo + 1).
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _splitmix64_at(seed, index):
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (index + np.uint64(1)) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def normal(shape, seed, mul=1.0, chunk_pairs=1 << 22):
    """float32 array of `shape`, N(0, 1) * mul."""
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(n + (n & 1), dtype=np.float32)
    n_pairs = (n + 1) // 2
    for p0 in range(0, n_pairs, chunk_pairs):  # chunked: the float64 temporaries of a 33M-element pool stay small
        pairs = np.arange(p0, min(p0 + chunk_pairs, n_pairs), dtype=np.uint64)
        a = _splitmix64_at(seed, np.uint64(2) * pairs)
        b = _splitmix64_at(seed, np.uint64(2) * pairs + np.uint64(1))
        u1 = ((a >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
        u2 = (b >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        r = np.sqrt(-2.0 * np.log(u1))
        ang = 6.283185307179586476925286766559 * u2
        lo, hi = 2 * p0, 2 * (p0 + len(pairs))
        out[lo:hi:2] = (r * np.cos(ang)).astype(np.float32) * np.float32(mul)
        out[lo + 1:hi:2] = (r * np.sin(ang)).astype(np.float32) * np.float32(mul)
    return out[:n].reshape(shape)


def uniform_int(n, seed, lo, hi):
    """int32 array of n values in [lo, hi]."""
    span = np.uint64(int(hi) - int(lo) + 1)
    z = _splitmix64_at(seed, np.arange(n, dtype=np.uint64))
    return (int(lo) + (z % span).astype(np.int64)).astype(np.int32)
