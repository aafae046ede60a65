"""Repo-owned deterministic counter-based generator for synthetic inputs.

Every draw is a pure function of (seed, stream, counter): the 64-bit word
``splitmix64_mix(seed * GOLDEN + stream * STREAM_MULT + counter)`` (the finaliser of
Steele/Lea/Flood's SplitMix64).  Uniforms take the top 24 bits (exact in fp32), normals are
Box-Muller on two such words evaluated in float64 and rounded once to fp32.  Nothing depends
on numpy's own distributions, so the streams are stable across numpy versions and can be
regenerated on a device with integer arithmetic only.

The reference's own seeded initialisation (one ``std::mt19937`` consumed in merged-group
order, src/genn/genn/code_generator/standardLibrary.cc:132-140) cannot be reproduced by an
independent implementation, so every backend under test *loads* arrays produced here.
"""
import numpy as np

GOLDEN = np.uint64(0x9E3779B97F4A7C15)
STREAM_MULT = np.uint64(0xD1B54A32D192ED03)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def words_at(seed, stream, ctr):
    """64-bit words of stream ``stream`` at the counters in ``ctr`` (any uint64 array)."""
    with np.errstate(over="ignore"):
        base = np.uint64(seed) * GOLDEN + np.uint64(stream) * STREAM_MULT
        return _mix(_mix(base + np.asarray(ctr, dtype=np.uint64)) + GOLDEN)


def words(seed, stream, start, count):
    """``count`` 64-bit words of stream ``stream`` beginning at counter ``start``."""
    return words_at(seed, stream, np.arange(start, start + count, dtype=np.uint64))


def normal_at(seed, stream, ctr):
    """Standard normals at arbitrary counters; normal(seed, stream, a, n) == normal_at(seed, stream, arange(a, a+n))."""
    ctr = np.asarray(ctr, dtype=np.uint64)
    u1 = ((words_at(seed, stream, ctr + np.uint64(0)) >> np.uint64(40)).astype(np.float64) + 1.0) * (1.0 / 16777216.0)
    u2 = (words_at(seed, stream + 0x40000000, ctr) >> np.uint64(40)).astype(np.float64) * (1.0 / 16777216.0)
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def uniform(seed, stream, start, count):
    """fp64 uniforms in [0,1) with 24 significant bits (so the fp32 cast is exact)."""
    return (words(seed, stream, start, count) >> np.uint64(40)).astype(np.float64) * (1.0 / 16777216.0)


def uniform_open(seed, stream, start, count):
    """Uniforms in (0,1]: safe as the argument of a logarithm."""
    return ((words(seed, stream, start, count) >> np.uint64(40)).astype(np.float64) + 1.0) * (1.0 / 16777216.0)


def randint(seed, stream, start, count, n):
    """Integers in [0,n) by multiply-shift of the top 32 bits (n < 2**32)."""
    hi = words(seed, stream, start, count) >> np.uint64(32)
    return ((hi * np.uint64(n)) >> np.uint64(32)).astype(np.uint32)


def normal(seed, stream, start, count):
    """Standard normals (Box-Muller, cosine branch) as fp64."""
    return normal_at(seed, stream, np.arange(start, start + count, dtype=np.uint64))
