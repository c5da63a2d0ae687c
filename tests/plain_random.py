"""The random weights of a model written out again in numpy, from the rule alone: element e of
the i-th tensor of a model with seed s is

    w  = hash(s, i, e)                                   a 32-bit word
    z  = q[w >> 16] + (q[(w >> 16) + 1] - q[w >> 16]) * ((w & 0xffff) / 65536)
    x  = mean + std * z

with q the standard normal quantile at j / 65536 (float32; the two ends at 2^-18 from 0 and 1)
and every operation a float32 operation rounded on its own.  The quantiles come from the
standard library's inverse CDF, not from the routine the engine uses.  It shares no code with
the engine."""
import statistics

import numpy as np

_Q = None


def quantiles():
    global _Q
    if _Q is None:
        inv = statistics.NormalDist().inv_cdf
        p = [j / 65536 for j in range(65537)]
        p[0], p[-1] = 2.0 ** -18, 1.0 - 2.0 ** -18
        _Q = np.array([inv(x) for x in p], dtype=np.float64).astype(np.float32)
    return _Q


def _mix(h):
    h = h.copy()
    h ^= h >> np.uint32(16)
    h *= np.uint32(0x85EBCA6B)
    h ^= h >> np.uint32(13)
    h *= np.uint32(0xC2B2AE35)
    h ^= h >> np.uint32(16)
    return h


def words(seed, index, n):
    """The 32-bit words of the first ``n`` elements of tensor ``index``."""
    seed &= (1 << 64) - 1
    lo, hi = np.uint32(seed & 0xFFFFFFFF), np.uint32(seed >> 32)
    with np.errstate(over="ignore"):
        k1 = _mix(_mix(np.array([index], dtype=np.uint32) ^ np.uint32(0x9E3779B9)) ^ lo)
        k2 = _mix(k1 + hi * np.uint32(0x85EBCA6B) + np.uint32(0x27D4EB2F))
        e = np.arange(n, dtype=np.uint64)
        h = _mix((e & np.uint64(0xFFFFFFFF)).astype(np.uint32) ^ k1)
        return _mix(h + (e >> np.uint64(32)).astype(np.uint32) * np.uint32(0x9E3779B1) + k2)


def normal(shape, seed, index, std=0.02, mean=0.0):
    """float32 array of ``shape``."""
    n = int(np.prod(shape))
    w = words(seed, index, n)
    q = quantiles()
    i = (w >> np.uint32(16)).astype(np.int64)
    a, b = q[i], q[i + 1]
    frac = (w & np.uint32(0xFFFF)).astype(np.float32) * np.float32(1.0 / 65536.0)
    z = a + (b - a) * frac                      # numpy rounds every float32 operation on its own
    return (np.float32(mean) + np.float32(std) * z).reshape(shape)


def to_bfloat16_bits(x):
    """float32 -> the 16 bits of its bfloat16, round to nearest, ties to even."""
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    return ((u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))) >> np.uint64(16)).astype(np.uint16)


def model_weights(names_shapes_inits, seed):
    """name -> float64 array holding the bfloat16 values of a random model whose tensors are
    declared in this order as (name, shape, "normal" | "ones_normal")."""
    out = {}
    for index, (name, shape, init) in enumerate(names_shapes_inits):
        x = normal(shape, seed, index, 0.02, 1.0 if init == "ones_normal" else 0.0)
        bits = to_bfloat16_bits(x).astype(np.uint32) << np.uint32(16)
        out[name] = bits.view(np.float32).astype(np.float64).reshape(shape)
    return out
