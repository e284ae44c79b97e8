"""The random stream of the random-weights mode: element i of a tensor is a function of
(key, i) alone, where the key comes from (seed, tensor name).  This is the host side in
numpy; csrc/random_fill.hip is the same arithmetic on the device, bit for bit: a folder
written on the CPU, the tensors an engine makes on the GPU and whatever else starts from
the same seed hold the same numbers.

Normal numbers are Box-Muller in float64 over one 64-bit hash per pair of elements.  So
that both sides round alike, no math library is used: logarithm, sine and cosine are
fixed sequences of float64 additions, multiplications and divisions and one square root,
all of which IEEE 754 rounds correctly everywhere.  Do not reorder an expression here
without the same change in the kernel.
"""
from __future__ import annotations

import hashlib

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_CHUNK = 1 << 14          # pairs at a time: the temporaries stay in the cache


def tensor_key(seed: int, name: str) -> int:
    """64 bits from (seed, tensor name)."""
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little")


def _mix(key: int, counters: np.ndarray) -> np.ndarray:
    """splitmix64 of key + (counter + 1) * golden, as the sampler's stream."""
    with np.errstate(over="ignore"):
        z = np.uint64(key) + (counters + np.uint64(1)) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def _minus_two_log(n: np.ndarray) -> np.ndarray:
    """-2 ln(n / 2^33) for odd 0 < n < 2^33 (uint64)."""
    m, e = np.frexp(n.astype(np.float64))            # n = m 2^e, m in [0.5, 1)
    low = m < 0.7071067811865476
    m = np.where(low, m * 2.0, m)
    e = np.where(low, e - 1, e)
    t = (m - 1.0) / (m + 1.0)
    t2 = t * t
    s = np.full_like(t, 1.0 / 23.0)
    for k in range(21, 0, -2):
        s = s * t2 + 1.0 / k
    log_m = 2.0 * (t * s)
    return 2.0 * ((33 - e).astype(np.float64) * 0.6931471805599453 - log_m)


def _cos_sin_turn(k: np.ndarray):
    """cos and sin of 2 pi k / 2^32 for k in uint64 below 2^32."""
    octant = (k >> np.uint64(29)).astype(np.int64)
    r = (k & np.uint64(0x1FFFFFFF)).astype(np.int64)
    r = np.where(octant & 1, 0x20000000 - r, r)
    x = r.astype(np.float64) * (0.7853981633974483 / 536870912.0)
    x2 = x * x
    c = np.ones_like(x)
    s = np.ones_like(x)
    for j in range(9, 0, -1):
        c = 1.0 - x2 * c * (1.0 / ((2 * j - 1) * (2 * j)))
        s = 1.0 - x2 * s * (1.0 / ((2 * j) * (2 * j + 1)))
    s = s * x
    swap = ((octant + 1) >> 1) & 1                   # octants 1, 2, 5, 6: cos from the sine series
    co = np.where(swap, s, c) * np.where((octant + 2) & 4, -1.0, 1.0)      # octants 2..5
    si = np.where(swap, c, s) * np.where(octant & 4, -1.0, 1.0)            # octants 4..7
    return co, si


def _normal_block(out: np.ndarray, key: int, count: int, std: float, plus_one: bool, first: int, last: int):
    """Pairs first..last-1 of the stream into out."""
    for lo in range(first, last, _CHUNK):
        n = min(_CHUNK, last - lo)
        h = _mix(key, np.arange(lo, lo + n, dtype=np.uint64))
        radius = np.sqrt(_minus_two_log(np.uint64(2) * (h >> np.uint64(32)) + np.uint64(1)))
        c, s = _cos_sin_turn(h & np.uint64(0xFFFFFFFF))
        z = np.empty(2 * n, dtype=np.float64)
        z[0::2] = std * (radius * c)
        z[1::2] = std * (radius * s)
        if plus_one:
            z = 1.0 + z
        stop = min(count, 2 * (lo + n))
        out[2 * lo:stop] = z[:stop - 2 * lo].astype(np.float32)


def normal(key: int, count: int, std: float, plus_one: bool = False) -> np.ndarray:
    """count float32 numbers: std * z (1 + std * z with plus_one), z standard normal,
    computed in float64 and rounded once.  (About 90 ns a number: a tensor of a large
    model is better made on the device, which gives the same bits.)"""
    out = np.empty(count, dtype=np.float32)
    _normal_block(out, key, count, float(std), plus_one, 0, (count + 1) // 2)
    return out


def integers(key: int, count: int, bound: int) -> np.ndarray:
    """count int32 numbers in [0, bound)."""
    if not 1 <= bound <= 0x7FFFFFFF:
        raise ValueError(f"bound must be in 1..2^31-1, got {bound}")
    out = np.empty(count, dtype=np.int32)
    for first in range(0, count, _CHUNK):
        n = min(_CHUNK, count - first)
        h = _mix(key, np.arange(first, first + n, dtype=np.uint64))
        out[first:first + n] = ((h >> np.uint64(11)) % np.uint64(bound)).astype(np.int32)
    return out
