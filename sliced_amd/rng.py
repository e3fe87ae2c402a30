"""Seeded, counter-based host RNG for reproducible inputs.

The reference draws its weights from an unseeded generator (src/rawops/cpu/rand.rs:7-12:
``fastrand::Rng::new()``), so no run of it can be reproduced.  This module defines the
stream used instead; the same definition exists as a device kernel
(``slhip_rand_uniform``), bit for bit.

    state = (seed XOR (tag << 40)) + i                       (mod 2^64)
    z     = splitmix64(state)
    u     = (z >> 40) * 2^-24                                 in [0, 1), exact in f32
    U(a, b) = fl32(a + fl32((b - a) * u))                     two separately rounded f32 ops

N(0, sigma^2) uses Box-Muller on the pair (u[2j], u[2j+1]) evaluated in f64 and rounded to f32.
"""
import numpy as np

DEFAULT_SEED = 0x51CED
_M = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(state):
    z = state + np.uint64(0x9E3779B97F4A7C15)
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def raw_u24(n, tag, seed=DEFAULT_SEED, start=0):
    """24-bit integers z >> 40 for counters start .. start+n-1 (uint32 array)."""
    out = np.empty(n, np.uint32)
    base = np.uint64((int(seed) ^ (int(tag) << 40)) & 0xFFFFFFFFFFFFFFFF)
    CH = 1 << 22
    with np.errstate(over="ignore"):
        for s in range(0, n, CH):
            e = min(n, s + CH)
            i = np.arange(start + s, start + e, dtype=np.uint64)
            out[s:e] = (_splitmix64(base + i) >> np.uint64(40)).astype(np.uint32)
    return out


def unit(n, tag, seed=DEFAULT_SEED):
    """u in [0,1) as float32 (exact)."""
    return raw_u24(n, tag, seed).astype(np.float32) * np.float32(2.0 ** -24)


def uniform(n, lo, hi, tag, seed=DEFAULT_SEED):
    u = unit(n, tag, seed)
    lo32, hi32 = np.float32(lo), np.float32(hi)
    return (lo32 + (hi32 - lo32) * u).astype(np.float32)


def normal(n, sigma, tag, seed=DEFAULT_SEED):
    m = (n + 1) // 2
    u = raw_u24(2 * m, tag, seed).astype(np.float64) * 2.0 ** -24
    u1 = 1.0 - u[0::2]            # (0, 1], keeps log finite
    u2 = u[1::2]
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.empty(2 * m, np.float64)
    z[0::2] = r * np.cos(2.0 * np.pi * u2)
    z[1::2] = r * np.sin(2.0 * np.pi * u2)
    return (z[:n] * float(sigma)).astype(np.float32)


def integers(n, k, tag, seed=DEFAULT_SEED):
    """Uniform integers in [0, k) (k << 2^24), as int64."""
    return (raw_u24(n, tag, seed).astype(np.int64) * int(k)) >> 24


def inject_row_max_ties(x, rows, cols, frac=0.01):
    """Copy each row's maximum into floor(frac*cols) other positions of that row (in place).

    Positions are spread deterministically (stride) so that the first maximal index of a row
    is usually not the original argmax: this is what separates a first-tie rule from an
    all-ties rule.
    """
    x = x.reshape(rows, cols)
    k = int(frac * cols)
    if k == 0:
        return x.reshape(-1)
    m = x.max(axis=1)
    stride = max(1, cols // k)
    for j in range(k):
        pos = (np.arange(rows) * 7 + j * stride + 3) % cols
        x[np.arange(rows), pos] = m
    return x.reshape(-1)


def inject_col_max_ties(x, rows, cols, frac=0.01):
    """Same along columns: copy each column's maximum into floor(frac*rows) other rows."""
    x = x.reshape(rows, cols)
    k = int(frac * rows)
    if k == 0:
        return x.reshape(-1)
    m = x.max(axis=0)
    stride = max(1, rows // k)
    for j in range(k):
        pos = (np.arange(cols) * 5 + j * stride + 1) % rows
        x[pos, np.arange(cols)] = m
    return x.reshape(-1)
