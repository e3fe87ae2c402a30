"""The device generator's values recomputed on the host at arbitrary element indices, so that tests on
large tensors need no host copy of them: a tensor filled by slhip_rand_uniform(seed, tag, lo, hi) holds
host_values(indices, tag, lo, hi, seed) at those indices, bit for bit."""
import numpy as np

from sliced_amd import rng


def host_values(idx, tag, lo=-1.0, hi=1.0, seed=rng.DEFAULT_SEED):
    idx = np.asarray(idx, dtype=np.uint64)
    base = np.uint64((int(seed) ^ (int(tag) << 40)) & 0xFFFFFFFFFFFFFFFF)
    with np.errstate(over="ignore"):
        u = (rng._splitmix64(base + idx) >> np.uint64(40)).astype(np.uint32).astype(np.float32) * np.float32(2.0 ** -24)
    return (np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u).astype(np.float32)


def host_range(start, n, tag, lo=-1.0, hi=1.0, seed=rng.DEFAULT_SEED):
    return host_values(np.arange(start, start + n, dtype=np.uint64), tag, lo, hi, seed)
