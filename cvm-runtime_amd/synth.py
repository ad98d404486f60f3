"""Reproducible synthetic tensors: splitmix64 streams keyed by (config, tensor name).

The same integers come out on every machine (no library RNG involved), so the
CPU oracle, the compiled reference and the GPU run can all regenerate identical
inputs from a name instead of shipping data files.
"""
import numpy as np

_MASK = (1 << 64) - 1
GLOBAL_SEED = 0x5EED


def fnv1a64(text):
    h = 0xCBF29CE484222325
    for ch in text.encode():
        h ^= ch
        h = (h * 0x100000001B3) & _MASK
    return h


def splitmix64(seed, n):
    """First n outputs of splitmix64 started at `seed` (uint64 array)."""
    with np.errstate(over="ignore"):
        idx = np.arange(1, n + 1, dtype=np.uint64)
        z = np.uint64(seed & _MASK) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def tensor(config_id, name, shape, lo, hi, seed=GLOBAL_SEED):
    """int32 tensor with values uniform in [lo, hi] from the stream of (config_id, name)."""
    n = int(np.prod(shape)) if len(shape) else 1
    stream = fnv1a64("%s:%s" % (config_id, name)) ^ seed
    u = splitmix64(stream, n)
    span = np.uint64(hi - lo + 1)
    return (np.int64(lo) + (u % span).astype(np.int64)).astype(np.int32).reshape(shape)
