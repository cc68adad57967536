"""Deterministic synthetic inputs shared by tests and the benchmark.

A counter-based generator (SplitMix64 -> Box-Muller in f64 -> cast to f32) so
that the CPU oracle and the GPU see the same bits on every machine and numpy
version, unlike a library RNG whose stream may change between releases.
"""
import numpy as np

SEED_BASE = 0x4D474E00  # + config index

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _splitmix64(seed, idx):
    """SplitMix64 output for counters idx (uint64 array), stateless."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (idx + np.uint64(1)) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def normal(seed, count, sigma=1.0, chunk=1 << 22):
    """count draws of N(0, sigma^2) as float32; element i depends on (seed, i) only."""
    out = np.empty(count, dtype=np.float32)
    sig = np.float64(sigma)
    for start in range(0, count, chunk):
        stop = min(count, start + chunk)
        p0, p1 = start // 2, (stop + 1) // 2  # Box-Muller pairs covering [start, stop)
        pair = np.arange(p0, p1, dtype=np.uint64)
        z1 = _splitmix64(seed, pair * np.uint64(2))
        z2 = _splitmix64(seed, pair * np.uint64(2) + np.uint64(1))
        u1 = ((z1 >> np.uint64(11)).astype(np.float64) + 1.0) * 2.0**-53  # (0, 1]
        u2 = (z2 >> np.uint64(11)).astype(np.float64) * 2.0**-53  # [0, 1)
        r = np.sqrt(-2.0 * np.log(u1)) * sig
        both = np.empty((p1 - p0) * 2, dtype=np.float64)
        both[0::2] = r * np.cos(2.0 * np.pi * u2)
        both[1::2] = r * np.sin(2.0 * np.pi * u2)
        out[start:stop] = both[start - 2 * p0 : stop - 2 * p0].astype(np.float32)
    return out


def weights(config_index, k, n, which=0, sigma=0.02):
    """W ~ N(0, sigma^2), f32 [k, n] row-major, for BASELINE config `config_index`."""
    return normal(SEED_BASE + config_index + (which << 20), k * n, sigma).reshape(k, n)


def activations(config_index, m, k, which=0):
    """x ~ N(0, 1), f32 [m, k]."""
    return normal(SEED_BASE + config_index + 0x80000 + (which << 20), m * k, 1.0).reshape(m, k)
