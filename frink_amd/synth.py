"""Seeded synthetic inputs for the benchmark configurations.

The reference fixes no generator for these shapes (its own fixtures use xorshift32 streams), so
this one is defined here and used by the tests and the benchmark alike:

    z_i   = splitmix64 output for counter i (state = seed + (i+1) * 0x9E3779B97F4A7C15)
    u1    = ((z_i >> 40) + 1) / 2^24          in (0, 1]
    u2    = ((z_i >> 16) & 0xFFFFFF) / 2^24   in [0, 1)
    n_i   = sqrt(-2 ln u1) * cos(2 pi u2)     in float64, then * sigma, cast to float32

Element i depends only on (seed, i), so any slice can be generated on its own.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def splitmix64(seed, start, count):
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        z = np.uint64(seed) + i * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def normal(seed, count, sigma=1.0, start=0):
    """`count` float32 values N(0, sigma) for counters start .. start+count.  (Large counts are generated in
    chunks by a few threads: element i depends on (seed, i) only, so the result does not depend on how.)"""
    out = np.empty(count, np.float32)
    step = 1 << 20

    def chunk(lo):
        n = min(step, count - lo)
        z = splitmix64(seed, start + lo, n)
        u1 = ((z >> np.uint64(40)).astype(np.float64) + 1.0) / 16777216.0
        u2 = ((z >> np.uint64(16)) & np.uint64(0xFFFFFF)).astype(np.float64) / 16777216.0
        out[lo:lo + n] = (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2) * sigma).astype(np.float32)

    starts = range(0, count, step)
    if count <= 4 * step:
        for lo in starts:
            chunk(lo)
    else:
        import os
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 1)) as pool:
            list(pool.map(chunk, starts))
    return out


def weights(seed, rows, cols, sigma=0.02):
    return normal(seed, rows * cols, sigma).reshape(rows, cols)


def activations(seed, batch, cols, outlier_frac=0.0, outlier_mag=20.0):
    """N(0,1) rows; with outlier_frac > 0 that share of the entries (chosen by a second stream
    from the same seed) is replaced by +-outlier_mag."""
    x = normal(seed, batch * cols, 1.0)
    if outlier_frac > 0:
        z = splitmix64(seed ^ 0x5DEECE66D, 0, batch * cols)
        pick = (z >> np.uint64(40)).astype(np.float64) / 16777216.0 < outlier_frac
        sign = np.where((z & np.uint64(1)).astype(bool), 1.0, -1.0).astype(np.float32)
        x = np.where(pick, sign * np.float32(outlier_mag), x).astype(np.float32)
    return x.reshape(batch, cols)
