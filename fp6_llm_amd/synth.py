"""Deterministic synthetic inputs for the benchmark configurations.

A counter-based generator (splitmix64 on the element index) is used instead of numpy's or torch's stateful generators so
that any machine regenerates bit-identical integer data from (seed, shape) alone.
"""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np

from . import quant

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed, n, offset=0):
    """n 64-bit values: element i = mix(seed + (offset+i+1) * golden)."""
    with np.errstate(over="ignore"):
        z = (np.uint64(seed) + (np.arange(offset + 1, offset + n + 1, dtype=np.uint64)) * np.uint64(0x9E3779B97F4A7C15)) & _MASK
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
        return z ^ (z >> np.uint64(31))


def uniform01(seed, n, offset=0):
    return (splitmix64(seed, n, offset) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def normal(seed, shape, sigma=1.0):
    n = int(np.prod(shape))
    m = (n + 1) // 2
    u1 = 1.0 - uniform01(seed, m)            # (0, 1]
    u2 = uniform01(seed ^ 0x5DEECE66D, m)
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:n]
    return (z * sigma).reshape(shape)


def uniform_codes(seed, OC, IC, E=3, M=2):
    """Uniform over all 2^x codes."""
    x = 1 + E + M
    return (splitmix64(seed, OC * IC) >> np.uint64(64 - x)).astype(np.uint8).reshape(OC, IC)


def uniform_scales(seed, OC, lo=1e-3, hi=1e-2):
    return (lo + (hi - lo) * uniform01(seed ^ 0xABCDEF, OC)).astype(np.float16)


def activations(seed, BS, IC, sigma=1.0):
    return normal(seed ^ 0x13579B, (BS, IC), sigma).astype(np.float16)


def uniform_problem(seed, OC, IC, BS, E=3, M=2):
    """Configs 1-2: uniform random codes, scales U[1e-3, 1e-2], activations N(0,1). Returns (raw int32, scales, x)."""
    codes = uniform_codes(seed, OC, IC, E, M)
    return quant.pack_raw(codes, E, M), uniform_scales(seed, OC), activations(seed, BS, IC)


def gaussian_problem(seed, OC, IC, BS, E=3, M=2, act_sigma=1.0, chunk_rows=256):
    """Configs 3-5: codes are the round-to-nearest quantisation of N(0,1) weights with per-row absmax fp16 scales."""
    def chunk(r0):
        rows = min(chunk_rows, OC - r0)
        w = normal(seed + 7919 * (r0 // chunk_rows + 1), (rows, IC))
        c, s = quant.quantize_rowwise(w, E, M)
        return quant.pack_raw(c, E, M), s

    # numpy releases the GIL inside its loops, so plain threads spread the chunks over the host cores
    with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 1)) as pool:
        parts = list(pool.map(chunk, range(0, OC, chunk_rows)))
    return (np.concatenate([p[0] for p in parts]), np.concatenate([p[1] for p in parts]),
            activations(seed, BS, IC, act_sigma))
