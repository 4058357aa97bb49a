"""FP16/FP32 -> FPx quantizer with per-row absmax scales, and raw-tensor packing.

The reference ships only a truncating FP16->FP6 cast that is not wired into any API (fp6_llm/csrc/utils/weight_quant.h:9-105,
"To be used in the future"); this one rounds to nearest, ties to even, clamps at the format maximum and covers every format of the
engine (e3m2, e2m2, e2m3, e2m1).
It is the step before the linear-layer path: it produces the raw int32 tensor that weight_prepacking*_cpu consumes.
"""
import numpy as np


FORMATS = ((3, 2), (2, 2), (2, 3), (2, 1))   # FP6_e3m2, FP5_e2m2, FP6_e2m3, FP4_e2m1


def _check(E, M):
    if (E, M) not in FORMATS:
        raise ValueError("unsupported format e%dm%d" % (E, M))
    return 1 + E + M


def magnitudes(E, M):
    """Ascending non-negative values of the format; index == magnitude bits of the code (exponent all-ones is ordinary)."""
    _check(E, M)
    bias = (1 << (E - 1)) - 1
    vals = []
    for e in range(1 << E):
        for m in range(1 << M):
            vals.append(2.0 ** (1 - bias) * m / (1 << M) if e == 0 else 2.0 ** (e - bias) * (1 + m / (1 << M)))
    return np.array(vals, dtype=np.float64)


def max_value(E, M):
    return float(magnitudes(E, M)[-1])


def quantize_codes(values, E=3, M=2):
    """values (any float array, already divided by the scale) -> uint8 codes, round-to-nearest, ties to the even code.
    +-Inf saturates to the largest magnitude, NaN becomes +0 (the device quantizer does the same)."""
    x = _check(E, M)
    v = np.asarray(values, dtype=np.float64)
    v = np.where(np.isnan(v), 0.0, v)
    mags = magnitudes(E, M)
    a = np.minimum(np.abs(v), mags[-1])
    hi = np.clip(np.searchsorted(mags, a, side="left"), 0, len(mags) - 1)   # first magnitude >= a
    lo = np.maximum(hi - 1, 0)
    d_hi, d_lo = mags[hi] - a, a - mags[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    idx = np.where(pick_lo, lo, hi).astype(np.uint8)
    sign = np.signbit(v).astype(np.uint8)
    return (sign << (x - 1)) | idx


def _finite_abs(w):
    return np.where(np.isfinite(w), np.abs(w), 0.0)


def quantize_rowwise(weight, E=3, M=2):
    """weight [OC, IC] float -> (codes uint8 [OC, IC], scales float16 [OC]) with scale = absmax(row) / max_value,
    rounded to fp16 first so that codes are chosen against the scale that will actually be applied."""
    w = np.asarray(weight, dtype=np.float64)
    absmax = _finite_abs(w).max(axis=1)          # NaN and +-Inf do not set the scale
    scale = (absmax / max_value(E, M)).astype(np.float16)
    scale = np.where(scale == 0, np.float16(1.0), scale).astype(np.float16)
    return quantize_codes(w / scale.astype(np.float64)[:, None], E, M), scale


GROUP = 128   # columns per group exponent: a lane's share of a half K block in the native layout


def quantize_groupwise(weight, E=3, M=2):
    """weight [OC, IC] float -> (codes uint8 [OC, IC], scales float16 [OC], exps uint8 [OC, ceil(IC/128)]).
    Two-level scaling: the row scale of quantize_rowwise, and per group of 128 columns the smallest power of two 2^(b-127),
    112 <= b <= 127, that still holds the group's largest magnitude: weight ~ value(code) * 2^(b-127) * scale[row].
    A group whose magnitudes are small next to the row maximum keeps up to 15 more bits of them than the row scale would."""
    w = np.asarray(weight, dtype=np.float64)
    OC, IC = w.shape
    top = max_value(E, M)
    scale = (_finite_abs(w).max(axis=1) / top).astype(np.float16)
    scale = np.where(scale == 0, np.float16(1.0), scale).astype(np.float16)
    groups = (IC + GROUP - 1) // GROUP
    pad = np.zeros((OC, groups * GROUP))
    pad[:, :IC] = _finite_abs(w)
    gmax = pad.reshape(OC, groups, GROUP).max(axis=2) / scale.astype(np.float64)[:, None]     # in units of the row scale
    with np.errstate(divide="ignore"):
        k = np.ceil(np.log2(gmax / top))                       # smallest k with gmax <= top * 2^k (checked below: log2 rounds)
    k = np.where(gmax > 0, k, -15.0)
    k = np.where(gmax > top * np.exp2(k), k + 1, k)
    k = np.where((k > -15) & (gmax <= top * np.exp2(k - 1)), k - 1, k)
    k = np.clip(k, -15, 0).astype(np.int64)
    factor = np.repeat(np.exp2(k.astype(np.float64)), GROUP, axis=1)[:, :IC] * scale.astype(np.float64)[:, None]
    return quantize_codes(w / factor, E, M), scale, (k + 127).astype(np.uint8)


def dequantize_grouped(codes, scales, exps, E=3, M=2):
    """float64 value(code) * 2^(b-127) * scale, for checks."""
    c = np.asarray(codes)
    f = np.repeat(np.exp2(np.asarray(exps, dtype=np.float64) - 127.0), GROUP, axis=1)[:, :c.shape[1]]
    return dequantize_codes(c, scales, E, M) * f


def pack_raw(codes, E=3, M=2):
    """codes uint8 [OC, IC] -> int32 [OC, IC/32*x]: each row an MSB-first bitstream carried in little-endian int32 words,
    the raw weight format of the reference (fp6_llm/csrc/utils/common.h:4-19; worked example
    tests/python/kernel_test_fpx.py:124-131)."""
    x = _check(E, M)
    c = np.asarray(codes, dtype=np.uint8)
    if c.ndim != 2 or c.shape[1] % 32:
        raise ValueError("codes must be [OC, IC] with IC % 32 == 0")
    if (c >> x).any():
        raise ValueError("a code does not fit in %d bits" % x)
    if x == 6:   # 4 codes -> 3 bytes
        q = c.reshape(c.shape[0], -1, 4)
        out = np.empty((c.shape[0], q.shape[1], 3), dtype=np.uint8)
        out[:, :, 0] = (q[:, :, 0] << 2) | (q[:, :, 1] >> 4)
        out[:, :, 1] = (q[:, :, 1] << 4) | (q[:, :, 2] >> 2)
        out[:, :, 2] = (q[:, :, 2] << 6) | q[:, :, 3]
    elif x == 4:  # 2 codes -> 1 byte
        out = (c[:, 0::2] << 4) | c[:, 1::2]
    else:        # 8 codes -> 5 bytes
        q = c.reshape(c.shape[0], -1, 8)
        out = np.empty((c.shape[0], q.shape[1], 5), dtype=np.uint8)
        out[:, :, 0] = (q[:, :, 0] << 3) | (q[:, :, 1] >> 2)
        out[:, :, 1] = (q[:, :, 1] << 6) | (q[:, :, 2] << 1) | (q[:, :, 3] >> 4)
        out[:, :, 2] = (q[:, :, 3] << 4) | (q[:, :, 4] >> 1)
        out[:, :, 3] = (q[:, :, 4] << 7) | (q[:, :, 5] << 2) | (q[:, :, 6] >> 3)
        out[:, :, 4] = (q[:, :, 6] << 5) | q[:, :, 7]
    return out.reshape(c.shape[0], -1).view(np.int32)


def unpack_raw(raw, E=3, M=2):
    """Inverse of pack_raw."""
    x = _check(E, M)
    b = np.ascontiguousarray(raw).view(np.uint8)
    bits = np.unpackbits(b, axis=1, bitorder="big").reshape(b.shape[0], -1, x)
    return (bits << np.arange(x - 1, -1, -1, dtype=np.uint8)).sum(axis=2).astype(np.uint8)


def dequantize_codes(codes, scales, E=3, M=2):
    """float64 value(code) * scale, for checks."""
    x = _check(E, M)
    c = np.asarray(codes)
    mags = magnitudes(E, M)
    v = np.where(c >> (x - 1), -1.0, 1.0) * mags[c & ((1 << (x - 1)) - 1)]
    return v * np.asarray(scales, dtype=np.float64)[:, None]
