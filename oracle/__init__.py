"""TEST INFRASTRUCTURE ONLY -- Python front end of the CPU oracle for the FPx linear-layer path.

Only tests/, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this package, and
only as the checker / timed CPU baseline.  The product (``fp6_llm_amd``) never imports it.

Three layers live here:

* ``liborc.so`` (``fpx_oracle.c``): scalar C restatement of the reference algorithm, reached through ctypes.
* numpy closed forms that do NOT share code with the C restatement (``prepack_closed_form``, ``value_table``,
  ``codes_to_raw``/``raw_to_codes``): used to cross-examine it.
* ``ref_prepack``: the reference's own ``weight_prepacking.h`` compiled unmodified (``oracle/_ref``), when built.
"""
import ctypes
import os
import subprocess
from fractions import Fraction

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None


def build(force=False):
    """Compile liborc.so (and oracle/_ref when the reference checkout exists) with the Makefile beside this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liborc.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        u8p, u16p, f32p = ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p
        L.orc_prepack.argtypes = [ctypes.c_int, ctypes.c_int, u8p, u8p, ctypes.c_size_t, ctypes.c_size_t]
        L.orc_prepack.restype = ctypes.c_int
        L.orc_unpack_codes.argtypes = [ctypes.c_int, ctypes.c_int, u8p, u8p, ctypes.c_size_t, ctypes.c_size_t]
        L.orc_unpack_codes.restype = ctypes.c_int
        L.orc_dequant.argtypes = [ctypes.c_int, ctypes.c_int, u16p, u8p, ctypes.c_size_t, ctypes.c_size_t, u16p]
        L.orc_dequant.restype = ctypes.c_int
        L.orc_splitk_range.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                       ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
        L.orc_splitk_range.restype = None
        L.orc_splitk_reduce.argtypes = [u16p, f32p, ctypes.c_size_t, ctypes.c_int]
        L.orc_splitk_reduce.restype = None
        L.orc_gemm.argtypes = [u16p, u16p, u16p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int]
        L.orc_gemm.restype = ctypes.c_int
        L.orc_tile_n.argtypes = [ctypes.c_size_t]
        L.orc_tile_n.restype = ctypes.c_int
        L.orc_num_wave.argtypes = [ctypes.c_long] * 4
        L.orc_num_wave.restype = ctypes.c_double
        L.orc_heuristic_splitk.argtypes = [ctypes.c_long] * 3
        L.orc_heuristic_splitk.restype = ctypes.c_int
        L.orc_float_to_half.argtypes = [ctypes.c_float]
        L.orc_float_to_half.restype = ctypes.c_uint16
        L.orc_half_to_float.argtypes = [ctypes.c_uint16]
        L.orc_half_to_float.restype = ctypes.c_float
        _LIB = L
    return _LIB


def ref_lib():
    """The reference's own prepacker (oracle/_ref/libref_prepack.so) or None when it was never built."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, "_ref", "libref_prepack.so")
        if not os.path.exists(path):
            return None
        R = ctypes.CDLL(path)
        R.ref_weight_matrix_prepacking_fp_eXmY.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                                           ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
        R.ref_weight_matrix_prepacking_fp_eXmY.restype = None
        R.ref_weight_matrix_prepacking.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
        R.ref_weight_matrix_prepacking.restype = None
        R.ref_weight_matrix_prepacking_x_bit.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                                         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
        R.ref_weight_matrix_prepacking_x_bit.restype = ctypes.c_int
        _REF = R
    return _REF


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def bit_width(E, M):
    return 1 + E + M


def _as_bytes(raw):
    """Accepts int32 [OC, IC/32*x] or uint8 [OC, IC*x/8]; returns a contiguous uint8 [OC, row_bytes] view."""
    raw = np.ascontiguousarray(raw)
    if raw.dtype != np.uint8:
        raw = raw.view(np.uint8)
    return raw


# ---------------------------------------------------------------------------------------------- C restatement


def prepack(raw, E=3, M=2):
    """Restates weight_matrix_prepacking_x_bit (utils/weight_prepacking.h:118-196). Returns uint8 of raw's shape."""
    b = _as_bytes(raw)
    rows, row_bytes = b.shape
    K = row_bytes * 8 // bit_width(E, M)
    out = np.empty_like(b)
    rc = lib().orc_prepack(E, M, _ptr(out), _ptr(b), rows, K)
    if rc != 0:
        raise ValueError("orc_prepack rejected E=%d M=%d rows=%d K=%d" % (E, M, rows, K))
    return out


def unpack_codes(raw, E=3, M=2):
    b = _as_bytes(raw)
    rows, row_bytes = b.shape
    K = row_bytes * 8 // bit_width(E, M)
    codes = np.empty((rows, K), dtype=np.uint8)
    rc = lib().orc_unpack_codes(E, M, _ptr(codes), _ptr(b), rows, K)
    if rc != 0:
        raise ValueError("orc_unpack_codes rejected the input")
    return codes


def dequant(raw, scale, E=3, M=2):
    """Restates DeQuantMatrix_FPx_To_FP16 (utils/weight_dequant.h:10-48). scale: float16 [OC]. Returns float16 [OC, IC]."""
    b = _as_bytes(raw)
    rows, row_bytes = b.shape
    K = row_bytes * 8 // bit_width(E, M)
    s = np.ascontiguousarray(scale, dtype=np.float16)
    assert s.shape == (rows,)
    out = np.empty((rows, K), dtype=np.float16)
    rc = lib().orc_dequant(E, M, _ptr(out), _ptr(b), rows, K, _ptr(s))
    if rc != 0:
        raise ValueError("orc_dequant rejected the input")
    return out


def gemm(wdq, x, splitK=1):
    """out[N, OC] = fp16_rn(sum_k float(wdq[m,k]) * float(x[n,k])), FP32 accumulation, reference split-K partition."""
    wdq = np.ascontiguousarray(wdq, dtype=np.float16)
    x = np.ascontiguousarray(x, dtype=np.float16)
    Mg, K = wdq.shape
    N = x.shape[0]
    assert x.shape[1] == K
    out = np.empty((N, Mg), dtype=np.float16)
    rc = lib().orc_gemm(_ptr(out), _ptr(wdq), _ptr(x), Mg, N, K, splitK)
    if rc != 0:
        raise ValueError("orc_gemm rejected the input")
    return out


def splitk_range(K, splitK, split):
    a, b = ctypes.c_size_t(), ctypes.c_size_t()
    lib().orc_splitk_range(K, splitK, split, ctypes.byref(a), ctypes.byref(b))
    return a.value, b.value


def splitk_reduce(workspace):
    """workspace float32 [splitK, N, OC] -> float16 [N, OC] (include/kernel_reduction.cuh:28-47)."""
    ws = np.ascontiguousarray(workspace, dtype=np.float32)
    s = ws.shape[0]
    out = np.empty(ws.shape[1:], dtype=np.float16)
    lib().orc_splitk_reduce(_ptr(out), _ptr(ws), out.size, s)
    return out


def tile_n(N):
    return lib().orc_tile_n(N)


def num_wave(M, N, splitK, sms):
    return lib().orc_num_wave(M, N, splitK, sms)


def heuristic_splitk(M, N, sms):
    return lib().orc_heuristic_splitk(M, N, sms)


# ---------------------------------------------------------------------------------------------- the real reference


def ref_prepack(raw, E=3, M=2):
    """The reference's own weight_matrix_prepacking_fp_eXmY. Input is padded: the reference reads one byte past it."""
    R = ref_lib()
    if R is None:
        raise RuntimeError("oracle/_ref is not built (needs the reference checkout)")
    b = _as_bytes(raw)
    rows, row_bytes = b.shape
    K = row_bytes * 8 // bit_width(E, M)
    padded = np.zeros(b.size + 64, dtype=np.uint8)
    padded[: b.size] = b.reshape(-1)
    out = np.zeros(b.size + 64, dtype=np.uint8)
    if (E, M) in ((3, 2), (2, 2)):
        R.ref_weight_matrix_prepacking_fp_eXmY(E, M, _ptr(out), _ptr(padded), rows, K)
    elif R.ref_weight_matrix_prepacking_x_bit(E, M, _ptr(out), _ptr(padded), rows, K) != 0:  # the template, other (E,M)
        raise ValueError("no instantiation of the reference's prepacking template for E=%d M=%d" % (E, M))
    return out[: b.size].reshape(b.shape).copy()


# ---------------------------------------------------------------------------------------------- independent numpy forms


def codes_to_raw(codes, E=3, M=2):
    """[OC, IC] codes -> uint8 [OC, IC*x/8]: per-row MSB-first bitstream (bit 0 = MSB of byte 0)."""
    x = bit_width(E, M)
    codes = np.asarray(codes, dtype=np.uint8)
    bits = (codes[:, :, None] >> np.arange(x - 1, -1, -1, dtype=np.uint8)) & 1
    return np.packbits(bits.reshape(codes.shape[0], -1), axis=1, bitorder="big")


def raw_to_codes(raw, E=3, M=2):
    x = bit_width(E, M)
    b = _as_bytes(raw)
    bits = np.unpackbits(b, axis=1, bitorder="big").reshape(b.shape[0], -1, x)
    weights = (1 << np.arange(x - 1, -1, -1)).astype(np.uint8)
    return (bits * weights).sum(axis=2).astype(np.uint8)


def value_of_code(code, E=3, M=2):
    """Format definition in exact arithmetic: (-1)^s 2^(e-b)(1+m/2^M), e=0 => (-1)^s 2^(1-b) m/2^M, b=2^(E-1)-1.
    The all-ones exponent is an ordinary value (utils/weight_quant.h:22-25: FP6 max 28, min subnormal 0.0625)."""
    x = bit_width(E, M)
    s = (code >> (x - 1)) & 1
    e = (code >> M) & ((1 << E) - 1)
    m = code & ((1 << M) - 1)
    b = (1 << (E - 1)) - 1
    if e == 0:
        v = Fraction(2) ** (1 - b) * Fraction(m, 1 << M)
    else:
        v = Fraction(2) ** (e - b) * (1 + Fraction(m, 1 << M))
    return -v if s else v


def value_table(E=3, M=2):
    x = bit_width(E, M)
    tab = np.array([float(value_of_code(c, E, M)) for c in range(1 << x)], dtype=np.float64)
    sign = np.where(np.arange(1 << x) >> (x - 1), -1.0, 1.0)
    return np.copysign(tab, sign)  # keeps the sign of the negative-zero code (sign bit set, all other bits clear)


_ORDER = {
    4: [2, 6, 4, 8, 1, 5, 3, 7],
    2: [2, 6, 10, 14, 4, 8, 12, 16, 1, 5, 9, 13, 3, 7, 11, 15],
    1: [2, 6, 10, 14, 18, 22, 26, 30, 4, 8, 12, 16, 20, 24, 28, 32,
        1, 5, 9, 13, 17, 21, 25, 29, 3, 7, 11, 15, 19, 23, 27, 31],
}


def prepack_closed_form(codes, E=3, M=2):
    """Reference layout from a closed-form index map (no passes, no per-lane streams): for every 32-bit word of a
    segment array and every fragment position in it, the (row, column) whose bits sit there.
    word = ((i*(K/16) + j)*w + q)*32 + lane; fragment p (MSB first) holds pre-interleave fragment order_w[p]-1 = pre;
    pre -> 16-row block k = q*(4/w) + pre//8, element el = pre%8; lane = 4g+t;
    row = 64i + 16k + g + 8*((el>>1)&1), col = 16j + 2t + (el&1) + 8*(el>>2)."""
    x = bit_width(E, M)
    codes = np.asarray(codes, dtype=np.uint32)
    rows, K = codes.shape
    out = []
    consumed = 0
    for w in (1, 2, 4):
        if not (x & w):
            continue
        shift = x - consumed - w  # segments are cut MSB-down in the order 1,2,4
        consumed += w
        piece = (codes >> shift) & ((1 << w) - 1)
        nfrag = 32 // w
        i, j, q, lane, p = np.meshgrid(np.arange(rows // 64), np.arange(K // 16), np.arange(w), np.arange(32),
                                       np.arange(nfrag), indexing="ij")
        pre = np.array(_ORDER[w])[p] - 1
        k = q * (4 // w) + pre // 8
        el = pre % 8
        g, t = lane // 4, lane % 4
        row = 64 * i + 16 * k + g + 8 * ((el >> 1) & 1)
        col = 16 * j + 2 * t + (el & 1) + 8 * (el >> 2)
        frag = piece[row, col].astype(np.uint64) << (32 - w * (p + 1)).astype(np.uint64)
        words = frag.sum(axis=-1).astype(np.uint32)  # fragments do not overlap, so the sum is an OR
        out.append(words.reshape(-1).view(np.uint8))
    return np.concatenate(out).reshape(rows, -1)


def dequant_from_definition(codes, scale, E=3, M=2):
    """fp16_rn(value(code) * scale) in float64 (the product has <= 3+11 significant bits, so it is exact)."""
    tab = value_table(E, M)
    prod = tab[np.asarray(codes)] * np.asarray(scale, dtype=np.float16).astype(np.float64)[:, None]
    return prod.astype(np.float16)


def dequant_grouped_from_definition(codes, scale, exps, E=3, M=2):
    """fp16_rn(value(code) * 2^(b-127) * scale) with one exponent byte b per (row, 128 columns): the definition of this
    build's per-group scales.  The reference has no per-group scales (one half per row, fp6_llm/csrc/fp6_linear.cuh:24), so
    no reference output exists for it; it is pinned by reduction to the row-scale dequantizer (tests/test_oracle.py): unit
    exponents give dequant_from_definition, a single exponent b with scale * 2^(b-127) representable gives
    dequant(raw, scale * 2^(b-127)) bit for bit, and mixed groups give the column blocks of those."""
    tab = value_table(E, M)
    codes = np.asarray(codes)
    f = np.repeat(np.exp2(np.asarray(exps, dtype=np.float64) - 127.0), 128, axis=1)[:, :codes.shape[1]]
    prod = tab[codes] * f * np.asarray(scale, dtype=np.float16).astype(np.float64)[:, None]   # exact in float64
    with np.errstate(over="ignore"):
        return prod.astype(np.float16)


# ---------------------------------------------------------------------------------------------- the quantizer, from its definition
# The reference ships no rounding quantizer: its only cast truncates, throws out of range and is wired to no API
# (fp6_llm/csrc/utils/weight_quant.h:9-105).  What the build's quantizers (numpy on the host, HIP on the device) must
# produce is therefore fixed here by the definition alone, in exact arithmetic, sharing no code with either of them:
#   scale[row] = fp16_rn(absmax(row) / max_value)   (absmax over the finite entries; 1.0 where that rounds to zero)
#   code       = the representable magnitude nearest to |w| / scale[row], ties to the even code, clamped at max_value,
#                with the sign of w;  NaN counts as +0, +-Inf as +-max_value.
# PARITY UNPINNED against reference output (there is none to compare with); pinned by: quantize(value(code) * s) == code for
# every code, ties between neighbours, monotonicity and the clamp (tests/test_oracle.py).


def _fp16_rn_of_fraction(q):
    """Round-to-nearest-even of a non-negative Fraction to binary16, returned as np.float16 (exact, no double rounding)."""
    if q <= 0:
        return np.float16(0.0)
    e = q.numerator.bit_length() - q.denominator.bit_length()
    if Fraction(2) ** e > q:
        e -= 1
    elif Fraction(2) ** (e + 1) <= q:
        e += 1
    ulp = Fraction(2) ** (max(e, -14) - 10)
    n = q / ulp
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    v = fl * ulp
    if v >= 65520:
        return np.float16(np.inf)
    return np.float16(float(v))     # exact: v is a binary16 value


def _nearest_codes_exact(w, factor, E, M):
    """codes for weights w (float64 holding fp16/bf16/fp32 values exactly) against per-element factors (float64 holding
    fp16 scale times a power of two exactly).  |w| >= mid * factor is decided on exact products: a midpoint between two
    neighbouring magnitudes has at most 7 significant bits and the factor 11, so mid * factor is exact in float64."""
    x = bit_width(E, M)
    mags = [abs(value_of_code(c, E, M)) for c in range(1 << (x - 1))]
    a = np.abs(w)
    idx = np.zeros(w.shape, dtype=np.int64)
    for i in range(len(mags) - 1):
        mid = float((mags[i] + mags[i + 1]) / 2)
        bound = mid * factor
        above = a > bound
        tie = a == bound
        # past the midpoint: at least i+1; exactly on it: the even one of i and i+1
        idx = np.where(above | (tie & (i % 2 == 1)), np.maximum(idx, i + 1), idx)
    idx = np.where(np.isnan(w), 0, idx)
    sign = np.where(np.isnan(w), 0, np.signbit(w).astype(np.int64))
    return ((sign << (x - 1)) | idx).astype(np.uint8)


def quantize_from_definition(weight, E=3, M=2):
    """weight [OC, IC] (float16 / float32 array; bf16 values passed as float32) -> (codes uint8 [OC, IC], scales float16 [OC])."""
    x = bit_width(E, M)
    w = np.asarray(weight, dtype=np.float64)
    top = abs(value_of_code((1 << (x - 1)) - 1, E, M))
    finite = np.where(np.isfinite(w), np.abs(w), 0.0)
    scales = np.array([_fp16_rn_of_fraction(Fraction(float(m)) / top) for m in finite.max(axis=1)], dtype=np.float16)
    scales = np.where(scales == 0, np.float16(1.0), scales).astype(np.float16)
    return _nearest_codes_exact(w, np.broadcast_to(scales.astype(np.float64)[:, None], w.shape), E, M), scales


def quantize_grouped_from_definition(weight, E=3, M=2):
    """As quantize_from_definition, plus one exponent byte per (row, 128 columns): 127 + k with k the smallest integer in
    [-15, 0] such that the group's largest finite |w| <= max_value * 2^k * scale[row] (decided on exact products); codes are
    chosen against scale[row] * 2^k.  -> (codes, scales, exps uint8 [OC, ceil(IC/128)]).  PARITY UNPINNED like the
    per-group scales themselves (no reference behaviour exists)."""
    x = bit_width(E, M)
    w = np.asarray(weight, dtype=np.float64)
    OC, IC = w.shape
    top = float(abs(value_of_code((1 << (x - 1)) - 1, E, M)))
    finite = np.where(np.isfinite(w), np.abs(w), 0.0)
    scales = np.array([_fp16_rn_of_fraction(Fraction(float(m)) / Fraction(top)) for m in finite.max(axis=1)], dtype=np.float16)
    scales = np.where(scales == 0, np.float16(1.0), scales).astype(np.float16)
    groups = (IC + 127) // 128
    pad = np.zeros((OC, groups * 128))
    pad[:, :IC] = finite
    gmax = pad.reshape(OC, groups, 128).max(axis=2)
    sc = scales.astype(np.float64)[:, None]
    k = np.zeros((OC, groups), dtype=np.int64)
    for cand in range(-1, -16, -1):      # top * 2^cand * scale is exact in float64 (4 + 11 significant bits)
        k = np.where(gmax <= top * np.exp2(float(cand)) * sc, cand, k)
    factor = np.repeat(np.exp2(k.astype(np.float64)), 128, axis=1)[:, :IC] * sc
    return _nearest_codes_exact(w, factor, E, M), scales, (k + 127).astype(np.uint8)


def gemm_f64(wdq, x):
    """float64 accumulation of the dequantized weights: the arbiter for GEMM tolerance checks. Returns float64 [N, OC]."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(wdq, dtype=np.float64).T
