"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each check is chosen so that a plausible mistake in the oracle fails it: fixtures produced by the reference's own
prepacker, the known-answer constants written in the reference's tests, an independent closed-form index map,
the format definition evaluated in exact rational arithmetic, and invariants (bijection, in-place == out-of-place).
"""
import glob
import hashlib
import json
import os
import re
import struct
from fractions import Fraction

import numpy as np
import pytest

import oracle

# Inputs are made here, with nothing of the product in the way: the oracle is pinned before the product is compared with it.


def _splitmix_codes(seed, OC, IC, E, M):
    """The codes of the committed fixtures: element i = top x bits of splitmix64(seed + (i+1) * golden ratio)."""
    mask = np.uint64(0xFFFFFFFFFFFFFFFF)
    with np.errstate(over="ignore"):
        z = (np.uint64(seed) + np.arange(1, OC * IC + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)) & mask
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & mask
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & mask
        z = z ^ (z >> np.uint64(31))
    return (z >> np.uint64(64 - (1 + E + M))).astype(np.uint8).reshape(OC, IC)


def _problem(seed, OC, IC, BS, E=3, M=2):
    """Uniform random codes, scales in [1e-3, 1e-2], N(0,1) activations: (raw int32, scales, x)."""
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 1 << (1 + E + M), size=(OC, IC), dtype=np.uint8)
    return (oracle.codes_to_raw(codes, E, M).view(np.int32), rng.uniform(1e-3, 1e-2, OC).astype(np.float16),
            rng.standard_normal((BS, IC)).astype(np.float16))

FORMATS = [(3, 2), (2, 2), (2, 3), (2, 1)]
CODE_OF_ONE = {(3, 2): 0b001100, (2, 2): 0b00100, (2, 3): 0b001000, (2, 1): 0b0010}   # sign 0, exponent = bias, mantissa 0
# "all weights = 1.0" bit patterns quoted in the reference: tests/python/kernel_test_fpx.py:88-107 (FP5_e2m2) and :110-131 (FP6_e3m2)
ONES = {(2, 2): [272762913, 1107829124, 136414224, 562303042, 2215657992], (3, 2): [806142768, 3274706115, 214118412]}


def _ones_raw(E, M, OC, IC):
    if (E, M) not in ONES:   # formats the reference's tests do not cover: the same tensor from the format definition
        return oracle.codes_to_raw(np.full((OC, IC), CODE_OF_ONE[(E, M)], np.uint8), E, M).view(np.int32)
    words = np.array(ONES[(E, M)], dtype=np.uint32)
    reps = IC // (32 * len(words) // (1 + E + M))
    return np.tile(words, (OC, reps)).view(np.int32)


# ------------------------------------------------------------------------------------------------ raw format
@pytest.mark.parametrize("E,M", FORMATS)
def test_all_ones_pattern_decodes_to_the_code_of_one(E, M):
    # 1.0 = sign 0, exponent = bias, mantissa 0: e3m2 -> 0 011 00 = 12, e2m2 -> 0 01 00 = 4 (kernel_test_fpx.py:102,125)
    raw = _ones_raw(E, M, 64, 128)
    codes = oracle.unpack_codes(raw, E, M)
    assert set(np.unique(codes)) == {CODE_OF_ONE[(E, M)]}
    assert (oracle.raw_to_codes(raw, E, M) == codes).all()


@pytest.mark.parametrize("E,M", FORMATS)
def test_bitstream_is_msb_first(E, M):
    x = 1 + E + M
    codes = np.zeros((64, 64), dtype=np.uint8)
    codes[0, 0] = (1 << x) - 1      # first code all ones -> top x bits of byte 0
    codes[0, 1] = 1                 # second code = 1 -> its LSB is bit 2x-1 of the stream
    raw = oracle.codes_to_raw(codes, E, M)
    assert raw[0, 0] >> (8 - x) == (1 << x) - 1
    bit = 2 * x - 1
    assert (raw[0, bit // 8] >> (7 - bit % 8)) & 1 == 1
    assert (oracle.unpack_codes(raw, E, M) == codes).all()


# ------------------------------------------------------------------------------------------------ prepacking
def test_golden_prepack_fixtures(golden_dir):
    files = sorted(glob.glob(os.path.join(golden_dir, "prepack_e*_*.npz")))
    assert len(files) == 12
    for f in files:
        E, M = (int(v) for v in re.search(r"prepack_e(\d)m(\d)_", f).groups())
        z = np.load(f)
        got = oracle.prepack(z["raw"], E, M)
        assert got.tobytes() == z["packed"].tobytes(), f
        # the fixture's input is what the generator produces from its seed (fixtures are reproducible)
        OC = z["raw"].shape[0]
        IC = z["raw"].shape[1] * 32 // (1 + E + M)
        assert (oracle.codes_to_raw(_splitmix_codes(int(z["seed"]), OC, IC, E, M), E, M).view(np.int32) == z["raw"]).all()


@pytest.mark.parametrize("E,M", FORMATS)
def test_golden_hash_config1(golden_dir, E, M):
    name = "e%dm%d_256x1024_seed1001" % (E, M)
    ref = json.load(open(os.path.join(golden_dir, "prepack_hashes.json")))[name]
    raw = oracle.codes_to_raw(_splitmix_codes(1001, 256, 1024, E, M), E, M).view(np.int32)
    assert hashlib.sha256(raw.tobytes()).hexdigest() == ref["raw_sha256"]
    assert hashlib.sha256(oracle.prepack(raw, E, M).tobytes()).hexdigest() == ref["packed_sha256"]


@pytest.mark.parametrize("E,M", FORMATS)
def test_prepack_matches_reference_build_when_present(E, M):
    if oracle.ref_lib() is None:
        pytest.skip("oracle/_ref not built on this machine")
    rng = np.random.default_rng(5)
    raw = rng.integers(0, 256, size=(192, 128 * (1 + E + M) // 8), dtype=np.uint8)
    assert (oracle.prepack(raw, E, M) == oracle.ref_prepack(raw, E, M)).all()


@pytest.mark.parametrize("E,M", FORMATS)
def test_prepack_closed_form_index_map(E, M):
    x = 1 + E + M
    rng = np.random.default_rng(7)
    codes = rng.integers(0, 1 << x, size=(128, 192), dtype=np.uint8)
    raw = oracle.codes_to_raw(codes, E, M)
    assert (oracle.prepack(raw, E, M) == oracle.prepack_closed_form(codes, E, M)).all()


@pytest.mark.parametrize("E,M", FORMATS)
def test_prepack_all_ones_known_answer(E, M):
    # 1.0 splits into an all-zero high segment (if any) and the low nibble of its code (1100 for e3m2, 0100 for e2m2,
    # 1000 for e2m3, 0010 for e2m1) in every 4-bit fragment
    raw = _ones_raw(E, M, 64, 128)
    words = oracle.prepack(raw, E, M).view(np.uint32).reshape(-1)
    hi_words = 64 * 128 * (1 + E + M - 4) // 32
    assert (words[:hi_words] == 0).all()
    assert (words[hi_words:] == (CODE_OF_ONE[(E, M)] & 15) * 0x11111111).all()


@pytest.mark.parametrize("E,M", FORMATS)
def test_prepack_is_a_bit_permutation_and_in_place_safe(E, M):
    x = 1 + E + M
    rng = np.random.default_rng(9)
    raw = rng.integers(0, 256, size=(64, 64 * x // 8), dtype=np.uint8)
    packed = oracle.prepack(raw, E, M)
    assert np.unpackbits(raw).sum() == np.unpackbits(packed).sum()
    # one-hot inputs map to one-hot outputs at distinct positions (bijection on bits), sampled
    seen = set()
    for bit in range(0, raw.size * 8, 97):
        one = np.zeros(raw.size, dtype=np.uint8)
        one[bit // 8] = 0x80 >> (bit % 8)
        out = np.unpackbits(oracle.prepack(one.reshape(raw.shape), E, M))
        assert out.sum() == 1
        seen.add(int(out.argmax()))
    assert len(seen) == len(range(0, raw.size * 8, 97))
    # aliased call
    buf = raw.copy()
    rc = oracle.lib().orc_prepack(E, M, buf.ctypes.data, buf.ctypes.data, 64, 64)
    assert rc == 0 and (buf == packed).all()


def test_prepack_rejects_what_the_reference_asserts():
    raw = np.zeros((32, 48), dtype=np.uint8)
    with pytest.raises(ValueError):
        oracle.prepack(raw, 3, 2)              # rows % 64
    with pytest.raises(ValueError):
        oracle.prepack(np.zeros((64, 48), np.uint8), 4, 3)  # unsupported format


# ------------------------------------------------------------------------------------------------ dequantisation
def _half_bits_of_fraction(v):
    """IEEE binary16 bits of an exact rational, rounded to nearest even by Python's own packer ('e' format)."""
    return struct.unpack("<H", struct.pack("<e", float(v)))[0]  # float(v) is exact here: <= 14 significant bits


@pytest.mark.parametrize("E,M", FORMATS)
def test_format_constants(E, M):
    tab = oracle.value_table(E, M)
    x = 1 + E + M
    if (E, M) == (3, 2):  # utils/weight_quant.h:22-25: max 28, smallest subnormal 0.0625
        assert tab[0b011111] == 28.0 and tab[0b000001] == 0.0625 and tab[0b001100] == 1.0
    elif (E, M) == (2, 2):
        assert tab[0b01111] == 7.0 and tab[0b00001] == 0.25 and tab[0b00100] == 1.0
    elif (E, M) == (2, 3):  # OCP Microscaling Formats (MX) v1.0, table 3: FP6 E2M3 max normal 7.5, min subnormal 0.125
        assert tab[0b011111] == 7.5 and tab[0b000001] == 0.125 and tab[0b001000] == 1.0 and tab[0b000111] == 0.875
    else:                   # same table: FP4 E2M1 max normal 6.0, min subnormal 0.5; the eight magnitudes of the format
        assert list(tab[:8]) == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert (tab[(1 << (x - 1)):] == -tab[: (1 << (x - 1))]).all()
    assert np.signbit(tab[1 << (x - 1)]) and tab[1 << (x - 1)] == 0.0   # negative zero exists
    assert np.isfinite(tab).all()                                       # exponent all-ones is an ordinary value
    assert (np.diff(tab[: (1 << (x - 1))]) > 0).all()                   # magnitude code order is value order


@pytest.mark.parametrize("E,M", FORMATS)
def test_dequant_all_ones_is_one(E, M):
    raw = _ones_raw(E, M, 64, 128)
    out = oracle.dequant(raw, np.ones(64, np.float16), E, M)
    assert (out == np.float16(1.0)).all()


@pytest.mark.parametrize("E,M", FORMATS)
def test_dequant_exhaustive_codes_times_scale_samples(E, M):
    """Every code against ~4000 fp16 scales spread over the whole fp16 range (normals, subnormals, zero, big values that
    overflow to inf), checked against the format definition in exact arithmetic."""
    x = 1 + E + M
    ncodes = 1 << x
    scale_bits = np.unique(np.concatenate([np.arange(0, 0x7C00, 8), [1, 2, 3, 0x03FF, 0x0400, 0x3C00, 0x7BFF, 0x8001, 0xBC00, 0xFBFF]]))
    scale_bits = scale_bits[: (len(scale_bits) // 64) * 64].astype(np.uint16)
    scales = scale_bits.view(np.float16)
    K = 64
    codes = np.tile(np.arange(ncodes, dtype=np.uint8), K // ncodes if ncodes <= K else 1)
    codes = np.resize(np.arange(ncodes, dtype=np.uint8), K)[None, :].repeat(len(scales), axis=0)
    raw = oracle.codes_to_raw(codes, E, M)
    got = oracle.dequant(raw, scales, E, M).view(np.uint16)
    # numpy float64 path (exact product, one rounding) for all entries
    want = oracle.dequant_from_definition(codes, scales, E, M).view(np.uint16)
    assert (got == want).all()
    # and, for a sample, pure-Python rationals rounded by struct's binary16 packer (shares nothing with numpy)
    for r in range(0, len(scales), 37):
        s = Fraction(float(scales[r]))
        for c in range(ncodes):
            v = oracle.value_of_code(int(codes[r, c % K]), E, M) * s
            if abs(v) >= 65520:
                want_bits = 0x7C00 | (0x8000 if v < 0 else 0)
            else:
                want_bits = _half_bits_of_fraction(v)
                if v == 0 and ((codes[r, c % K] >> (x - 1)) ^ (scale_bits[r] >> 15)) & 1:
                    want_bits |= 0x8000
            assert got[r, c % K] == want_bits, (r, c, float(scales[r]))


def test_half_conversion_helpers_against_numpy():
    L = oracle.lib()
    rng = np.random.default_rng(3)
    vals = np.concatenate([rng.standard_normal(2000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 2000),
                           np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5], np.float32)])
    for v in vals:
        assert L.orc_float_to_half(float(v)) == np.float32(v).astype(np.float16).view(np.uint16), v
    for h in range(0, 0x7C00, 13):
        assert L.orc_half_to_float(h) == float(np.uint16(h).view(np.float16))


# ------------------------------------------------------------------------------------------------ split-K, launcher logic
@pytest.mark.parametrize("K,s", [(64, 1), (4096, 3), (4096, 13), (1024, 16), (1024, 17), (11008, 5), (256, 8)])
def test_splitk_partition_closed_form(K, s):
    nb = K // 64
    ranges = [oracle.splitk_range(K, s, i) for i in range(s)]
    pos = 0
    for i, (start, n) in enumerate(ranges):
        assert start == pos
        assert n == nb // s + (1 if i < nb % s else 0)   # first nb % s splits are one block longer
        pos += n
    assert pos == nb


def test_splitk_reduce_sums_in_split_order():
    ws = np.zeros((3, 2, 256), dtype=np.float32)
    ws[0] += 1e8
    ws[1] += 1.0
    ws[2] -= 1e8
    out = oracle.splitk_reduce(ws)   # (1e8 + 1) - 1e8 in fp32 = 0, not 1: order matters
    assert (out == 0).all()
    ws2 = np.random.default_rng(1).standard_normal((4, 3, 256)).astype(np.float32)
    want = ((ws2[0] + ws2[1]) + ws2[2]) + ws2[3]
    assert (oracle.splitk_reduce(ws2) == want.astype(np.float16)).all()


def test_tile_n_buckets():
    # fp6_linear.cu:61-75
    assert [oracle.tile_n(n) for n in (1, 8, 9, 16, 17, 32, 33, 64, 65, 128, 129, 1000)] == [8, 8, 16, 16, 32, 32, 64, 64, 64, 64, 64, 64]


def test_heuristic_known_answers():
    # hand-evaluated from fp6_llm/__init__.py:6-23
    known = {(4096, 8, 108): 11, (11008, 8, 108): 4, (10240, 32, 108): 5, (28672, 32, 108): 5, (8192, 32, 108): 6,
             (8192, 128, 108): 3, (8192, 512, 108): 3, (4096, 8, 256): 26, (11008, 8, 256): 10, (8192, 32, 256): 13,
             (8192, 512, 256): 2, (256, 1, 256): 1, (256, 1, 108): 87}
    for args, want in known.items():
        assert oracle.heuristic_splitk(*args) == want, args
    # 4096x8 on 108 SMs: ceil(4096/512)=8 CTAs per split; 11 splits -> 88/108 = 0.815 of one wave, 10 -> 0.74
    assert abs(oracle.num_wave(4096, 8, 11, 108) - 88 / 108) < 1e-12


# ------------------------------------------------------------------------------------------------ GEMM definition
@pytest.mark.parametrize("E,M", FORMATS)
def test_gemm_special_cases(E, M):
    OC, IC = 64, 128
    ones = _ones_raw(E, M, OC, IC)
    wdq = oracle.dequant(ones, np.ones(OC, np.float16), E, M)
    out = oracle.gemm(wdq, np.ones((3, IC), np.float16))
    assert (out == np.float16(IC)).all()                     # all ones => every output = IC (kernel_test_fpx.py:98-99)
    # one-hot activations pick a column of the dequantized weights exactly
    raw, sc, _ = _problem(3, OC, IC, 1, E, M)
    wdq = oracle.dequant(raw, sc, E, M)
    x = np.zeros((2, IC), np.float16)
    x[0, 5] = 1
    x[1, 77] = 1
    out = oracle.gemm(wdq, x)
    # (value equality: a negative-zero weight sums to +0)
    assert (out[0] == wdq[:, 5]).all() and (out[1] == wdq[:, 77]).all()


def test_gemm_against_float64_and_split_k():
    raw, sc, x = _problem(11, 64, 256, 5)
    wdq = oracle.dequant(raw, sc)
    ref = oracle.gemm_f64(wdq, x)
    for s in (1, 2, 3, 4, 7):
        out = oracle.gemm(wdq, x, s).astype(np.float64)
        den = np.maximum(np.abs(ref), np.sqrt((ref ** 2).mean()))
        assert (np.abs(out - ref) / den).max() < 2e-3
    with pytest.raises(ValueError):
        oracle.gemm(wdq, x, 0)


# ------------------------------------------------------------------------------------------------ the quantizer's definition
def test_fp16_rounding_of_exact_fractions():
    """oracle._fp16_rn_of_fraction against Python's binary16 packer on values that are exact doubles (so the packer sees the
    true value and rounds once), including halfway cases, subnormals and the overflow threshold."""
    rng = np.random.default_rng(77)
    vals = [0.0, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25, 2.0 ** -14, 65504.0, 65519.99, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11,
            (1 + 2.0 ** -10) * 2.0 ** -14, 6.1e-5, 0.333251953125]
    vals += list(np.exp(rng.uniform(np.log(1e-8), np.log(6e4), 3000)))
    vals += [float(np.float16(v)) + float(np.float16(v)) * 2.0 ** -11 for v in np.exp(rng.uniform(np.log(1e-4), np.log(3e4), 500))]   # near ties
    for v in vals:
        want = np.frombuffer(struct.pack("<e", v), dtype=np.float16)[0]
        got = oracle._fp16_rn_of_fraction(Fraction(v))
        assert got.view(np.uint16) == want.view(np.uint16), (v, got, want)
    assert np.isinf(oracle._fp16_rn_of_fraction(Fraction(65520)))
    # a value no double holds exactly: 1/3 rounds to 0x3555
    assert oracle._fp16_rn_of_fraction(Fraction(1, 3)).view(np.uint16) == 0x3555


@pytest.mark.parametrize("E,M", FORMATS)
def test_quantizer_definition_is_pinned(E, M):
    """Nothing in the reference says which code a value rounds to (its cast truncates, utils/weight_quant.h:30-53), so the
    definition in oracle.quantize_from_definition is pinned by what the mathematics fixes."""
    x = 1 + E + M
    half = 1 << (x - 1)
    vals = np.array([float(oracle.value_of_code(c, E, M)) for c in range(1 << x)])
    vals = np.copysign(np.abs(vals), np.where(np.arange(1 << x) >= half, -1.0, 1.0))
    top = np.abs(vals).max()
    for s in (1.0, 0.5, 0.0078125, 3.0, float(np.float16(0.00123)), float(np.float16(1.7)), 2.0 ** -20):
        # every representable value times the scale maps back to its own code (the row holds the maximum, so scale == s)
        codes, sc = oracle.quantize_from_definition((vals * s)[None, :], E, M)
        assert float(sc[0]) == s, (s, sc)
        assert (codes[0] == np.arange(1 << x)).all()
        # midpoints between neighbours go to the even code; a hair to either side goes to that side
        mags = np.abs(vals[:half])
        mid = (mags[:-1] + mags[1:]) / 2
        row = np.concatenate([[top], mid, mid * (1 + 2.0 ** -20), mid * (1 - 2.0 ** -20)]) * s
        codes, sc = oracle.quantize_from_definition(row[None, :], E, M)
        n = len(mid)
        assert (codes[0, 1:1 + n] % 2 == 0).all() and (np.abs(codes[0, 1:1 + n].astype(int) - np.arange(n)) <= 1).all()
        assert (codes[0, 1 + n:1 + 2 * n] == np.arange(1, n + 1)).all() and (codes[0, 1 + 2 * n:] == np.arange(n)).all()
    # monotone, and never farther than half a step from the value
    v = np.linspace(-top, top, 5001)
    codes, sc = oracle.quantize_from_definition(v[None, :], E, M)
    assert float(sc[0]) == 1.0
    deq = vals[codes[0]]
    assert (np.diff(deq) >= 0).all() and (np.abs(deq - v) <= np.diff(np.abs(vals[:half])).max() / 2).all()
    # clamp, signs, zeros, non-finite entries
    row = np.array([top, 5 * top, -7 * top, 0.0, -0.0, np.nan, np.inf, -np.inf])
    codes, sc = oracle.quantize_from_definition(row[None, :], E, M)
    assert float(sc[0]) == 5.0 or float(sc[0]) == 7.0     # absmax of the finite entries is 7 * top
    assert codes[0].tolist()[2:] == [2 * half - 1, 0, half, 0, half - 1, 2 * half - 1]
    z, sz = oracle.quantize_from_definition(np.zeros((2, 32)), E, M)
    assert (z == 0).all() and (sz == 1).all()
    # the scale is the correctly rounded quotient: absmax = top * s for an fp16 s gives s back, and one fp32 ulp more does too
    s16 = np.float16(0.0123)
    _, sc = oracle.quantize_from_definition(np.array([[top * float(s16) * (1 + 2.0 ** -23)]]), E, M)
    assert sc[0] == s16


@pytest.mark.parametrize("E,M", FORMATS)
def test_grouped_quantizer_definition(E, M):
    """PARITY UNPINNED (no reference behaviour): the per-group exponent is the smallest of 112..127 that holds the group."""
    x = 1 + E + M
    top = float(abs(oracle.value_of_code((1 << (x - 1)) - 1, E, M)))
    w = np.zeros((2, 384))
    w[0, 0] = top                      # group 0 holds the row maximum: factor 1
    w[0, 128] = top / 4                # exactly on a boundary: fits under 2^-2
    w[0, 256] = top / 4 * (1 + 2.0 ** -20)   # a hair above it: needs 2^-1
    w[1, 5] = 1.0
    w[1, 300] = 2.0 ** -30             # far below: the smallest factor, 2^-15
    codes, sc, ex = oracle.quantize_grouped_from_definition(w, E, M)
    assert sc[0] == 1.0 and ex[0].tolist() == [127, 125, 126]
    assert ex[1].tolist() == [127, 112, 112]
    c_row, s_row = oracle.quantize_from_definition(w, E, M)
    assert (s_row == sc).all() and (codes[:, :128] == c_row[:, :128]).all()
    assert codes[0, 128] == (1 << (x - 1)) - 1      # against scale/4 the value top/4 is the largest code


# ------------------------------------------------------------------------------------------------ per-group dequantization
# The reference scales per row only (fp6_llm/csrc/fp6_linear.cuh:24, utils/weight_dequant.h:30-43), so the grouped dequantizer
# is pinned by what the mathematics fixes: where the group factor can be folded into a representable row scale it must
# reproduce the (pinned) row-scale dequantizer bit for bit, and a matrix of mixed groups is the column blocks of those.
def _foldable_scales(rng, rows, shift):
    """fp16 scales s such that s * 2^shift is again a normal fp16 number (the product is then exact)."""
    e = rng.integers(max(-14, -14 - shift) + 1, min(15, 15 - shift) - 1, rows)
    m = rng.integers(0, 1024, rows)
    return ((1.0 + m / 1024.0) * np.exp2(e.astype(np.float64))).astype(np.float16)


@pytest.mark.parametrize("E,M", FORMATS)
def test_grouped_dequant_with_unit_factors_is_the_row_scale_dequantizer(E, M):
    rng = np.random.default_rng(7100 + 10 * E + M)
    codes = rng.integers(0, 1 << (1 + E + M), size=(64, 448), dtype=np.uint8)          # 3.5 groups: the last one is cut
    sc = rng.uniform(1e-3, 1e-2, 64).astype(np.float16)
    exps = np.full((64, 4), 127, np.uint8)
    got = oracle.dequant_grouped_from_definition(codes, sc, exps, E, M).view(np.uint16)
    assert (got == oracle.dequant_from_definition(codes, sc, E, M).view(np.uint16)).all()
    assert (got == oracle.dequant(oracle.codes_to_raw(codes, E, M), sc, E, M).view(np.uint16)).all()


@pytest.mark.parametrize("E,M", FORMATS)
@pytest.mark.parametrize("b", [112, 120, 126, 128, 131])
def test_grouped_dequant_with_one_factor_folds_into_the_row_scale(E, M, b):
    """exps == b everywhere and scale * 2^(b-127) representable: the answer is dequant(raw, scale * 2^(b-127)), the C oracle
    that the exhaustive rational check pins."""
    rng = np.random.default_rng(7200 + 100 * b + 10 * E + M)
    codes = np.resize(np.arange(1 << (1 + E + M), dtype=np.uint8), (32, 256))            # every code in every row
    codes = np.roll(codes, rng.integers(0, 64), axis=1)
    sc = _foldable_scales(rng, 32, b - 127)
    folded = (sc.astype(np.float64) * 2.0 ** (b - 127)).astype(np.float16)
    assert (folded.astype(np.float64) == sc.astype(np.float64) * 2.0 ** (b - 127)).all()  # the fold itself is exact
    got = oracle.dequant_grouped_from_definition(codes, sc, np.full((32, 2), b, np.uint8), E, M).view(np.uint16)
    want = oracle.dequant(oracle.codes_to_raw(codes, E, M), folded, E, M).view(np.uint16)
    assert (got == want).all()


@pytest.mark.parametrize("E,M", FORMATS)
def test_grouped_dequant_of_mixed_groups_is_column_blocks_of_folded_ones(E, M):
    """Each 128-column group with its own exponent equals the same columns of the row-scale dequantizer run with that
    group's folded scale; a transposed or off-by-one group index, or a wrong sign of the exponent, fails here."""
    rng = np.random.default_rng(7300 + 10 * E + M)
    rows, K = 48, 576                                                                     # 4.5 groups
    codes = rng.integers(0, 1 << (1 + E + M), size=(rows, K), dtype=np.uint8)
    exps = rng.integers(118, 131, size=(rows, 5)).astype(np.uint8)
    sc = _foldable_scales(rng, rows, -9)[:]                                                # leaves room for shifts in -9..+3
    sc = np.where(np.abs(np.log2(sc.astype(np.float64))) < 4, sc, np.float16(0.75))
    got = oracle.dequant_grouped_from_definition(codes, sc, exps, E, M).view(np.uint16)
    raw = oracle.codes_to_raw(codes, E, M)
    for g in range(5):
        for b in np.unique(exps[:, g]):
            sel = np.nonzero(exps[:, g] == b)[0]
            folded = (sc.astype(np.float64) * 2.0 ** (int(b) - 127)).astype(np.float16)
            assert (folded.astype(np.float64) == sc.astype(np.float64) * 2.0 ** (int(b) - 127)).all()
            want = oracle.dequant(raw, folded, E, M).view(np.uint16)
            lo, hi = 128 * g, min(K, 128 * g + 128)
            assert (got[sel, lo:hi] == want[sel, lo:hi]).all(), (g, int(b))


def test_grouped_dequant_hand_values():
    """e3m2 code 0b001100 is 1.0, 0b011111 is 28: with scale 0.5 and exponents 126 / 129 the values are 0.25, 7 / 2, 56."""
    codes = np.array([[0b001100] * 128 + [0b011111] * 128], np.uint8)
    out = oracle.dequant_grouped_from_definition(codes, np.array([0.5], np.float16), np.array([[126, 126]], np.uint8), 3, 2)
    assert out[0, 0] == np.float16(0.25) and out[0, 128] == np.float16(7.0)
    out = oracle.dequant_grouped_from_definition(codes, np.array([0.5], np.float16), np.array([[129, 129]], np.uint8), 3, 2)
    assert out[0, 0] == np.float16(2.0) and out[0, 128] == np.float16(56.0)
