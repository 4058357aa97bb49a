"""CPU-side product code (libfp6mi.so through the C ABI and the Python API) against the oracle and the golden fixtures.
No GPU compute is called here; the library must load and export every symbol that include/fp6mi.h declares."""
import ctypes
import glob
import hashlib
import json
import os
import re

import numpy as np
import pytest
import torch

import oracle
import fp6_llm_amd as fp6
from fp6_llm_amd import _lib, quant, synth

FORMATS = [(3, 2), (2, 2), (2, 3), (2, 1)]
BLOCK_BYTES = {6: 3072, 5: 2560, 4: 2048}   # native layout: bytes of a 16-row x 256-column block, by bit width
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _problem(seed, OC, IC, E, M):
    raw, sc, _ = synth.uniform_problem(seed, OC, IC, 1, E, M)
    return raw, sc


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fp6mi.h")).read()
    declared = set(re.findall(r"\b(fp6mi_[a-z0-9_]+)\s*\(", header))
    assert declared and declared == set(_lib.EXPORTED)
    L = _lib.lib()
    for name in declared:
        assert hasattr(L, name), name
    assert L.fp6mi_version() >= 100
    assert b"success" in L.fp6mi_error_string(0)


def test_golden_prepack_fixtures(golden_dir):
    for f in sorted(glob.glob(os.path.join(golden_dir, "prepack_e*_*.npz"))):
        E, M = (int(v) for v in re.search(r"prepack_e(\d)m(\d)_", f).groups())
        z = np.load(f)
        raw = np.ascontiguousarray(z["raw"])
        OC, IC = raw.shape[0], raw.shape[1] * 32 // (1 + E + M)
        got = np.empty_like(raw)   # through the C ABI: the Python wrapper keeps the reference's OC % 256 rule
        assert _lib.lib().fp6mi_prepack_ref(E, M, got.ctypes.data, raw.ctypes.data, OC, IC) == 0
        assert got.tobytes() == z["packed"].tobytes(), f


@pytest.mark.parametrize("E,M", FORMATS)
def test_prepack_hash_at_benchmark_size(golden_dir, E, M):
    """Config 2 size (4096x4096): bytes identical to what the reference's prepacker produced (committed SHA-256)."""
    ref = json.load(open(os.path.join(golden_dir, "prepack_hashes.json")))["e%dm%d_4096x4096_seed2001" % (E, M)]
    raw = quant.pack_raw(synth.uniform_codes(2001, 4096, 4096, E, M), E, M)
    assert hashlib.sha256(raw.tobytes()).hexdigest() == ref["raw_sha256"]
    packed = fp6.weight_prepacking_eXmY_cpu(E, M, torch.from_numpy(raw)).numpy()
    assert hashlib.sha256(packed.tobytes()).hexdigest() == ref["packed_sha256"]


@pytest.mark.parametrize("E,M", FORMATS)
@pytest.mark.parametrize("OC,IC", [(256, 64), (256, 320), (512, 1024)])
def test_prepack_dequant_native_against_oracle(E, M, OC, IC):
    raw, sc = _problem(OC + IC, OC, IC, E, M)
    t = torch.from_numpy(raw)
    packed = fp6.weight_prepacking_eXmY_cpu(E, M, t)
    assert packed.shape == t.shape and packed.dtype == torch.int32
    assert packed.numpy().tobytes() == oracle.prepack(raw, E, M).tobytes()
    dq = fp6.weight_dequant_eXmY_cpu(E, M, t, torch.from_numpy(sc)).numpy()
    assert dq.shape == (OC, IC)
    assert (dq.view(np.uint16) == oracle.dequant(raw, sc, E, M).view(np.uint16)).all()
    # native layout: same bits by both routes, and a lossless round trip
    nat = fp6.weight_prepacking_native_cpu(E, M, t)
    assert nat.numel() * 4 == fp6.native_bytes(E, M, OC, IC) == (OC // 16) * ((IC + 255) // 256) * BLOCK_BYTES[1 + E + M]
    assert torch.equal(nat, fp6.to_native(packed, E, M))
    L = _lib.lib()
    back = np.empty_like(raw)
    assert L.fp6mi_unpack_native(E, M, back.ctypes.data, nat.data_ptr(), OC, IC) == 0 and (back == raw).all()
    back2 = np.empty_like(raw)
    assert L.fp6mi_unpack_ref(E, M, back2.ctypes.data, packed.data_ptr(), OC, IC) == 0 and (back2 == raw).all()


def test_fp6_wrappers_are_the_e3m2_case():
    raw, sc = _problem(1, 256, 128, 3, 2)
    t, s = torch.from_numpy(raw), torch.from_numpy(sc)
    assert torch.equal(fp6.weight_prepacking_cpu(t), fp6.weight_prepacking_eXmY_cpu(3, 2, t))
    assert torch.equal(fp6.weight_dequant_cpu(t, s), fp6.weight_dequant_eXmY_cpu(3, 2, t, s))


@pytest.mark.parametrize("E,M", FORMATS)
def test_native_fp6_lane_image_is_the_hardware_operand(E, M):
    """Layout spot check written from the layout's definition, not from the packer: row 16R+m, K block U, lane m+16q,
    code index ci = 8s+j  <->  column 256U + 32s + 8q + j."""
    x = 1 + E + M
    OC, IC = 32, 512
    codes = synth.uniform_codes(42, OC, IC, E, M)
    nat = fp6.weight_prepacking_native_cpu(E, M, torch.from_numpy(quant.pack_raw(codes, E, M))).numpy().view(np.uint32)
    bb = BLOCK_BYTES[x] // 4
    for (R, U, lane) in [(0, 0, 0), (1, 1, 37), (0, 1, 63), (1, 0, 16)]:
        m, q = lane % 16, lane // 16
        blk = nat[(R * 2 + U) * bb:(R * 2 + U + 1) * bb]
        want = [codes[16 * R + m, 256 * U + 32 * s + 8 * q + j] for s in range(8) for j in range(8)]
        if x == 4:
            d = [blk[(i // 4) * 256 + lane * 4 + i % 4] for i in range(8)]
            # four stored dwords per string; dwords five and six of the 6-bit string sit in the two fixed-zero low bits of the fields
            P, Q, R = 0xC30C30C3, 0x30C30C30, 0x0C30C30C
            for h in range(2):
                S = [int(d[4 * h + k]) for k in range(4)]
                D = [S[0] & ~P, S[1] & ~Q, S[2] & ~R, S[3] & ~P, (S[0] & P) | (S[2] & R), (S[1] & Q) | (S[3] & P)]
                big = sum(D[w] << (32 * w) for w in range(6))
                fields = [(big >> (6 * i)) & 63 for i in range(32)]
                assert all(f & 3 == 0 for f in fields)                 # the two bits appended below the mantissa
                assert [f >> 2 for f in fields] == [int(v) for v in want[32 * h:32 * h + 32]]
        elif x == 6:
            d = [blk[(i // 4) * 256 + lane * 4 + i % 4] for i in range(12)]
            for h in range(2):
                big = sum(int(d[6 * h + w]) << (32 * w) for w in range(6))
                got = [(big >> (6 * i)) & 63 for i in range(32)]
                assert got == [int(v) for v in want[32 * h:32 * h + 32]]
        else:
            d = [blk[(i // 4) * 256 + lane * 4 + i % 4] for i in range(8)] + [blk[512 + lane * 2 + i] for i in range(2)]
            # five stored dwords per string; the sixth dword of the 6-bit string sits in the fixed-zero bit of every field
            A, B, C = 0x10410410, 0x04104104, 0x41041041
            for h in range(2):
                S = [int(d[4 * h + k]) for k in range(4)] + [int(d[8 + h])]
                D = [S[0] & ~A, S[1] & ~B, S[2] & ~C, S[3] & ~A, S[4] & ~B,
                     (S[0] & A) | (S[1] & B) | ((((S[2] & C) | (S[3] & A) | (S[4] & B)) << 1) & 0xFFFFFFFF)]
                big = sum(D[w] << (32 * w) for w in range(6))
                fields = [(big >> (6 * i)) & 63 for i in range(32)]
                assert all((f >> 4) & 1 == 0 for f in fields)          # the inserted exponent bit
                got = [(f & 15) | ((f >> 5) << 4) for f in fields]
                assert got == [int(v) for v in want[32 * h:32 * h + 32]]


def test_prepack_in_place_and_padding_is_zero():
    E, M = 3, 2
    raw, _ = _problem(9, 256, 320, E, M)
    L = _lib.lib()
    buf = raw.copy()
    assert L.fp6mi_prepack_ref(E, M, buf.ctypes.data, buf.ctypes.data, 256, 320) == 0
    assert buf.tobytes() == oracle.prepack(raw, E, M).tobytes()
    # K = 320 is padded to 512 in the native layout: the padded columns hold code 0
    nat = fp6.weight_prepacking_native_cpu(E, M, torch.from_numpy(raw))
    wide = np.zeros((256, 512), np.uint8)
    wide[:, :320] = quant.unpack_raw(raw, E, M)
    assert torch.equal(nat, fp6.weight_prepacking_native_cpu(E, M, torch.from_numpy(quant.pack_raw(wide, E, M))))


def test_error_codes_instead_of_aborts():
    L = _lib.lib()
    buf = np.zeros(1 << 16, np.uint8)
    p = buf.ctypes.data
    assert L.fp6mi_prepack_ref(4, 3, p, p, 64, 64) == -1                      # unsupported format (reference: exit(-1))
    assert L.fp6mi_prepack_ref(3, 2, p, p, 32, 64) == -2                      # M % 64 (reference: assert)
    assert L.fp6mi_prepack_ref(3, 2, p, p, 64, 96) == -2                      # K % 64
    assert L.fp6mi_prepack_ref(3, 2, None, p, 64, 64) == -3
    assert L.fp6mi_dequant(1, 2, p, p, 64, 64, p) == -1
    assert L.fp6mi_native_bytes(3, 2, 24, 64) == 0
    assert L.fp6mi_prepack_native(3, 2, p, p, 64, 64) == -2                   # may not alias
    # GEMM argument checks happen on the host before anything is launched
    assert L.fp6mi_linear_native(3, 2, None, p, p, p, p, 100, 1, 64, None, 1) == -2      # M % 256
    assert L.fp6mi_linear_native(3, 2, None, p, p, p, p, 256, 0, 64, None, 1) == -2      # N == 0
    assert L.fp6mi_linear_native(3, 2, None, p, p, p, p, 256, 1, 96, None, 1) == -2      # K % 64
    assert L.fp6mi_linear_native(5, 2, None, p, p, p, p, 256, 1, 64, None, 1) == -1
    assert L.fp6mi_linear_native(3, 2, None, p, p, p, p, 256, 1, 64, None, 2) == -4      # splitK without workspace
    assert L.fp6mi_linear_native(3, 2, None, p, p, p, p, 256, 1, 64, None, 0) == -5
    assert L.fp6mi_linear_native(3, 2, None, None, p, p, p, 256, 1, 64, None, 1) == -3
    assert L.fp6mi_linear_native(3, 2, None, p + 4, p, p, p, 256, 1, 64, None, 1) == -6  # alignment
    assert L.fp6mi_linear_native(3, 2, None, p, p + 1, p, p, 256, 1, 64, None, 1) == -6  # scales are halfs: 2-byte alignment
    for code in (-1, -2, -3, -4, -5, -6, -7, -8):
        assert len(L.fp6mi_error_string(code)) > 8
    assert L.fp6mi_workspace_bytes(256, 8, 1) == 0 and L.fp6mi_workspace_bytes(256, 8, 3) == 3 * 256 * 8 * 4


def test_python_api_argument_errors():
    t = torch.zeros((256, 12), dtype=torch.int32)
    with pytest.raises(ValueError):
        fp6.weight_prepacking_cpu(torch.zeros((100, 12), dtype=torch.int32))      # OC % 256
    with pytest.raises(ValueError):
        fp6.weight_prepacking_cpu(torch.zeros((256, 13), dtype=torch.int32))      # width not a multiple of x
    with pytest.raises(ValueError):
        fp6.weight_prepacking_cpu(t.to(torch.int64))
    with pytest.raises(ValueError):
        fp6.weight_prepacking_eXmY_cpu(4, 3, t)
    with pytest.raises(ValueError):
        fp6.weight_dequant_cpu(t, torch.ones(100, dtype=torch.float16))
    with pytest.raises(ValueError):
        fp6.linear_forward_cuda(torch.zeros(1, 64, dtype=torch.float16), t, torch.ones(256, dtype=torch.float16), 1)  # not on GPU


def test_reference_heuristic_is_kept_verbatim():
    for args in [(4096, 8, 108), (11008, 8, 108), (8192, 512, 256), (256, 1, 108), (28672, 32, 108), (4096, 8, 256)]:
        assert fp6.HeuristicFuntion_SplitK(*args) == oracle.heuristic_splitk(*args)
        assert fp6.Num_Wave(args[0], args[1], 3, args[2]) == pytest.approx(oracle.num_wave(args[0], args[1], 3, args[2]))


def test_mi355x_heuristic_prefers_no_split_when_rows_fill_the_chip():
    for (M, N, K) in [(4096, 8, 4096), (11008, 8, 4096), (8192, 16, 8192), (28672, 8, 8192), (8192, 512, 8192)]:
        assert fp6.heuristic_splitk_mi355x(M, N, K) == 1
    # batches above 16 tile the rows in blocks of 64..256: K is cut to make up the missing parallelism, into 2, 3, 4, 6 or 8
    # pieces and never into more pieces than there are 256-column K blocks
    for (M, N, K) in [(8192, 32, 8192), (28672, 32, 8192), (8192, 64, 8192), (4096, 32, 11008), (10240, 32, 8192), (4096, 128, 512)]:
        s = fp6.heuristic_splitk_mi355x(M, N, K)
        assert s in (1, 2, 3, 4, 6, 8) and s <= (K + 255) // 256, (M, N, K, s)
    assert fp6.heuristic_splitk_mi355x(8192, 32, 8192) > 1          # 64 row blocks alone leave three quarters of the CUs idle
    s = fp6.heuristic_splitk_mi355x(256, 8, 28672)      # 16 row tiles cannot occupy 256 CUs: splitting K pays
    assert 2 <= s <= 64
    assert fp6.heuristic_splitk_mi355x(256, 1, 1024) == 1  # too little work to pay for a second launch


def test_rule_based_heuristic_for_other_cu_counts():
    """With a CU count that has no measured table the cost rules decide; known answers of those rules for a 304-CU part."""
    assert fp6.heuristic_splitk_mi355x(4096, 8, 4096, 304) == 1
    assert fp6.heuristic_splitk_mi355x(8192, 512, 8192, 304) == 1
    for (M, N, K) in [(8192, 32, 8192), (28672, 32, 8192), (8192, 64, 8192)]:
        s = fp6.heuristic_splitk_mi355x(M, N, K, 304)
        assert s in (1, 2, 4, 8)
    assert fp6.heuristic_splitk_mi355x(8192, 32, 8192, 304) >= fp6.heuristic_splitk_mi355x(28672, 32, 8192, 304)


def test_compiled_launch_shape_lists_match_the_kernel_source():
    from fp6_llm_amd import tune
    src = open(os.path.join(os.path.dirname(fp6.__file__), "csrc", "fp6mi_gemm.hip")).read()
    stream = {(0, int(a), int(b), 1, int(c)) for a, b, c in re.findall(r"FP6MI_CASE\((\d+), (\d+), (\d+)\)", src)}
    tile_src, ws_src = src.split("c.kind == 2")    # the wave-specialized shapes are listed after those of the tile kernel
    tile = {(1, int(a), int(b), int(c), int(d)) for a, b, c, d in re.findall(r"FP6MI_CASE\((\d+), (\d+), (\d+), (\d+)\)", tile_src)}
    ws = {(2, int(a), int(b), int(c), int(d)) for a, b, c, d in re.findall(r"FP6MI_CASE\((\d+), (\d+), (\d+), (\d+)\)", ws_src)}
    assert stream == set(tune.COMPILED_STREAM) and tile == set(tune.COMPILED_TILE) and ws == set(tune.COMPILED_WS)
    assert set(tune.STREAM_SMALL + tune.STREAM_WIDE) <= stream and set(tune.TILE) <= tile


def test_measured_table_holds_only_compiled_shapes_and_query_launch_follows_it():
    from fp6_llm_amd import tune
    compiled = set(tune.COMPILED_STREAM + tune.COMPILED_TILE + tune.COMPILED_WS)
    inc = open(tune.INC_PATH).read()
    entries = re.findall(r"^\{(\d+),(\d+),(\d+),(\d+),\{(.*)\}\},$", inc, flags=re.M)
    L = _lib.lib()
    shape = (ctypes.c_int * 5)()
    for xb, m256, k64, n, cells in entries:
        E, Mb = {6: (3, 2), 5: (2, 2), 4: (2, 1)}[int(xb)]
        OC, IC, BS = int(m256) * 256, int(k64) * 64, int(n)
        for i, cell in enumerate(re.findall(r"\{([\d,]+)\}", cells)):
            v = tuple(int(t) for t in cell.split(","))
            if v[0] == 255:
                continue
            assert v[:5] in compiled, (xb, OC, IC, BS, v)
            assert v[0] == 0 or OC % tune.tile_rows(v[:5]) == 0      # (the stream kernel's last workgroup holds what is left of the row tiles)
            assert L.fp6mi_query_launch(E, Mb, OC, BS, IC, tune.SPLITS[i], shape) == 0
            assert tuple(shape) == v[:5], (xb, OC, IC, BS, tune.SPLITS[i], tuple(shape), v)
    # any legal problem gets a compiled shape that divides its rows, measured neighbour or not
    for (OC, IC, BS, sk) in [(256, 64, 1, 1), (768, 1088, 3, 2), (4352, 4160, 8, 1), (9984, 3008, 40, 3), (65536, 16384, 700, 1), (512, 64, 17, 1)]:
        for (E, Mb) in FORMATS:
            assert L.fp6mi_query_launch(E, Mb, OC, BS, IC, sk, shape) == 0
            assert tuple(shape) in compiled and (shape[0] == 0 or OC % tune.tile_rows(tuple(shape)) == 0), (OC, IC, BS, sk, tuple(shape))
    assert L.fp6mi_query_launch(3, 2, 100, 1, 64, 1, shape) == -2 and L.fp6mi_query_launch(4, 3, 256, 1, 64, 1, shape) == -1


@pytest.mark.parametrize("E,M", FORMATS)
def test_quantizer(E, M):
    x = 1 + E + M
    mags = quant.magnitudes(E, M)
    assert (mags == np.abs(oracle.value_table(E, M)[: 1 << (x - 1)])).all()
    allc = np.arange(1 << x, dtype=np.uint8)
    vals = oracle.value_table(E, M)
    q = quant.quantize_codes(vals, E, M)
    assert (q == allc).all()                                       # exact values map to their own code (incl. -0)
    assert quant.quantize_codes(np.array([1e9, -1e9]), E, M).tolist() == [(1 << (x - 1)) - 1, (1 << x) - 1]  # clamp
    mid = (mags[:-1] + mags[1:]) / 2
    tie = quant.quantize_codes(mid, E, M)
    assert (tie % 2 == 0).all()                                    # ties go to the even code
    v = np.linspace(-mags[-1], mags[-1], 4001)
    assert (np.diff(vals[quant.quantize_codes(v, E, M)]) >= 0).all()  # monotone
    assert (np.abs(vals[quant.quantize_codes(v, E, M)] - v) <= np.diff(mags).max() / 2 + 1e-12).all()
    w = synth.normal(5, (64, 128))
    codes, scale = quant.quantize_rowwise(w, E, M)
    assert scale.dtype == np.float16 and codes.max() < (1 << x)
    deq = quant.dequantize_codes(codes, scale, E, M)
    assert np.abs(deq - w).max() <= np.abs(w).max() / mags[-1] * np.diff(mags).max() * 0.51
    raw = quant.pack_raw(codes, E, M)
    assert (quant.unpack_raw(raw, E, M) == codes).all() and (oracle.unpack_codes(raw, E, M) == codes).all()


def _awkward_weights(seed, OC, IC):
    """Gaussian weights with what a quantizer gets wrong: zero rows, a row whose scale is an fp16 subnormal, a huge row,
    negative zeros, exact ties of the scaled grid, and NaN / +-Inf entries."""
    w = synth.normal(seed, (OC, IC)).astype(np.float32)
    w[1, :] = 0.0
    w[2, :] *= 1e-7
    w[3, :] *= 3000.0
    w[4, ::3] = -0.0
    w[5, :] = 0.0
    w[5, 0] = 28.0
    w[5, 1:65] = np.arange(64, dtype=np.float32) * 0.4375
    w[6, :] = -w[5, :]
    w[7, 3] = np.nan
    w[7, 4] = np.inf
    w[7, 5] = -np.inf
    return w


@pytest.mark.parametrize("E,M", FORMATS)
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_host_quantizer_equals_the_exact_definition(E, M, dtype):
    """quant.quantize_rowwise / quantize_groupwise (float64 quotients, searchsorted) against the oracle's definition in exact
    arithmetic: same scales, same codes, same group exponents."""
    with np.errstate(over="ignore"):
        w = _awkward_weights(61, 64, 320).astype(dtype)
    codes, sc = quant.quantize_rowwise(w, E, M)
    c0, s0 = oracle.quantize_from_definition(w, E, M)
    assert np.array_equal(sc.view(np.uint16), s0.view(np.uint16)) and np.array_equal(codes, c0)
    spread = np.exp(np.random.default_rng(5).normal(0, 2.0, (64, 3))).repeat(128, axis=1)[:, :320]
    spread[:8] = 1.0
    with np.errstate(over="ignore", invalid="ignore"):
        wg = (w.astype(np.float64) * spread).astype(dtype)
    codes, sc, ex = quant.quantize_groupwise(wg, E, M)
    c0, s0, e0 = oracle.quantize_grouped_from_definition(wg, E, M)
    assert np.array_equal(sc.view(np.uint16), s0.view(np.uint16)) and np.array_equal(ex, e0) and np.array_equal(codes, c0)


def test_native_weight_file_round_trip(tmp_path):
    from fp6_llm_amd import module
    raw, sc = _problem(21, 256, 320, 2, 2)
    nat = fp6.weight_prepacking_native_cpu(2, 2, torch.from_numpy(raw))
    path = str(tmp_path / "w.fp6mi")
    module.save_native(path, nat, torch.from_numpy(sc), 2, 2, 256, 320)
    nat2, sc2, hdr = module.load_native(path)
    assert torch.equal(nat, nat2) and (sc2.numpy() == sc).all() and hdr["in_features"] == 320 and hdr["exponent"] == 2
    with open(path, "r+b") as f:
        f.truncate(4000)
    with pytest.raises(ValueError):
        module.load_native(path)
    with open(path, "wb") as f:
        f.write(b"not a weight file")
    with pytest.raises(ValueError):
        module.load_native(path)


# ------------------------------------------------------------------------------------------------ per-group exponents
def _grouped_problem(seed, OC, IC, E, M):
    """Gaussian weights whose groups of 128 columns differ in magnitude by powers of e, so that the exponents vary."""
    rng = np.random.default_rng(seed)
    spread = np.exp(rng.normal(0, 1.5, (OC, (IC + 127) // 128))).repeat(128, axis=1)[:, :IC]
    return synth.normal(seed, (OC, IC)) * spread


@pytest.mark.parametrize("E,M", FORMATS)
def test_groupwise_quantizer(E, M):
    OC, IC = 64, 320   # the last group has 64 columns
    w = _grouped_problem(31, OC, IC, E, M)
    codes, sc, ex = quant.quantize_groupwise(w, E, M)
    top = quant.max_value(E, M)
    assert ex.dtype == np.uint8 and ex.shape == (OC, 3) and ex.min() >= 112 and ex.max() == 127 and len(np.unique(ex)) > 3
    _, sc_row = quant.quantize_rowwise(w, E, M)
    assert (sc == sc_row).all()                                  # the row scale is the row-wise one
    for g in range(3):
        blockmax = np.abs(w[:, 128 * g:128 * g + 128]).max(axis=1) / sc.astype(np.float64)
        f = np.exp2(ex[:, g].astype(np.float64) - 127)
        # the group fits under its factor (the row's largest group only up to the rounding of the fp16 row scale, like row-wise) ...
        assert ((blockmax <= top * f) | ((ex[:, g] == 127) & (blockmax <= top * (1 + 2.0 ** -10)))).all()
        assert ((blockmax > top * f / 2) | (ex[:, g] == 112)).all()   # ... and would not fit under half of it
    deq = quant.dequantize_grouped(codes, sc, ex, E, M)
    rw_codes, _ = quant.quantize_rowwise(w, E, M)
    assert np.abs(deq - w).mean() < np.abs(quant.dequantize_codes(rw_codes, sc, E, M) - w).mean()
    # weights without spread between groups of a row's own maximum group keep factor 1 there
    assert (ex.max(axis=1) == 127).all()
    # a zero matrix: scale 1, any exponent, all codes zero magnitude
    c0, s0, e0 = quant.quantize_groupwise(np.zeros((16, 128)), E, M)
    assert (s0 == 1).all() and (c0 & ((1 << (E + M)) - 1) == 0).all() and e0.shape == (16, 1)


@pytest.mark.parametrize("E,M", FORMATS)
def test_grouped_dequant_and_exponent_packing(E, M):
    OC, IC = 64, 320
    codes, sc, ex = quant.quantize_groupwise(_grouped_problem(32, OC, IC, E, M), E, M)
    raw = torch.from_numpy(quant.pack_raw(codes, E, M))
    dq = fp6.weight_dequant_grouped_cpu(E, M, raw, torch.from_numpy(sc), torch.from_numpy(ex)).numpy()
    assert (dq.view(np.uint16) == oracle.dequant_grouped_from_definition(codes, sc, ex, E, M).view(np.uint16)).all()
    ones = torch.full((OC, 3), 127, dtype=torch.uint8)               # factor 1 everywhere = the reference's dequantizer
    assert torch.equal(fp6.weight_dequant_grouped_cpu(E, M, raw, torch.from_numpy(sc), ones),
                       fp6.weight_dequant_eXmY_cpu(E, M, raw, torch.from_numpy(sc)))
    # packed order, from its definition: [row tile][K block][row in tile][half]; halves beyond IC hold 127
    nat = fp6.pack_group_exps(torch.from_numpy(ex), OC, IC).numpy()
    assert nat.size == fp6.group_exps_bytes(OC, IC) == (OC // 16) * 2 * 32
    for (R, U, m, h) in [(0, 0, 0, 0), (3, 0, 15, 1), (2, 1, 7, 0), (1, 1, 9, 1)]:
        want = ex[16 * R + m, 2 * U + h] if 2 * U + h < 3 else 127
        assert nat[((R * 2 + U) * 16 + m) * 2 + h] == want
    with pytest.raises(ValueError):
        fp6.pack_group_exps(torch.from_numpy(ex[:, :2].copy()), OC, IC)


def test_grouped_weight_file_and_fused_layers(tmp_path):
    from fp6_llm_amd import module
    E, M = 2, 1
    ws = [torch.from_numpy(_grouped_problem(40 + i, oc, 384, E, M)).float() for i, oc in enumerate((256, 512))]
    parts = [module.FPxLinear.from_float(w, E, M, group_scales=True) for w in ws]
    whole = module.FPxLinear.from_float(torch.cat(ws), E, M, group_scales=True)
    fused = module.FPxLinear.fused(parts)
    assert fused.group_exps is not None and torch.equal(fused.group_exps, whole.group_exps)
    assert torch.equal(fused.weight_native, whole.weight_native) and torch.equal(fused.scales, whole.scales)
    with pytest.raises(ValueError):
        module.FPxLinear.fused([parts[0], module.FPxLinear.from_float(ws[1], E, M)])
    # a layer built empty with group_scales=True takes the state of a quantized one
    blank = module.FPxLinear(384, 768, E, M, group_scales=True)
    assert (blank.group_exps == 127).all()
    blank.load_state_dict(whole.state_dict())
    assert torch.equal(blank.group_exps, whole.group_exps) and torch.equal(blank.weight_native, whole.weight_native)
    assert "group_exps" not in module.FPxLinear(384, 768, E, M).state_dict()
    path = str(tmp_path / "g.fp6mi")
    module.save_native(path, whole.weight_native, whole.scales, E, M, 768, 384, whole.group_exps)
    nat2, sc2, hdr = module.load_native(path)
    assert torch.equal(nat2, whole.weight_native) and torch.equal(sc2, whole.scales) and torch.equal(hdr["group_exps"], whole.group_exps)
    module.save_native(path, whole.weight_native, whole.scales, E, M, 768, 384)
    assert "group_exps" not in module.load_native(path)[2]


def test_module_construction_routes_agree():
    from fp6_llm_amd import module
    raw, sc = _problem(22, 256, 128, 3, 2)
    t, s = torch.from_numpy(raw), torch.from_numpy(sc)
    a = module.FPxLinear.from_raw(t, s)
    b = module.FPxLinear.from_prepacked(fp6.weight_prepacking_cpu(t), s)
    assert torch.equal(a.weight_native, b.weight_native) and torch.equal(a.scales, b.scales)
    w = torch.from_numpy(synth.normal(3, (256, 128))).float()
    c = module.FPxLinear.from_float(w)
    codes, scales = quant.quantize_rowwise(w.numpy(), 3, 2)
    assert torch.equal(c.weight_native, fp6.weight_prepacking_native_cpu(3, 2, torch.from_numpy(quant.pack_raw(codes, 3, 2))))
    with pytest.raises(ValueError):
        module.FPxLinear(100, 256)


def test_split_heuristic_per_format():
    L = _lib.lib()
    for (M, N, K) in [(4096, 8, 4096), (8192, 32, 8192), (256, 8, 28672), (17920, 32, 6656), (1024, 300, 2048)]:
        assert L.fp6mi_heuristic_splitk_format(3, 2, M, N, K, 256) == L.fp6mi_heuristic_splitk(M, N, K, 256)
        assert L.fp6mi_heuristic_splitk_format(2, 3, M, N, K, 256) == L.fp6mi_heuristic_splitk(M, N, K, 256)   # same bytes, same table
        for (E, Mb) in FORMATS:
            s = fp6.heuristic_splitk_mi355x(M, N, K, EXPONENT=E, MANTISSA=Mb)
            assert 1 <= s <= 64 and s <= (K + 255) // 256


def test_fused_layers_are_the_concatenation():
    """Fusing layers over one input = quantizing the row-concatenated weight: native tiles are stored row tile after row tile."""
    from fp6_llm_amd import module
    for (E, M) in FORMATS:
        ws = [torch.from_numpy(synth.normal(61 + i, (oc, 320))).float() for i, oc in enumerate((256, 512, 256))]
        bs = [torch.from_numpy(synth.normal(71 + i, (w.shape[0],))).half() for i, w in enumerate(ws)]
        parts = [module.FPxLinear.from_float(w, E, M, bias=b) for w, b in zip(ws, bs)]
        fused = module.FPxLinear.fused(parts)
        whole = module.FPxLinear.from_float(torch.cat(ws), E, M, bias=torch.cat(bs))
        assert fused.out_features == 1024 and fused.in_features == 320
        assert torch.equal(fused.weight_native, whole.weight_native)
        assert torch.equal(fused.scales, whole.scales) and torch.equal(fused.bias, whole.bias)
    with pytest.raises(ValueError):
        module.FPxLinear.fused([module.FPxLinear.from_float(ws[0], 3, 2), module.FPxLinear.from_float(ws[0], 2, 2)])


def test_e2m2_code_read_as_e3m2_is_a_quarter_of_its_value():
    """What the FP5 native layout relies on: inserting a zero above the two exponent bits of an e2m2 code gives the e3m2
    code of exactly a quarter of its value, for all 32 codes (subnormals and signed zeros included)."""
    v5, v6 = oracle.value_table(2, 2), oracle.value_table(3, 2)
    for code in range(32):
        field = (code & 15) | ((code >> 4) << 5)
        assert v6[field] * 4.0 == v5[code] and np.signbit(v6[field]) == np.signbit(v5[code])


def test_e2m1_code_with_two_zeros_appended_is_the_e2m3_code_of_its_value():
    """What the FP4 native layout relies on: an e2m1 code shifted left by two bits is the e2m3 code of the same value, for all
    16 codes (the subnormal and the signed zeros included)."""
    v4, v6 = oracle.value_table(2, 1), oracle.value_table(2, 3)
    for code in range(16):
        assert v6[code << 2] == v4[code] and np.signbit(v6[code << 2]) == np.signbit(v4[code])


def test_bench_refuses_more_than_one_gpu_and_lists_the_benchmark_configurations():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0 and "ONE GPU" in res.stderr
    sys.path.insert(0, root)
    import bench
    assert bench.WORKLOADS[bench.HEADLINE] == (3, 2, 4096, 4096, 8)
    # every shape of the five benchmark configurations is a workload: 4096^2 at 1/8/16, the two 7B MLP shapes at 8/32, the three
    # 70B shapes at 32, and 8192^2 at ten batch sizes in both formats
    assert len([w for w in bench.WORKLOADS if w.startswith(("fp6_", "fp5_"))]) == 3 + 4 + 3 + 20
    assert bench.weight_bytes(3, 2, 4096, 4096) == 12582912 and bench.algorithmic_bytes(3, 2, 4096, 4096, 8) == 12722176


def test_tuner_candidates_and_table_emission(tmp_path, monkeypatch):
    from fp6_llm_amd import tune
    compiled = set(tune.COMPILED_STREAM + tune.COMPILED_TILE + tune.COMPILED_WS)
    for (OC, IC, BS) in [(256, 64, 1), (4096, 4096, 8), (4096, 4096, 17), (11008, 4096, 64), (768, 2048, 512), (8192, 8192, 2048)]:
        cands = list(tune.candidates(OC, IC, BS))
        assert cands, (OC, IC, BS)
        for cfg, sk in cands:
            ragged = cfg[0] == 0                       # the stream kernel's last workgroup holds what is left of the row tiles
            assert cfg in compiled and (ragged or OC % tune.tile_rows(cfg) == 0) and 1 <= sk <= (IC + 255) // 256
            assert cfg[0] != 0 or BS <= 64 or (BS <= 128 and OC <= 2560)     # the stream kernel is a candidate up to four column blocks, eight on short matrices
            assert cfg[0] == 0 or BS > 16
    src = tmp_path / "t.jsonl"
    src.write_text(json.dumps({"E": 3, "M": 2, "OC": 512, "IC": 1024, "BS": 8, "best": {"1": [[0, 1, 1, 1, 8], 3.21], "4": [[0, 1, 2, 1, 4], 4.0]}}) + "\n")
    monkeypatch.setattr(tune, "INC_PATH", str(tmp_path / "out.inc"))
    tune.main(["emit", str(src)])
    lines = [l for l in (tmp_path / "out.inc").read_text().splitlines() if l.startswith("{")]
    assert lines == ["{6,2,16,8,{{0,1,1,1,8,160},{255,0,0,0,0,0},{255,0,0,0,0,0},{0,1,2,1,4,200},{255,0,0,0,0,0},{255,0,0,0,0,0}}},"]


# ------------------------------------------------------------------------------------------------ randomized round trips
def test_packers_round_trip_on_random_shapes_and_bits():
    """Property check with hypothesis: for any supported format, any legal shape and any bit pattern, the reference layout and
    the native layout both unpack to the raw tensor they were packed from, both routes to the native layout agree, and the
    host prepacker equals the oracle's."""
    from hypothesis import given, settings, strategies as st

    @settings(max_examples=40, deadline=None)
    @given(fmt=st.sampled_from(FORMATS), tiles=st.integers(1, 3), kblocks=st.integers(1, 9), seed=st.integers(0, 2 ** 31 - 1))
    def check(fmt, tiles, kblocks, seed):
        E, M = fmt
        x = 1 + E + M
        OC, IC = 64 * tiles, 64 * kblocks
        raw = np.random.default_rng(seed).integers(0, 2 ** 32, size=(OC, IC // 32 * x), dtype=np.uint64).astype(np.uint32).view(np.int32)
        L = _lib.lib()
        packed, back = np.empty_like(raw), np.empty_like(raw)
        assert L.fp6mi_prepack_ref(E, M, packed.ctypes.data, raw.ctypes.data, OC, IC) == 0
        assert packed.tobytes() == oracle.prepack(raw, E, M).tobytes()
        assert L.fp6mi_unpack_ref(E, M, back.ctypes.data, packed.ctypes.data, OC, IC) == 0 and (back == raw).all()
        nat = np.empty(fp6.native_bytes(E, M, OC, IC), np.uint8)
        nat2 = np.empty_like(nat)
        assert L.fp6mi_prepack_native(E, M, nat.ctypes.data, raw.ctypes.data, OC, IC) == 0
        assert L.fp6mi_relayout_ref_to_native(E, M, nat2.ctypes.data, packed.ctypes.data, OC, IC) == 0 and (nat == nat2).all()
        back[:] = 0
        assert L.fp6mi_unpack_native(E, M, back.ctypes.data, nat.ctypes.data, OC, IC) == 0 and (back == raw).all()

    check()



def test_host_code_and_oracle_are_clean_under_asan_and_ubsan():
    """Builds tests/sanitize (the engine's CPU functions + the oracle with AddressSanitizer and UBSan, ROCm's clang) and runs its
    driver over every format, cut K blocks, in-place packing and the grouped dequantizer."""
    import shutil
    import subprocess
    d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sanitize")
    if not os.path.exists("/opt/rocm/llvm/bin/clang++") or not shutil.which("make") or not os.path.isdir(d):
        pytest.skip("needs ROCm's clang and make")
    res = subprocess.run(["make", "-C", d, "-B", "run"], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0 and "clean under ASan + UBSan" in res.stdout, res.stdout[-2000:] + res.stderr[-2000:]


def test_the_reference_package_name_imports_the_same_functions():
    """`import fp6_llm` (the reference's package name, fp6_llm/__init__.py:1) gives the engine's functions under the reference's names."""
    import fp6_llm
    for name in ["linear_forward_cuda", "weight_prepacking_cpu", "weight_dequant_cpu", "linear_forward_eXmY_cuda", "weight_prepacking_eXmY_cpu",
                 "weight_dequant_eXmY_cpu", "Num_Wave", "HeuristicFuntion_SplitK"]:
        assert getattr(fp6_llm, name) is getattr(fp6, name)


def test_launch_source_tells_measured_from_carried_over_from_rules():
    L = _lib.lib()
    assert L.fp6mi_launch_source(3, 2, 4096, 8, 4096, 1) == 0          # in the table
    assert L.fp6mi_launch_source(3, 2, 4096, 7, 4096, 1) == 0          # the next larger measured batch of a measured matrix
    assert L.fp6mi_launch_source(3, 2, 4352, 8, 4160, 1) == 1          # neighbours within a factor 1.5
    assert L.fp6mi_launch_source(3, 2, 256, 8, 64, 1) == 2               # far from every measured problem
    assert L.fp6mi_launch_source(3, 2, 4096, 8, 4096, 5) == 2          # a split the table does not hold
    assert L.fp6mi_launch_source(4, 3, 4096, 8, 4096, 1) == -1 and L.fp6mi_launch_source(3, 2, 100, 8, 4096, 1) == -2
    assert b"library version" in L.fp6mi_tuning_info()


def test_cpp_torch_entry_points_carry_the_reference_names():
    """The torch extension defines the reference's six C++ functions (fp6_llm/csrc/fp6_linear.cuh:50-90) and binds them under the
    reference's Python names (fp6_llm/csrc/pybind.cpp:8-15); the CPU ones must give the oracle's bytes."""
    ext = pytest.importorskip("fp6_llm_amd._fp6mi_torch")
    for name in ("linear_forward_cuda", "weight_prepacking_cpu", "weight_dequant_cpu", "linear_forward_eXmY_cuda", "weight_prepacking_eXmY_cpu",
                 "weight_dequant_eXmY_cpu"):
        assert callable(getattr(ext, name))
    header = open(os.path.join(os.path.dirname(fp6.__file__), "csrc", "fp6_linear_torch.h")).read()
    for name in ("fp6_linear_forward_cuda", "fp_eXmY_linear_forward_cuda", "weight_matrix_prepacking_cpu", "weight_matrix_prepacking_fp_eXmY_cpu",
                 "weight_matrix_dequant_cpu", "weight_matrix_dequant_fp_eXmY_cpu"):
        assert name in header
    for (E, M) in FORMATS:
        raw, sc, _ = synth.uniform_problem(70 + E + M, 256, 320, 1, E, M)
        packed = ext.weight_prepacking_eXmY_cpu(E, M, torch.from_numpy(raw))
        assert packed.numpy().tobytes() == oracle.prepack(raw, E, M).tobytes()
        deq = ext.weight_dequant_eXmY_cpu(E, M, torch.from_numpy(raw), torch.from_numpy(sc))
        assert (deq.numpy().view(np.uint16) == oracle.dequant(raw, sc, E, M).view(np.uint16)).all()
    raw, sc, _ = synth.uniform_problem(71, 256, 320, 1, 3, 2)
    assert torch.equal(ext.weight_prepacking_cpu(torch.from_numpy(raw)), fp6.weight_prepacking_cpu(torch.from_numpy(raw)))
    assert torch.equal(ext.weight_dequant_cpu(torch.from_numpy(raw), torch.from_numpy(sc)), fp6.weight_dequant_cpu(torch.from_numpy(raw), torch.from_numpy(sc)))
    with pytest.raises(ValueError):
        ext.weight_prepacking_cpu(torch.zeros((100, 12), dtype=torch.int32))           # OC % 256 (the reference asserts)
    with pytest.raises(ValueError):
        ext.weight_prepacking_eXmY_cpu(4, 3, torch.zeros((256, 16), dtype=torch.int32))  # a format nobody has
    with pytest.raises(ValueError):
        ext.weight_dequant_cpu(torch.zeros((256, 12), dtype=torch.int32), torch.zeros(255, dtype=torch.float16))
