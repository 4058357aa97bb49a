"""Launch-shape tuner of the FPx x FP16 GEMM.

The engine chooses, per (format, M, N, K, splitK), one of its compiled kernel shapes.  A rule derived from first principles
covers any shape; for the shapes of real models a measured table does better, the way BLAS libraries ship solution tables.
This tool measures every candidate shape on the GPU it runs on and writes that table:

    python -m fp6_llm_amd.tune sweep --format 6 --out fp6_llm_amd/tuning/fp6_mi355x.jsonl      # minutes of GPU time
    python -m fp6_llm_amd.tune compact fp6_llm_amd/tuning/*.jsonl                               # after re-measuring with --append
    python -m fp6_llm_amd.tune sweep --format 6 --kinds stream --n 8,12,16 --out part.jsonl     # after a change to one kernel:
    python -m fp6_llm_amd.tune merge fp6_llm_amd/tuning/fp6_mi355x.jsonl part.jsonl             #   only its candidates are re-measured
    python -m fp6_llm_amd.tune emit fp6_llm_amd/tuning/*.jsonl                                  # -> csrc/fp6mi_tuning.inc
    python -m fp6_llm_amd.build

Timing protocol: weights rotate through a pool of distinct buffers larger than the last-level cache, `iters` launches are
captured into one HIP graph, a replay is timed with events `reps` times and the MEDIAN counts (some shapes with many small
workgroups have a lucky fast mode now and then; a best-of would favour them, and the benchmark sees their typical time).
"""
import argparse
import glob
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
INC_PATH = os.path.join(HERE, "csrc", "fp6mi_tuning.inc")

# (kind, n_tiles, row_tiles, row_waves, k_waves); kind 0 = stream kernel (batch <= 16 per n_tile), 1 = tile kernel, 2 = wave-specialized tile kernel
STREAM_SMALL = [(0, 1, rt, 1, wk) for rt in (1, 2, 3, 4, 5, 6, 7, 8) for wk in (4, 8, 16) if wk == 4 or (wk == 8 and rt <= 6) or rt <= 2]
STREAM_WIDE = [(0, 2, 1, 1, 8), (0, 2, 2, 1, 4), (0, 2, 3, 1, 4), (0, 2, 3, 1, 8), (0, 2, 4, 1, 4), (0, 2, 4, 1, 8), (0, 2, 5, 1, 4), (0, 2, 5, 1, 8),
               (0, 2, 6, 1, 4), (0, 2, 7, 1, 4), (0, 2, 8, 1, 4)]   # two 16-column tiles per workgroup, batches 17..32
TILE = [(1, 2, 1, 4, 4), (1, 2, 1, 2, 4), (1, 2, 2, 4, 1), (1, 2, 2, 4, 2), (1, 4, 1, 4, 2), (1, 4, 1, 8, 2), (1, 4, 2, 4, 2), (1, 4, 2, 8, 1),
        (1, 8, 2, 8, 1)]
SPLITS = (1, 2, 3, 4, 6, 8)      # 3 and 6 fill 256 CUs where 80 or 40 row blocks leave a power of two short (M = 10240, 5120)
FORMAT_OF_BITS = {6: (3, 2), 5: (2, 2), 4: (2, 1)}   # the table is keyed by bit width

# every shape compiled into the library (FP6MI_CASE tables of csrc/fp6mi_gemm.hip, the same for every format); the candidates above are the ones that
# ever came within 3 % of the best in exhaustive sweeps
COMPILED_STREAM = [(0, nt, rt, 1, wk) for (nt, rt, wk) in
                   [(1, 1, 4), (1, 1, 8), (1, 1, 16), (1, 2, 4), (1, 2, 8), (1, 2, 16), (1, 3, 4), (1, 3, 8), (1, 4, 4), (1, 4, 8), (1, 5, 4),
                    (1, 5, 8), (1, 6, 4), (1, 6, 8), (1, 7, 4), (1, 8, 4), (2, 1, 4), (2, 1, 8), (2, 2, 4), (2, 2, 8), (2, 3, 4), (2, 3, 8),
                    (2, 4, 4), (2, 4, 8), (2, 5, 4), (2, 5, 8), (2, 6, 4), (2, 7, 4), (2, 8, 4)]]
COMPILED_TILE = [(1,) + c for c in
                 [(2, 1, 4, 4), (2, 2, 4, 4), (2, 2, 4, 2), (2, 2, 4, 1), (2, 4, 4, 1), (2, 4, 4, 2), (4, 2, 4, 2), (4, 2, 4, 1), (4, 4, 4, 1),
                  (4, 4, 2, 1), (4, 4, 2, 2), (8, 2, 4, 1), (8, 2, 2, 1), (4, 2, 8, 1), (4, 2, 8, 2), (2, 2, 8, 1), (2, 2, 8, 2), (8, 2, 8, 1),
                  (4, 1, 8, 2), (4, 1, 8, 1), (4, 1, 4, 2), (2, 1, 2, 4)]]

# kind 2 = wave-specialized tile kernel: (2, n_tiles, row_tiles, arithmetic wavefronts, loading wavefronts)
COMPILED_WS = [(2, 4, 2, 8, 4), (2, 4, 2, 4, 4), (2, 2, 2, 8, 4)]

BLOCK_BYTES = {6: 3072, 5: 2560, 4: 2048}   # one native 16-row x 256-column block per bit width


def shape_compiled_for(cfg, bits):
    """Every stream and tile shape exists for every format; a wave-specialized shape needs its weight stage to be a whole number
    of 1 KB transfers per loading wavefront (FP5 blocks are 2.5 KB, so its 64-row tiles are out)."""
    kind, nt, rt, wr, wk = cfg
    return kind < 2 or (wr * rt * BLOCK_BYTES[bits]) % (1024 * wk) == 0


GRID_M = [1024, 2048, 3072, 4096, 5120, 6144, 8192, 10240, 11008, 12288, 14336, 16384, 22016, 28672, 32768]
GRID_K = [2048, 4096, 5120, 8192, 11008, 14336, 28672]
GRID_N_SMALL = [1, 4, 8, 12, 16]
GRID_N_LARGE = [24, 32, 48, 64, 96, 128, 256, 512, 1024, 2048]
MAX_WEIGHTS = 240 * 1000 * 1000   # the grid skips matrices beyond the largest layer of a 70B model (28672 x 8192)
# Layer shapes (OC, IC) of common decoder models that the grid does not hit: hidden/MLP sizes 2560, 3072, 3584, 5120, 6656,
# 7168 with their fused QKV and gate+up projections (13B/14B/30B/32B LLaMA- and Qwen-shaped models, 7B Qwen2, Gemma, Phi-3,
# OPT-30B).  Swept with `--pairs models`; off the grid the carry-over from neighbours costs 2 % on average, 15 % at worst.
MODEL_PAIRS = [(15360, 5120), (13824, 5120), (27648, 5120), (5120, 13824), (7168, 5120), (5120, 27648),
               (6656, 6656), (19968, 6656), (17920, 6656), (35840, 6656), (6656, 17920),
               (8192, 22016), (24576, 8192),
               (3584, 3584), (4608, 3584), (18944, 3584), (37888, 3584), (3584, 18944),
               (3072, 3072), (9216, 3072), (16384, 3072), (24576, 3072), (49152, 3072), (3072, 24576),
               (2048, 16384), (2560, 2560), (7680, 2560), (2560, 9728), (9728, 2560), (19456, 2560),
               (7168, 7168), (21504, 7168), (28672, 7168), (7168, 28672),
               # the remaining shapes of the reference's run scripts (tests/python/run.sh:33-34, tests/cpp/run.sh:14-15): LLaMA-2-70B's fused
               # gate+up projection and the OPT-66B / OPT-175B layers
               (57344, 8192), (27648, 9216), (9216, 9216), (36864, 9216), (9216, 36864), (36864, 12288), (12288, 12288), (49152, 12288),
               (12288, 49152)]


def tile_rows(cfg):
    kind, nt, rt, wr, wk = cfg
    return 16 * rt * (wr if kind >= 1 else 1)


KIND_NAMES = ("stream", "tile", "ws")


def candidates(OC, IC, BS, kinds=None, splits=None, bits=6, shapes=None):
    """(shape, splitK) pairs worth measuring; `kinds` ("stream", "tile", "ws"), `splits` and `shapes` (a set of shape tuples)
    narrow the list for a partial sweep."""
    for cfg, sk in _all_candidates(OC, IC, BS, bits):
        if kinds and KIND_NAMES[cfg[0]] not in kinds:
            continue
        if shapes and tuple(cfg) not in shapes:
            continue
        if splits and sk not in splits:
            continue
        yield cfg, sk


def _all_candidates(OC, IC, BS, bits=6):
    if BS <= 16:
        cfgs = STREAM_SMALL
    else:
        cfgs = [c for c in TILE if (c[1] * 16 < 2 * BS + 16 or c[1] == 2) and (BS <= 512 or c[1] >= 4)]
        if BS <= 64:    # the stream kernel over several column blocks (each re-reads the weights, out of L2): wins on small M, where
            cfgs = cfgs + STREAM_WIDE + STREAM_SMALL   # a tile kernel would have to split K to fill the chip (4096 x 4096 batch 24-64)
        elif BS <= 128 and OC <= 2560:   # the same for matrices of so few rows that even at batch 128 no tile shape fills the chip
            cfgs = cfgs + STREAM_WIDE + STREAM_SMALL
        if BS >= 96:    # the wave-specialized tiles pay from about 128 columns up (256 x 64 from 256 up on 8192 x 8192)
            cfgs = cfgs + [c for c in COMPILED_WS if c[1] * 16 <= BS]
    units = (IC + 255) // 256
    for cfg in cfgs:
        if OC % tile_rows(cfg) and cfg[0] != 0:   # (the stream kernel takes any number of row tiles per workgroup: the last one holds the rest)
            continue
        for sk in SPLITS:
            if sk > units or (cfg[0] == 0 and sk > 1 and OC > 4096):   # the stream kernel splits K inside the workgroup already
                continue
            if sk > 1 and (sk * 8 * BS > IC * 0.75 or BS > 512):   # the FP32 partial sums would outweigh the weights themselves
                continue
            yield cfg, sk


class Bench:
    """Times one launch shape on one problem; keeps the weight pool of the current (format, OC, IC) alive between calls."""

    def __init__(self, iters=30, reps=5, pool_bytes=1 << 30):
        import torch

        from . import _lib
        self.torch, self.L = torch, _lib.lib()
        self.iters, self.reps, self.pool_bytes = iters, reps, pool_bytes
        self.dev = torch.device("cuda:0")
        self.key = None
        self.lib_version, self.rocm = int(self.L.fp6mi_version()), str(torch.version.hip)   # stamped on every row measured

    def _pool(self, E, M, OC, IC):
        torch = self.torch
        from . import native_bytes
        if self.key != (E, M, OC, IC):
            self.bufs = None
            torch.cuda.empty_cache()
            nb = native_bytes(E, M, OC, IC)
            nbuf = max(2, min(48, self.pool_bytes // nb))
            w0 = torch.randint(-2 ** 31, 2 ** 31 - 1, (nb // 4,), dtype=torch.int32)   # every bit pattern is a valid weight
            self.bufs = [torch.roll(w0, 17 * i).to(self.dev) for i in range(nbuf)]
            self.scales = (torch.rand(OC) * 0.009 + 0.001).half().to(self.dev)
            self.key = (E, M, OC, IC)
        return self.bufs, self.scales

    def __call__(self, E, M, OC, IC, BS, cfg, sk):
        torch = self.torch
        bufs, scales = self._pool(E, M, OC, IC)
        x = torch.randn(BS, IC).half().to(self.dev)
        out = torch.empty(BS, OC, dtype=torch.float16, device=self.dev)
        ws = torch.empty(sk * BS * OC, dtype=torch.float32, device=self.dev) if sk > 1 else None

        def launch(i):
            st = torch.cuda.current_stream().cuda_stream
            return self.L.fp6mi_linear_native_cfg(E, M, st, bufs[i % len(bufs)].data_ptr(), scales.data_ptr(), x.data_ptr(), out.data_ptr(),
                                                  OC, BS, IC, ws.data_ptr() if ws is not None else None, sk, *cfg)
        times = []
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            if launch(0) != 0:
                return None
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(self.iters):
                    launch(i)
            # replays until about 8 ms have passed before any is timed: right after the idle spell of a capture the clocks are low,
            # which costs a long kernel more than a short one
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            for _ in range(int(min(200, 8.0 / max(e0.elapsed_time(e1), 1e-3)))):
                graph.replay()
            torch.cuda.synchronize()
            for _ in range(self.reps):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                graph.replay()
                e1.record()
                torch.cuda.synchronize()
                times.append(e0.elapsed_time(e1) * 1e3 / self.iters)
        return sorted(times)[len(times) // 2]


def sweep(args):
    E, M = FORMAT_OF_BITS[args.format]
    Ms = [int(v) for v in args.m.split(",")] if args.m else GRID_M
    Ks = [int(v) for v in args.k.split(",")] if args.k else GRID_K
    Ns = [int(v) for v in args.n.split(",")] if args.n else GRID_N_SMALL + GRID_N_LARGE
    if args.pairs == "models":
        problems = MODEL_PAIRS
    elif args.pairs:
        problems = [tuple(int(v) for v in p.split("x")) for p in args.pairs.split(",")]
    else:
        problems = [(OC, IC) for OC in Ms for IC in Ks]
    kinds = set(args.kinds.split(",")) if args.kinds else None
    splits = set(int(v) for v in args.splits.split(",")) if args.splits else None
    shapes = set(tuple(int(v) for v in sh.split(".")) for sh in args.shapes.split(",")) if args.shapes else None
    bench = Bench(args.iters, args.reps)
    os.makedirs(os.path.dirname(os.path.abspath(args.out)), exist_ok=True)
    with open(args.out, "a" if args.append else "w") as f:
        for (OC, IC) in problems:
            if True:
                if OC * IC > MAX_WEIGHTS and not args.pairs:
                    continue
                for BS in Ns:
                    best = {}
                    for cfg, sk in candidates(OC, IC, BS, kinds, splits, args.format, shapes):
                        t = bench(E, M, OC, IC, BS, cfg, sk)
                        if t is not None and (str(sk) not in best or t < best[str(sk)][1]):
                            best[str(sk)] = [list(cfg), round(t, 3)]
                    row = {"E": E, "M": M, "OC": OC, "IC": IC, "BS": BS, "best": best, "lib": bench.lib_version, "rocm": bench.rocm}
                    if shapes:            # new shapes only: nothing measured before is out of date, `merge` keeps the faster entry
                        if not best:
                            continue
                        row["partial"] = {"kinds": [], "splits": []}
                    elif kinds or splits:   # a partial row: `merge` folds it into a full one
                        row["partial"] = {"kinds": sorted(kinds) if kinds else list(KIND_NAMES), "splits": sorted(splits) if splits else list(SPLITS)}
                    f.write(json.dumps(row) + "\n")
                    f.flush()
                    print("e%dm%d %dx%d N=%d: " % (E, M, OC, IC, BS) + "  ".join("sk%s %s %.2f" % (k, "".join(map(str, v[0])), v[1]) for k, v in best.items()),
                          flush=True)


def emit(args):
    rows = {}
    for path in sorted(p for pat in args.files for p in glob.glob(pat)):
        for line in open(path):
            r = json.loads(line)
            rows[(1 + r["E"] + r["M"], r["BS"], r["OC"], r["IC"])] = r   # later files override earlier ones
    stamps = {}
    for r in rows.values():
        key = "library version %s, ROCm %s" % (r["lib"], r["rocm"]) if "lib" in r else "unstamped (before rows carried a stamp)"
        stamps[key] = stamps.get(key, 0) + 1
    stamp_text = "; ".join("%d rows: %s" % (n, k) for k, n in sorted(stamps.items()))
    lines = ["// Measured launch shapes: generated by `python -m fp6_llm_amd.tune emit`; do not edit by hand.",
             "// Measured on one MI355X (256 CUs). " + stamp_text,
             "// {bits, M/256, K/64, N, {best shape for splitK 1, 2, 3, 4, 6, 8: kind, n_tiles, row_tiles, row_waves, k_waves, time in 0.02 us}}"]
    for (xb, BS, OC, IC) in sorted(rows):
        r = rows[(xb, BS, OC, IC)]
        cells = []
        for sk in (str(v) for v in SPLITS):
            if sk in r["best"]:
                cfg, t = r["best"][sk]
                cells.append("{%d,%d,%d,%d,%d,%d}" % (*cfg, min(65535, int(round(t / 0.02)))))
            else:
                cells.append("{255,0,0,0,0,0}")
        lines.append("{%d,%d,%d,%d,{%s}}," % (xb, OC // 256, IC // 64, BS, ",".join(cells)))
    with open(INC_PATH, "w") as f:
        f.write("\n".join(lines) + "\n")
    note_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuning", "note.txt")   # what differs between the versions of the stamps
    note = " ".join(open(note_path).read().split()) if os.path.exists(note_path) else ""
    with open(INC_PATH.replace(".inc", "_info.inc"), "w") as f:   # the same stamp as a string the library can report
        f.write('"%d entries; %s%s"\n' % (len(rows), stamp_text.replace('"', "'"), ("; " + note.replace('"', "'")) if note else ""))
    print("%d entries -> %s" % (len(rows), INC_PATH))


def merge(args):
    """Folds partial rows (sweeps with --kinds / --splits) into the full measurement file: within the kinds and splits a
    partial row covers, the old entry is stale and gives way; elsewhere the faster of the two stands."""
    rows = {}
    for line in open(args.main):
        r = json.loads(line)
        rows[(r["E"], r["M"], r["OC"], r["IC"], r["BS"])] = r
    changed = 0
    for path in args.parts:
        for line in open(path):
            p = json.loads(line)
            key = (p["E"], p["M"], p["OC"], p["IC"], p["BS"])
            part = p.get("partial", {"kinds": list(KIND_NAMES), "splits": list(SPLITS)})
            old = rows.get(key, {"E": p["E"], "M": p["M"], "OC": p["OC"], "IC": p["IC"], "BS": p["BS"], "best": {}})
            best = {}
            for sk in sorted(set(old["best"]) | set(p["best"]), key=int):
                o, n = old["best"].get(sk), p["best"].get(sk)
                if o is not None and int(sk) in part["splits"] and KIND_NAMES[o[0][0]] in part["kinds"]:
                    o = None   # re-measured: whatever the old entry says about this kind is out of date
                cands = [c for c in (o, n) if c is not None]
                if cands:
                    best[sk] = min(cands, key=lambda c: c[1])
            old["best"] = best
            for stamp in ("lib", "rocm"):   # the row is as new as its newest part
                if stamp in p:
                    old[stamp] = p[stamp]
            rows[key] = old
            changed += 1
    with open(args.main, "w") as f:
        for key in sorted(rows):
            f.write(json.dumps(rows[key]) + "\n")
    print("%s: %d problems, %d partial rows folded in" % (args.main, len(rows), changed))


def compact(args):
    """Rewrites measurement files in place with one line per problem, the latest (re-measured shapes are appended by `sweep --append`)."""
    for path in sorted(p for pat in args.files for p in glob.glob(pat)):
        rows = {}
        for line in open(path):
            r = json.loads(line)
            rows[(r["E"], r["M"], r["OC"], r["IC"], r["BS"])] = r
        with open(path, "w") as f:
            for key in sorted(rows):
                f.write(json.dumps(rows[key]) + "\n")
        print("%s: %d problems" % (path, len(rows)))


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    s = sub.add_parser("sweep")
    s.add_argument("--format", type=int, choices=sorted(FORMAT_OF_BITS), default=6,
                   help="bit width: 6 = e3m2 (e2m3 streams the same bytes and shares its table), 5 = e2m2, 4 = e2m1")
    s.add_argument("--out", required=True)
    s.add_argument("--append", action="store_true")
    s.add_argument("--m", default="")
    s.add_argument("--k", default="")
    s.add_argument("--n", default="")
    s.add_argument("--pairs", default="", help="OCxIC,OCxIC,... instead of the m x k grid, or `models` for the built-in list of layer shapes")
    s.add_argument("--kinds", default="", help="stream, tile, ws (comma-separated): measure only these kernels' shapes (the rows are partial: see merge)")
    s.add_argument("--splits", default="", help="measure only these splitK values (the rows are partial: see merge)")
    s.add_argument("--shapes", default="", help="measure only these shapes, kind.nt.rt.wr.wk,... (shapes added to the library: merge keeps the faster of old and new)")
    s.add_argument("--iters", type=int, default=30)
    s.add_argument("--reps", type=int, default=5)
    s.set_defaults(fn=sweep)
    e = sub.add_parser("emit")
    e.add_argument("files", nargs="+")
    e.set_defaults(fn=emit)
    m = sub.add_parser("merge")
    m.add_argument("main")
    m.add_argument("parts", nargs="+")
    m.set_defaults(fn=merge)
    c = sub.add_parser("compact")
    c.add_argument("files", nargs="+")
    c.set_defaults(fn=compact)
    args = ap.parse_args(argv)
    args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
