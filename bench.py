#!/usr/bin/env python3
"""Benchmark of the FPx x FP16 linear layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--sweep]

A step is one GEMM of the workload (default: the headline one, FP6_e3m2 4096x4096, batch 8, split-K from the engine's
heuristic).  Weights are synthetic, already resident in HBM, and ROTATE through a pool of distinct buffers larger than the
256 MB last-level cache, so every step streams its weights from HBM like consecutive layers of a model would ("cold");
--warm (and --sweep) add the same-buffer figure.  The K steps are captured once into a HIP graph and replayed inside
the timed region, which removes the Python launch cost (~6 us/launch) from a ~5 us kernel.  The graph is first replayed
untimed for ~60 ms (right after an idle spell the GPU runs 10-15 % slow); then the K-step graph is replayed back to back, as
many times as it takes to cover ~10 ms, between ONE pair of events, five times over, and the median is reported as time per
step = event time / (replays x steps in the graph); a graph holds the K steps several times over when K is small -- a
20-step graph would spread the 6-8 us between two replays over only 20 kernels of 5 us.  The FP16 baseline and the read-only floor are timed the same way.
The default run also times every point of the benchmark configurations (`detail.configs`, 29 workloads) beside an FP16 GEMM of
its shape, and one large FP16 library GEMM as the measured MFMA rate of this GPU (`detail.fp16_peak_tflops_measured`).

Prints ONE JSON line: value = weight bytes streamed per second (the bandwidth figure the reference's design is judged
on), ms_per_step = time per GEMM; `roofline` prices the GEMM kernel against the 8 TB/s HBM peak from HIP-event time on the
launch stream; `cpu_baseline` times the reference's CPU path (dequantize, then a torch CPU matmul) on this host;
`detail.read_floor_us` is the time of a kernel that only reads the same weight buffers the same way (no arithmetic).
--sweep additionally runs every benchmark configuration and writes one JSON line per configuration to --sweep-out.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
POOL_BYTES = 1 << 30            # distinct weight buffers cycled through: 4x the 256 MB last-level cache

WORKLOADS = {
    # name: (E, M, OC, IC, BS)
    "fp6_4096x4096_bs8": (3, 2, 4096, 4096, 8),
    "fp6_4096x4096_bs1": (3, 2, 4096, 4096, 1),
    "fp6_4096x4096_bs16": (3, 2, 4096, 4096, 16),
    "fp6_11008x4096_bs8": (3, 2, 11008, 4096, 8),
    "fp6_11008x4096_bs32": (3, 2, 11008, 4096, 32),
    "fp6_4096x11008_bs8": (3, 2, 4096, 11008, 8),
    "fp6_4096x11008_bs32": (3, 2, 4096, 11008, 32),
    "fp6_10240x8192_bs32": (3, 2, 10240, 8192, 32),
    "fp6_28672x8192_bs32": (3, 2, 28672, 8192, 32),
    "fp6_8192x28672_bs32": (3, 2, 8192, 28672, 32),
}
for _bs in (1, 2, 4, 8, 16, 32, 64, 128, 256, 512):
    WORKLOADS["fp6_8192x8192_bs%d" % _bs] = (3, 2, 8192, 8192, _bs)
    WORKLOADS["fp5_8192x8192_bs%d" % _bs] = (2, 2, 8192, 8192, _bs)
for _bs in (1, 8, 32, 128):   # the two formats beyond the reference's: same shapes, for the sweep
    WORKLOADS["fp6e2m3_8192x8192_bs%d" % _bs] = (2, 3, 8192, 8192, _bs)
    WORKLOADS["fp4_8192x8192_bs%d" % _bs] = (2, 1, 8192, 8192, _bs)
WORKLOADS["fp4_4096x4096_bs8"] = (2, 1, 4096, 4096, 8)
HEADLINE = "fp6_4096x4096_bs8"

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what the same counter reads
# for a 64 MiB device copy (`--calibrate-copy`); the runs and readings are in profiles/gemm_*_<workload>.md.
MEASURED_TRAFFIC_BYTES = {   # workload: bytes per launch of the GEMM kernel, and fp6mi_version() of the library that was profiled
    "fp4_8192x8192_bs8": {"bytes": 34856037, "lib_version": 134},
    "fp5_8192x8192_bs1": {"bytes": 42218021, "lib_version": 134},
    "fp5_8192x8192_bs64": {"bytes": 58875593, "lib_version": 134},
    "fp5_8192x8192_bs8": {"bytes": 43262175, "lib_version": 134},
    "fp6_10240x8192_bs32": {"bytes": 75087832, "lib_version": 134},
    "fp6_11008x4096_bs32": {"bytes": 36735643, "lib_version": 134},
    "fp6_11008x4096_bs8": {"bytes": 34670774, "lib_version": 134},
    "fp6_28672x8192_bs32": {"bytes": 182364291, "lib_version": 134},
    "fp6_4096x4096_bs8": {"bytes": 13288927, "lib_version": 134},
    "fp6_8192x8192_bs1": {"bytes": 50623135, "lib_version": 134},
    "fp6_8192x8192_bs512": {"bytes": 125930205, "lib_version": 134},
    "fp6_8192x8192_bs64": {"bytes": 67853755, "lib_version": 134},
    "fp6_8192x8192_bs8": {"bytes": 51635556, "lib_version": 134},
}


def weight_bytes(E, M, OC, IC):
    return OC * IC * (1 + E + M) // 8


def algorithmic_bytes(E, M, OC, IC, BS):
    """weights + scales + activations once + output once"""
    return weight_bytes(E, M, OC, IC) + 2 * OC + 2 * BS * IC + 2 * BS * OC


class WeightPool:
    """Native-layout weight buffers of one (format, OC, IC), distinct contents, together larger than the last-level cache, and
    the row scales; shared by the problems that differ only in their batch."""

    def __init__(self, E, M, OC, IC, device):
        import torch
        import fp6_llm_amd as fp6
        from fp6_llm_amd import quant, synth

        self.E, self.M, self.OC, self.IC, self.device = E, M, OC, IC, device
        nbytes = fp6.native_bytes(E, M, OC, IC)
        self.nbuf = int(max(2, min(128, POOL_BYTES // nbytes)))
        # distinct buffers, distinct contents: uniform random codes (every bit pattern is a valid weight)
        self.weights = []
        rows = min(OC, 1024)
        block = fp6.weight_prepacking_native_cpu(E, M, torch.from_numpy(quant.pack_raw(synth.uniform_codes(2001, rows, IC, E, M), E, M)))
        reps = OC // rows + (1 if OC % rows else 0)
        base = block.repeat(reps)[: nbytes // 4].contiguous().to(device)
        for i in range(self.nbuf):
            self.weights.append(torch.roll(base, shifts=257 * i) if i else base)
        self.scales = torch.from_numpy(synth.uniform_scales(2001, OC)).to(device)


class Problem:
    """Device buffers of one workload: a pool of native-layout weight buffers, scales, activations, output, workspace."""

    def __init__(self, E, M, OC, IC, BS, device, pool=None):
        import torch
        import fp6_llm_amd as fp6
        from fp6_llm_amd import synth

        self.E, self.M, self.OC, self.IC, self.BS = E, M, OC, IC, BS
        self.splitK = fp6.heuristic_splitk_mi355x(OC, BS, IC, EXPONENT=E, MANTISSA=M)
        pool = pool or WeightPool(E, M, OC, IC, device)
        self.nbuf, self.weights, self.scales = pool.nbuf, pool.weights, pool.scales
        self.x = torch.from_numpy(synth.activations(2001, BS, IC)).to(device)
        self.out = torch.empty((BS, OC), dtype=torch.float16, device=device)
        self.ws = torch.empty(self.splitK * BS * OC, dtype=torch.float32, device=device) if self.splitK > 1 else None

    def step(self, i, cold=True):
        import fp6_llm_amd as fp6

        w = self.weights[i % self.nbuf] if cold else self.weights[0]
        fp6.linear_forward_native(self.E, self.M, self.x, w, self.scales, self.OC, self.splitK, out=self.out, workspace=self.ws)


CLOCK_WARMUP_MS = 60.0   # untimed graph replays before the timed ones: the first replays after an idle spell run 10-15 % slow
TIMED_REGION_MS = 10.0   # one timed region = back-to-back replays of the K-step graph covering about this long
TIMED_REGIONS = 5        # the median over this many regions is reported


def _timed_replays(graph, steps):
    """Replays the captured K-step graph untimed until the clocks have settled, then times TIMED_REGIONS regions of R
    back-to-back replays each, R chosen so that a region lasts about TIMED_REGION_MS.
    Returns (median wall seconds per step, median HIP-event microseconds per step, R)."""
    import torch

    spent, n, last = 0.0, 0, 0.0
    while n < 2 or (spent < CLOCK_WARMUP_MS and n < 200):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        last = e0.elapsed_time(e1)
        spent += last
        n += 1
    replays = int(max(1, min(20000, round(TIMED_REGION_MS / max(last, 1e-3)))))
    walls, evs = [], []
    for _ in range(TIMED_REGIONS):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for _r in range(replays):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - t0) / (replays * steps))
        evs.append(e0.elapsed_time(e1) * 1e3 / (replays * steps))
    return sorted(walls)[len(walls) // 2], sorted(evs)[len(evs) // 2], replays


MIN_GRAPH_STEPS = 240    # a captured graph holds the K steps this many times over if K is smaller: starting and ending a replay costs
                         # 6-8 us on this stack, which a 20-step graph of 5 us kernels would book as 0.3-0.4 us per step


def _capture_and_time(step, steps, warmup):
    """`step(i)` enqueues step i on the current stream.  W eager warm-up steps, then the K steps (several times over when K is
    small, see MIN_GRAPH_STEPS) captured into one graph and timed by _timed_replays; all figures are per step."""
    import torch

    stream = torch.cuda.Stream()
    rounds = max(1, -(-MIN_GRAPH_STEPS // steps))
    with torch.cuda.stream(stream):
        for i in range(max(warmup, 1)):
            step(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(steps * rounds):
                step(warmup + i)
        return _timed_replays(graph, steps * rounds)


def time_steps(prob, steps, warmup, cold):
    """Returns (wall seconds per step, HIP-event microseconds per step on the launch stream, replays per timed region)."""
    return _capture_and_time(lambda i: prob.step(i, cold), steps, warmup)


def read_floor_us(prob, steps, warmup):
    """Time of a kernel that only reads the same weight buffers (same rotation, same graph protocol, same 128-bit
    non-temporal loads and launch geometry as the small-batch GEMM): what any single-pass kernel over these bytes pays."""
    import ctypes

    import torch

    path = os.path.join(ROOT, "fp6_llm_amd", "libfp6mi_probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.fp6mi_probe_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.fp6mi_probe_stream_read.restype = ctypes.c_int
    sink = torch.zeros(16, dtype=torch.int32, device=prob.x.device)
    nbytes = prob.weights[0].numel() * prob.weights[0].element_size()

    def step(i):
        w = prob.weights[i % prob.nbuf]
        rc = lib.fp6mi_probe_stream_read(torch.cuda.current_stream().cuda_stream, w.data_ptr(), nbytes, sink.data_ptr())
        assert rc == 0, rc

    return _capture_and_time(step, steps, warmup)[1]


def xcd_locality_probe(device):
    """Pairs of kernels in the benchmark's back-to-back graph: the first writes `wgs` regions, the second reads them, region
    (b + shift) mod wgs by workgroup b.  Workgroup ids congruent mod 8 share an XCD, so shift 0 and 8 read through the L2 the
    data was written through, shift 1 and 3 from another XCD.  Returns microseconds per pair, launches included."""
    import ctypes

    import torch

    lib = ctypes.CDLL(os.path.join(ROOT, "fp6_llm_amd", "libfp6mi_probe.so"))
    lib.fp6mi_probe_write_then_read.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_void_p]
    lib.fp6mi_probe_write_then_read.restype = ctypes.c_int
    buf = torch.empty(256 << 20, dtype=torch.uint8, device=device)
    sink = torch.zeros(16, dtype=torch.int32, device=device)
    rows = []
    for wgs, per in ((256, 4), (256, 16), (256, 64), (512, 8)):
        row = {"megabytes": round(wgs * per * 4096 / 1e6, 2), "workgroups": wgs}
        for shift in (0, 8, 1, 3):
            def step(i):
                rc = lib.fp6mi_probe_write_then_read(torch.cuda.current_stream().cuda_stream, buf.data_ptr(), wgs, per, shift, sink.data_ptr())
                assert rc == 0, rc
            row["shift_%d_%s_xcd_us" % (shift, "same" if shift % 8 == 0 else "other")] = round(_capture_and_time(step, 100, 5)[1], 3)
        rows.append(row)
    return {"probe": "write kernel then read kernel, us per pair in a back-to-back graph", "rows": rows}


class _RocblasFp16:
    """rocblas_gemm_ex (FP16 in/out, FP32 accumulation) through ctypes: the second FP16 library path on this stack, which
    for some shapes picks a faster kernel than torch's F.linear and for others a much slower one."""

    def __init__(self):
        import ctypes
        self.ct = ctypes
        self.lib = ctypes.CDLL("librocblas.so")
        self.handle = ctypes.c_void_p()
        if self.lib.rocblas_create_handle(ctypes.byref(self.handle)) != 0:
            raise RuntimeError("rocblas_create_handle failed")
        vp, ci, u32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint32
        self.lib.rocblas_set_stream.argtypes = [vp, vp]
        self.lib.rocblas_gemm_ex.argtypes = [vp, ci, ci, ci, ci, ci, vp, vp, ci, ci, vp, ci, ci, vp, vp, ci, ci, vp, ci, ci, ci, ci, ctypes.c_int32, u32]
        self.alpha, self.beta = ctypes.c_float(1.0), ctypes.c_float(0.0)

    def linear(self, x, w, out, stream):
        """out[B, OC] = x[B, IC] @ w[OC, IC]^T; column-major view: C[OC x B] = op_T(w as IC x OC) * (x as IC x B)."""
        ct = self.ct
        B, IC = x.shape
        OC = w.shape[0]
        self.lib.rocblas_set_stream(self.handle, stream)
        rc = self.lib.rocblas_gemm_ex(self.handle, 112, 111, OC, B, IC, ct.addressof(self.alpha), w.data_ptr(), 150, IC, x.data_ptr(), 150, IC,
                                      ct.addressof(self.beta), out.data_ptr(), 150, OC, out.data_ptr(), 150, OC, 151, 0, 0, 0)
        if rc != 0:
            raise RuntimeError("rocblas_gemm_ex failed with status %d" % rc)


def _time_fp16(fn, steps, warmup):
    import torch

    try:
        return _capture_and_time(fn, steps, warmup)[1]
    except RuntimeError:  # the BLAS library refused capture: time plain launches instead
        torch.cuda.synchronize()
        for i in range(3 * steps):   # untimed, to settle the clocks
            fn(i)
        reps = max(steps, 200)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(reps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps


def fp16_baseline_us(prob, steps, warmup, with_rocblas=True):
    """FP16 GEMM of the same shape on the same GPU, weights rotating the same way: the counterpart of the reference's cuBLAS
    baseline (tests/python/kernel_test_fp6.py:45-62, tests/cpp/kernel_test_fpx.cu:80-103).  Two library paths are timed,
    torch F.linear (hipBLASLt) and rocblas_gemm_ex; returns (the faster one, {path: us})."""
    import torch

    dev = prob.x.device
    nb = prob.OC * prob.IC * 2
    nbuf = int(max(2, min(64, POOL_BYTES // nb)))
    ws = [torch.randn(prob.OC, prob.IC, dtype=torch.float16, device=dev) for _ in range(nbuf)]
    out = torch.empty(prob.BS, prob.OC, dtype=torch.float16, device=dev)
    res = {"torch_F_linear": _time_fp16(lambda i: torch.nn.functional.linear(prob.x, ws[i % nbuf]), steps, warmup)}
    try:
        if not with_rocblas:
            raise OSError("second library path not wanted")
        rb = _RocblasFp16()
        # same answer as F.linear before it is trusted as a baseline
        rb.linear(prob.x, ws[0], out, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        ref = torch.nn.functional.linear(prob.x, ws[0])
        if torch.allclose(out.float(), ref.float(), rtol=2e-2, atol=2e-2 * float(ref.float().abs().mean())):
            res["rocblas_gemm_ex"] = _time_fp16(lambda i: rb.linear(prob.x, ws[i % nbuf], out, torch.cuda.current_stream().cuda_stream), steps, warmup)
    except (OSError, RuntimeError, AttributeError):
        pass
    return min(res.values()), res


def fp16_system_blas_us(OC, IC, BS, steps):
    """The same FP16 GEMM through the SYSTEM's rocBLAS/hipBLASLt, in a process of its own (torch bundles older copies of
    those libraries, and the newer ones pick a faster kernel for some shapes): the C++ driver's `fp16` mode, eager
    launches back to back on one stream, weights rotating through 1 GiB.  None if the driver is not built."""
    import re
    import subprocess

    exe = os.path.join(ROOT, "fp6_llm_amd", "kernel_bench")
    if not os.path.exists(exe):
        return None
    try:
        res = subprocess.run([exe, "fp16", str(OC), str(IC), str(BS), str(steps), "20"], capture_output=True, text=True, timeout=300)
    except (OSError, subprocess.SubprocessError):
        return None
    m = re.search(r": ([0-9.]+) us/GEMM", res.stdout)
    return float(m.group(1)) if res.returncode == 0 and m else None


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _best_median(fn, min_reps=3, budget_s=4.0):
    ts = []
    while len(ts) < min_reps or (sum(ts) < budget_s and len(ts) < 50):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[0], ts[len(ts) // 2], len(ts)


def cpu_baseline(E, M, OC, IC, BS):
    """The reference's CPU path on this host, each leg timed by itself (at least 3 repeats, best and median):
      prepack  weight_matrix_prepacking      (utils/weight_prepacking.h:118-196)  -> this build's bit-exact fp6mi_prepack_ref (one thread per host cpu)
      dequant  DeQuantMatrix_FPx_To_FP16     (utils/weight_dequant.h:10-48)       -> fp6mi_dequant (one thread per host cpu) and the scalar C oracle (1 thread)
      matmul   torch CPU fp16 F.linear of the dequantized weights (tests/python/kernel_test_fp6.py:48-58, on the CPU)
    `value` is the per-GEMM path the reference runs, dequantize + matmul, with the oracle's dequantizer (kind "port"), in
    weight bytes per second; prepacking is ahead-of-time work and reported beside it."""
    import numpy as np
    import torch

    import oracle
    import fp6_llm_amd as fp6
    from fp6_llm_amd import quant, synth

    raw = quant.pack_raw(synth.uniform_codes(2001, OC, IC, E, M), E, M)
    sc = synth.uniform_scales(2001, OC)
    x = torch.from_numpy(synth.activations(2001, BS, IC))
    raw_t, sc_t = torch.from_numpy(raw), torch.from_numpy(sc)
    threads = int(torch.get_num_threads())
    prepack = _best_median(lambda: fp6.weight_prepacking_eXmY_cpu(E, M, raw_t), budget_s=3.0)
    deq_own = _best_median(lambda: fp6.weight_dequant_eXmY_cpu(E, M, raw_t, sc_t), budget_s=3.0)
    deq_orc = _best_median(lambda: oracle.dequant(raw, sc, E, M), budget_s=5.0)
    w = torch.from_numpy(oracle.dequant(raw, sc, E, M))
    assert np.array_equal(fp6.weight_dequant_eXmY_cpu(E, M, raw_t, sc_t).numpy().view(np.uint16), w.numpy().view(np.uint16))
    mm = _best_median(lambda: torch.nn.functional.linear(x, w), budget_s=3.0)
    per = deq_orc[1] + mm[1]
    ms = lambda t: round(t * 1e3, 3)
    return {
        "value": round(weight_bytes(E, M, OC, IC) / per / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "FP%d %dx%d BS %d on '%s' (%d cpus, torch threads %d), median of >= 3 repeats per leg: oracle dequant (1 thread) %.1f ms + "
                  "torch CPU fp16 F.linear (%d threads) %.2f ms per GEMM; ahead of time: fp6mi_prepack_ref (all host threads) %.1f ms; "
                  "fp6mi_dequant (all host threads) %.1f ms"
                  % (1 + E + M, OC, IC, BS, _cpu_model(), os.cpu_count(), threads, deq_orc[1] * 1e3, threads, mm[1] * 1e3, prepack[1] * 1e3, deq_own[1] * 1e3),
        "us_per_gemm": round(per * 1e6, 1),
        "legs_ms": {"prepack_fp6mi_all_threads": {"best": ms(prepack[0]), "median": ms(prepack[1]), "repeats": prepack[2]},
                    "dequant_fp6mi_all_threads": {"best": ms(deq_own[0]), "median": ms(deq_own[1]), "repeats": deq_own[2]},
                    "dequant_oracle_1thread": {"best": ms(deq_orc[0]), "median": ms(deq_orc[1]), "repeats": deq_orc[2]},
                    "matmul_torch_fp16": {"best": ms(mm[0]), "median": ms(mm[1]), "repeats": mm[2], "threads": threads}},
        "cpu_model": _cpu_model(), "host_cpus": os.cpu_count(),
    }


def run_workload(name, steps, warmup, device, with_fp16=True, with_warm=True, with_system_blas=True, with_floor=True):
    E, M, OC, IC, BS = WORKLOADS[name]
    prob = Problem(E, M, OC, IC, BS, device)
    wall_s, us, replays = time_steps(prob, steps, warmup, cold=True)
    wb = weight_bytes(E, M, OC, IC)
    flops = 2.0 * OC * IC * BS
    res = {
        "workload": name, "us_per_gemm": round(us, 3), "us_per_gemm_wall": round(wall_s * 1e6, 3), "replays_per_timed_region": replays,
        "weight_GBps": round(wb / us / 1e3, 1), "tflops": round(flops / us / 1e6, 2),
        "hbm_frac": round(wb / us / 1e3 / HBM_PEAK_GBPS, 4), "mfma_frac": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4),
        "splitK": prob.splitK, "weight_buffers": prob.nbuf, "weight_bytes": wb, "algorithmic_bytes": algorithmic_bytes(E, M, OC, IC, BS),
    }
    if with_warm:   # same weight buffer every step: served by the last-level cache when it fits
        us_warm = time_steps(prob, steps, warmup, cold=False)[1]
        res["us_per_gemm_warm"] = round(us_warm, 3)
        res["weight_GBps_warm"] = round(wb / us_warm / 1e3, 1)
    floor = read_floor_us(prob, steps, warmup) if with_floor else None
    if floor is not None:
        res["read_floor_us"] = round(floor, 3)               # a kernel that only reads these weight buffers once
        res["read_floor_GBps"] = round(wb / floor / 1e3, 1)
        res["frac_of_read_floor"] = round(floor / us, 4)
    if with_fp16:
        del prob.weights[2:]
        import torch
        torch.cuda.empty_cache()
        f16, paths = fp16_baseline_us(prob, min(steps, 200), min(warmup, 10), with_rocblas=with_system_blas)
        if with_system_blas:
            del prob
            torch.cuda.empty_cache()
            ext = fp16_system_blas_us(OC, IC, BS, 500)
            if ext is not None:
                paths["system_rocblas_own_process"] = ext
                f16 = min(f16, ext)
        res["fp16_gemm_us"] = round(f16, 3)             # the fastest of the FP16 library paths
        res["fp16_gemm_us_by_path"] = {k: round(v, 3) for k, v in paths.items()}
        res["speedup_vs_fp16"] = round(f16 / us, 3)
    return res


# Every point of the benchmark configurations beyond the headline one, timed by the default run (`detail.configs`): 4096 x 4096 at
# batch 1 and 16, the two MLP shapes of a 7B model at batch 8 and 32, the three GEMMs of a 70B layer at batch 32, and the
# 8192 x 8192 sweep over ten batches in both of the reference's formats (the sweep of tests/python/run.sh:37-46).
CONFIG_WORKLOADS = (["fp6_4096x4096_bs1", "fp6_4096x4096_bs16", "fp6_11008x4096_bs8", "fp6_11008x4096_bs32", "fp6_4096x11008_bs8", "fp6_4096x11008_bs32",
                     "fp6_10240x8192_bs32", "fp6_28672x8192_bs32", "fp6_8192x28672_bs32"]
                    + ["fp%d_8192x8192_bs%d" % (x, bs) for bs in (1, 2, 4, 8, 16, 32, 64, 128, 256, 512) for x in (6, 5)])


class _Fp16Pool:
    """fp16 weights of one shape rotating through 1 GiB like the FPx ones, for the FP16 library GEMM beside each workload."""

    def __init__(self, OC, IC, device):
        import torch
        nb = OC * IC * 2
        self.nbuf = int(max(2, min(64, POOL_BYTES // nb)))
        self.ws = [torch.randn(OC, IC, dtype=torch.float16, device=device) for _ in range(self.nbuf)]


def fp16_peak_tflops(device):
    """One large square FP16 GEMM through torch (hipBLASLt): the MFMA rate a tuned library reaches on this GPU, to read the
    large-batch figures against (the published peak of 2.5 PFLOP/s is not reached by any GEMM here)."""
    import torch

    n = 8192
    a = torch.randn(n, n, dtype=torch.float16, device=device)
    b = torch.randn(n, n, dtype=torch.float16, device=device)
    for _ in range(5):
        torch.matmul(a, b)
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            torch.matmul(a, b)
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) / 10 * 1e-3
        best = t if best is None or t < best else best
    return round(2.0 * n * n * n / best / 1e12, 1)


def run_configs(device, budget_s):
    """[{workload, us, splitK, hbm_frac | mfma_frac, fp16_us, speedup}] within a time budget (workloads that no longer fit are listed
    as skipped).  FP16 = torch F.linear (hipBLASLt) on fp16 weights of the same shape rotating the same way, same graph protocol;
    workloads that share a weight matrix share its buffers, and an FP16 time is measured once per (shape, batch)."""
    import torch

    out, t0 = [], time.perf_counter()
    pool, pool_key, f16pool, f16_key, f16_us = None, None, None, None, {}
    for name in CONFIG_WORKLOADS:
        if time.perf_counter() - t0 > budget_s:
            out.append({"workload": name, "skipped": "time budget"})
            continue
        E, M, OC, IC, BS = WORKLOADS[name]
        if pool_key != (E, M, OC, IC):
            pool = None
            torch.cuda.empty_cache()
            pool, pool_key = WeightPool(E, M, OC, IC, device), (E, M, OC, IC)
        big = OC * IC > 64e6
        steps = 40 if big else 100
        prob = Problem(E, M, OC, IC, BS, device, pool)
        us = time_steps(prob, steps, 5, cold=True)[1]
        wb, flops = weight_bytes(E, M, OC, IC), 2.0 * OC * IC * BS
        entry = {"workload": name, "us": round(us, 3), "splitK": prob.splitK, "weight_GBps": round(wb / us / 1e3, 1), "tflops": round(flops / us / 1e6, 2)}
        if BS >= 128:
            entry["mfma_frac"] = round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)
        else:
            entry["hbm_frac"] = round(wb / us / 1e3 / HBM_PEAK_GBPS, 4)
        if (OC, IC, BS) not in f16_us:
            if f16_key != (OC, IC):
                f16pool = None
                torch.cuda.empty_cache()
                f16pool, f16_key = _Fp16Pool(OC, IC, device), (OC, IC)
            fw, x = f16pool, prob.x
            f16_us[(OC, IC, BS)] = _time_fp16(lambda i: torch.nn.functional.linear(x, fw.ws[i % fw.nbuf]), steps, 5)
        entry["fp16_us"] = round(f16_us[(OC, IC, BS)], 3)
        entry["speedup"] = round(f16_us[(OC, IC, BS)] / us, 3)
        out.append(entry)
        del prob
    return out


def measured_traffic(workload):
    """HBM bytes per launch from the committed profiler summary of this workload, or None when there is none or when it was
    taken with another version of the library than the one loaded now (a changed kernel makes the figure stale)."""
    import fp6_llm_amd._lib as _lib

    rec = MEASURED_TRAFFIC_BYTES.get(workload)
    if rec is None or rec["lib_version"] != _lib.lib().fp6mi_version():
        return None
    return rec["bytes"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--sweep", action="store_true", help="also run every benchmark configuration with all its legs")
    ap.add_argument("--sweep-out", default="bench_sweep.jsonl", help="where --sweep writes its JSON lines")
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the legs that run outside this process's GPU stream: the CPU path and the system-BLAS FP16 baseline (a child process)")
    ap.add_argument("--no-configs", action="store_true", help="skip detail.configs (one workload per benchmark configuration)")
    ap.add_argument("--configs-budget", type=float, default=110.0, help="seconds the default run may spend on detail.configs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="profiling aid: also run ten 64 MiB device-to-device copies, a kernel of known traffic to scale profiler byte counters by; "
                         "skips the FP16, CPU and per-configuration legs")
    ap.add_argument("--probe-xcd-locality", action="store_true",
                    help="measurement aid: instead of the benchmark, time a write kernel followed by a read kernel whose workgroups run on "
                         "the writer's XCD or on another one, and print the pair times")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path runs on ONE GPU (a linear layer shards by output rows without any collective); use --gpus 1")

    import torch

    import fp6_llm_amd  # noqa: F401  (raises if libfp6mi.so is missing: there is no fallback)
    from fp6_llm_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.probe_xcd_locality:
        print(json.dumps(xcd_locality_probe(device)))
        return
    if args.calibrate_copy:
        src = torch.empty(64 << 20, dtype=torch.uint8, device=device).random_()
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
    res = run_workload(args.workload, args.steps, args.warmup, device, with_fp16=not args.calibrate_copy, with_warm=not args.calibrate_copy,
                       with_system_blas=not args.no_cpu_baseline)
    E, M, OC, IC, BS = WORKLOADS[args.workload]
    res["lib_version"] = _lib.lib().fp6mi_version()
    res["launch_table"] = _lib.lib().fp6mi_tuning_info().decode()
    if not (args.no_configs or args.calibrate_copy):
        res["configs"] = run_configs(device, args.configs_budget)
        res["fp16_peak_tflops_measured"] = fp16_peak_tflops(device)   # 8192^3 FP16 GEMM, torch/hipBLASLt
    compute_bound = BS >= 128
    line = {
        "metric": "weight bytes streamed per second by the FPx x FP16 GEMM (us/GEMM in ms_per_step)", "value": res["weight_GBps"], "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(res["us_per_gemm"] / 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "%s: FP%d_e%dm%d weights [%d,%d] x fp16 activations [%d,%d], weights rotating through %d distinct HBM buffers, splitK=%d"
                               % (args.workload, 1 + E + M, E, M, OC, IC, BS, IC, res["weight_buffers"], res["splitK"])},
        "roofline": ({"bound": "mfma", "achieved": res["tflops"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": res["mfma_frac"]} if compute_bound else
                     {"bound": "hbm", "achieved": res["weight_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": res["hbm_frac"]}),
        "detail": res,
    }
    line["roofline"].update({"traffic": measured_traffic(args.workload), "bytes_per_launch": res["weight_bytes"], "kernel_us": res["us_per_gemm"]})
    if not (args.no_cpu_baseline or args.calibrate_copy):
        line["cpu_baseline"] = cpu_baseline(E, M, OC, IC, BS)
    if args.sweep:
        os.makedirs(os.path.dirname(os.path.abspath(args.sweep_out)), exist_ok=True)
        with open(args.sweep_out, "w") as f:
            for name in WORKLOADS:
                big = WORKLOADS[name][2] * WORKLOADS[name][3] > 64e6
                r = run_workload(name, 40 if big else 100, 10, device)
                f.write(json.dumps(r) + "\n")
                f.flush()
                print("%-22s %8.2f us  %7.0f GB/s (%.1f%% HBM)  %7.1f TFLOP/s  read-only %7.2f us  fp16 %8.2f us  x%.2f" % (
                    name, r["us_per_gemm"], r["weight_GBps"], 100 * r["hbm_frac"], r["tflops"], r.get("read_floor_us", float("nan")),
                    r["fp16_gemm_us"], r["speedup_vs_fp16"]), file=sys.stderr, flush=True)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
