"""Command-line check of one GEMM through the reference-named API, the counterpart of the reference's Python harness
(tests/python/kernel_test_fp6.py, kernel_test_fpx.py: same flags, same quantities, this package's own code):

    python -m fp6_llm_amd.kernel_test --OC 4096 --IC 4096 --BS 8 [--splitK 0] [--EXP 3 --MAN 2] [--repeat 1000]

Random raw weights -> weight_prepacking_eXmY_cpu -> linear_forward_eXmY_cuda, timed with HIP events over `repeat` eager
launches after a warm-up; the FP16 GEMM of the same shape on the same GPU (torch F.linear on weight_dequant_eXmY_cpu's
output, i.e. hipBLASLt) is timed the same way.  Prints time, TFLOP/s = 2*OC*IC*BS/t, the speed-up, and the error of the
FPx result against the FP16 GEMM (mean|err| / mean|ref|, the reference's figure) and against an FP32 matmul of the
dequantized weights (max |err| / max(|ref|, rms ref)).  --splitK 0 asks the engine's heuristic.
Eager launches include Python and launch overhead (several microseconds each); bench.py replays HIP graphs instead.

    python -m fp6_llm_amd.kernel_test --suite llama2-70b [--BS 1,8,32] [--EXP 3 --MAN 2]

runs the shape lists of the reference's run scripts (tests/python/run.sh:33-34, tests/cpp/run.sh:7-8,14-15,22-23) one after
the other, each at the batch sizes given (default: the scripts' own 1..64) with the engine's split-K, and prints one summary
line per GEMM."""
import argparse
import sys


def run(OC, IC, BS, splitK=0, EXP=3, MAN=2, repeat=1000, warmup=10, seed=0, out=sys.stdout):
    import torch

    import fp6_llm_amd as fp6

    if OC % 256 or IC % 64 or BS < 1:
        raise ValueError("need OC % 256 == 0, IC % 64 == 0, BS >= 1")
    bits = 1 + EXP + MAN
    gen = torch.Generator().manual_seed(seed)
    raw = torch.randint(-2 ** 31, 2 ** 31 - 1, (OC, IC // 32 * bits), generator=gen, dtype=torch.int64).to(torch.int32)  # every bit pattern is a weight
    scale = (torch.rand(OC, generator=gen) + 0.5).half()
    act = (torch.rand(BS, IC, generator=gen) + 0.5).half()
    if splitK <= 0:
        splitK = fp6.heuristic_splitk_mi355x(OC, BS, IC, EXPONENT=EXP, MANTISSA=MAN)

    dev = torch.device("cuda:0")
    packed = fp6.weight_prepacking_eXmY_cpu(EXP, MAN, raw).to(dev)
    scale_d, act_d = scale.to(dev), act.to(dev)

    def timed(fn):
        for _ in range(warmup):
            y = fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(repeat):
            y = fn()
        e1.record()
        torch.cuda.synchronize()
        return y, e0.elapsed_time(e1) / repeat

    y_fpx, ms_fpx = timed(lambda: fp6.linear_forward_eXmY_cuda(EXP, MAN, act_d, packed, scale_d, splitK))
    w16 = fp6.weight_dequant_eXmY_cpu(EXP, MAN, raw, scale).to(dev)
    y_f16, ms_f16 = timed(lambda: torch.nn.functional.linear(act_d, w16))
    ref32 = act_d.float() @ w16.float().t()

    flops = 2.0 * OC * IC * BS
    err16 = (y_f16.float() - y_fpx.float()).abs().mean().item() / y_f16.float().abs().mean().item()
    denom = torch.maximum(ref32.abs(), ref32.pow(2).mean().sqrt())
    err32 = ((y_fpx.float() - ref32).abs() / denom).max().item()
    res = {"OC": OC, "IC": IC, "BS": BS, "splitK": splitK, "EXP": EXP, "MAN": MAN, "fpx_ms": ms_fpx, "fp16_ms": ms_f16,
           "fpx_tflops": flops / ms_fpx / 1e9, "fp16_tflops": flops / ms_f16 / 1e9, "speedup": ms_f16 / ms_fpx,
           "mean_err_vs_fp16_gemm": err16, "max_rel_err_vs_fp32": err32}
    print("FP%d_e%dm%d  OC=%d IC=%d BS=%d splitK=%d  (%d eager launches each)" % (bits, EXP, MAN, OC, IC, BS, splitK, repeat), file=out)
    print("fp16 GEMM (hipBLASLt) : %8.4f ms  %8.1f TFLOP/s" % (ms_f16, res["fp16_tflops"]), file=out)
    print("FPx  GEMM (this code) : %8.4f ms  %8.1f TFLOP/s" % (ms_fpx, res["fpx_tflops"]), file=out)
    print("speed-up              : %8.2f" % res["speedup"], file=out)
    print("mean|err|/mean|ref| vs the fp16 GEMM            : %.3e" % err16, file=out)
    print("max |err|/max(|ref|, rms ref) vs fp32 matmul     : %.3e" % err32, file=out)
    return res


# (OC, IC) lists of the reference's run scripts
SUITES = {
    "llama2-70b": [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)],                                   # tests/python/run.sh:33-34
    "llama1-65b": [(13824, 5120), (5120, 13824), (22016, 8192), (8192, 22016)],                                  # tests/cpp/run.sh:7-8
    "opt": [(21504, 7168), (7168, 7168), (28672, 7168), (7168, 28672), (27648, 9216), (9216, 9216), (36864, 9216), (9216, 36864),
            (36864, 12288), (12288, 12288), (49152, 12288), (12288, 49152)],                                     # tests/cpp/run.sh:14-15
    "llama1": [(12288, 4096), (4096, 4096), (11008, 4096), (4096, 11008), (15360, 5120), (5120, 5120), (13824, 5120), (5120, 13824),
               (19968, 6656), (6656, 6656), (17920, 6656), (6656, 17920), (24576, 8192), (8192, 8192), (22016, 8192), (8192, 22016)],  # :22-23
}


def run_suite(name, batches, EXP, MAN, repeat, out=sys.stdout):
    import io
    rows = []
    for (OC, IC) in SUITES[name]:
        for BS in batches:
            r = run(OC, IC, BS, 0, EXP, MAN, repeat, out=io.StringIO())
            rows.append(r)
            print("OC=%6d IC=%6d BS=%4d splitK=%d  FPx %8.4f ms %7.1f TFLOP/s   fp16 %8.4f ms   speed-up %5.2f   max rel err %.2e"
                  % (OC, IC, BS, r["splitK"], r["fpx_ms"], r["fpx_tflops"], r["fp16_ms"], r["speedup"], r["max_rel_err_vs_fp32"]), file=out, flush=True)
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description="One FPx x FP16 GEMM: (OC, IC) weights times (BS, IC) activations -> (BS, OC).")
    ap.add_argument("--OC", type=int, default=4096, help="rows of the weight matrix (multiple of 256)")
    ap.add_argument("--IC", type=int, default=4096, help="columns of the weight matrix (multiple of 64)")
    ap.add_argument("--BS", default="32", help="batch size (a comma-separated list with --suite)")
    ap.add_argument("--suite", choices=sorted(SUITES), help="run a shape list of the reference's run scripts instead of one GEMM")
    ap.add_argument("--splitK", type=int, default=0, help="split of the K dimension; 0 = the engine's heuristic")
    ap.add_argument("--EXP", type=int, default=3, choices=(2, 3), help="exponent bits")
    ap.add_argument("--MAN", type=int, default=2, choices=(1, 2, 3), help="mantissa bits (e3m2, e2m2, e2m3 and e2m1 exist)")
    ap.add_argument("--repeat", type=int, default=1000)
    a = ap.parse_args(argv)
    batches = [int(b) for b in str(a.BS).split(",")]
    if a.suite:
        run_suite(a.suite, batches if "," in str(a.BS) or a.BS != "32" else [1, 2, 4, 8, 16, 32, 64], a.EXP, a.MAN, min(a.repeat, 200))
        return
    run(a.OC, a.IC, batches[0], a.splitK, a.EXP, a.MAN, a.repeat)


if __name__ == "__main__":
    main()
