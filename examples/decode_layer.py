#!/usr/bin/env python3
"""The linear layers of one transformer decoder layer at decode batch sizes, FPx weights against FP16 weights.

    python examples/decode_layer.py [--model 7b|70b] [--format 6|5|4] [--batch 1,8,32] [--group-scales]

Builds the four GEMMs of a LLaMA-shaped layer as `FPxLinear` modules -- Q, K and V fused into one launch and gate and up
into another with `FPxLinear.fused` -- quantizes random weights on the GPU, captures one pass over the four layers into a
HIP graph (the attention and activation functions between them are left out: this measures the weight-streaming part of
a decode step) and times it against the same four GEMMs on FP16 weights through `torch.nn.functional.linear`.
Weights are synthetic; each layer's weights rotate through enough copies that every pass streams them from HBM.
"""
import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from fp6_llm_amd.module import FPxLinear  # noqa: E402

SHAPES = {   # hidden, heads*head_dim for K/V (grouped-query attention in the 70B model), MLP width
    "7b": dict(hidden=4096, kv=4096, mlp=11008),
    "70b": dict(hidden=8192, kv=1024, mlp=28672),
}


def timed_graph(fn, copies, reps=20):
    """Median microseconds of one call of fn(i) for i over the weight copies, captured as a graph of `copies` passes."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(copies):
            fn(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(copies):
                fn(i)
        for _ in range(5):
            graph.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) * 1e3 / copies)
    return sorted(times)[len(times) // 2]


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", default="7b", choices=sorted(SHAPES))
    ap.add_argument("--format", type=int, default=6, choices=(4, 5, 6), help="6 = FP6_e3m2, 5 = FP5_e2m2, 4 = FP4_e2m1")
    ap.add_argument("--batch", default="1,8,32")
    ap.add_argument("--group-scales", action="store_true", help="a power-of-two factor per row and 128 columns besides the row scales")
    args = ap.parse_args()
    dims = SHAPES[args.model]
    H, KV, F = dims["hidden"], dims["kv"], dims["mlp"]
    E, M = {6: (3, 2), 5: (2, 2), 4: (2, 1)}[args.format]
    dev = torch.device("cuda:0")
    layer_bytes_fp16 = 2 * (H * (H + 2 * KV) + H * H + 2 * F * H + H * F)
    copies = max(2, min(16, (1 << 30) // layer_bytes_fp16 + 1))   # > 256 MB of distinct weights per pass over the copies

    def make(copy):
        g = torch.Generator(device=dev).manual_seed(copy)
        w = lambda o, i: torch.randn(o, i, generator=g, device=dev, dtype=torch.float16) * 0.02   # noqa: E731
        wq, wk, wv, wo, wg, wu, wd = w(H, H), w(KV, H), w(KV, H), w(H, H), w(F, H), w(F, H), w(H, F)
        q = lambda t: FPxLinear.from_float(t, E, M, group_scales=args.group_scales)   # noqa: E731
        fpx = dict(qkv=FPxLinear.fused([q(t) for t in (wq, wk, wv)]), o=q(wo), gate_up=FPxLinear.fused([q(t) for t in (wg, wu)]), down=q(wd))
        f16 = dict(qkv=torch.cat([wq, wk, wv]), o=wo, gate_up=torch.cat([wg, wu]), down=wd)
        return fpx, f16

    layers = [make(c) for c in range(copies)]
    print("LLaMA-%s-shaped layer, FP%d_e%dm%d vs FP16, %d weight copies rotating (%.0f MB of FP16 weights per layer)"
          % (args.model, 1 + E + M, E, M, copies, layer_bytes_fp16 / 1e6))
    for B in [int(b) for b in args.batch.split(",")]:
        x_h = torch.randn(B, H, device=dev, dtype=torch.float16)
        x_f = torch.randn(B, F, device=dev, dtype=torch.float16)

        def run_fpx(i):
            L = layers[i][0]
            L["qkv"](x_h), L["o"](x_h), L["gate_up"](x_h), L["down"](x_f)

        def run_f16(i):
            W = layers[i][1]
            lin = torch.nn.functional.linear
            lin(x_h, W["qkv"]), lin(x_h, W["o"]), lin(x_h, W["gate_up"]), lin(x_f, W["down"])

        t_fpx, t_f16 = timed_graph(run_fpx, copies), timed_graph(run_f16, copies)
        print("batch %3d: four GEMMs per layer  FPx %7.1f us   FP16 %7.1f us   speed-up %.2f" % (B, t_fpx, t_f16, t_f16 / t_fpx))


if __name__ == "__main__":
    main()
