"""Prefill benchmark over the linear layers of one decoder layer.

Times `marlin_nanoquant_forward` (two one-bit GEMMs per linear, the reference's prefill path:
src/nanoquant/modules/linear.py:131-133, src/nanoquant/kernel/cuda/gemm.cpp:112-122) on synthetic weights at the
shapes of the chosen model, one linear after the other and, unless --no_group, all linears of the layer in shared
launches (`ops.gemm_group_forward`).  Rates count 2 * tokens * r * (m + n) flops per linear at the nominal rank; the
fraction is of the 2.5 PFLOP/s dense fp16 matrix peak of an MI355X.

    python -m nanoquant_amd.bench_prefill --model_shape llama2-7b --tokens 128,512 --iters 5

With --no_graph the calls are launched eagerly (for profilers that should see every launch of its own); otherwise
`--reps` passes are captured in one HIP graph and the graph is replayed `--iters` times.
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import Any, Dict, List

from .bench_decode import MODEL_SHAPES, parse_int_list

MFMA_F16_PEAK_TFLOPS = 2500.0


def prefill_rank(m: int, n: int, bpw: float) -> int:
    """Rank at which r (m + n) sign bits are bpw bits per weight."""
    return max(32, int(round(bpw * m * n / (m + n))))


def run(argv=None) -> List[Dict[str, Any]]:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model_shape", default="llama2-7b", choices=sorted(MODEL_SHAPES))
    ap.add_argument("--tokens", default="128,512")
    ap.add_argument("--bpw", type=float, default=1.0)
    ap.add_argument("--dtype", default="float16", choices=("float16", "bfloat16"))
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--reps", type=int, default=5, help="passes over the layer per graph")
    ap.add_argument("--no_graph", action="store_true")
    ap.add_argument("--no_group", action="store_true")
    ap.add_argument("--no_single", action="store_true", help="skip the one-linear-after-the-other leg")
    ap.add_argument("--panel", default="auto", choices=("auto", "always", "never"),
                    help="grouped leg: persistent panel launches where the library's policy picks them (auto), for every "
                         "stage (always), or the launches without a workspace only (never)")
    ap.add_argument("--constant_data", action="store_true",
                    help="activations 0 and all signs +1 instead of random data: the same instructions with nothing "
                         "toggling in the multipliers, to show how much of the time is the part's response to switching power")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args(argv)

    import torch

    import nanoquant_amd  # noqa: F401  registers torch.ops.binary_kernels
    from . import ops, packing

    if not torch.cuda.is_available():
        raise RuntimeError("bench_prefill needs a GPU: the prefill kernels have no CPU path")
    dev = torch.device("cuda:0")
    dtype = getattr(torch, args.dtype)
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)
    shapes = MODEL_SHAPES[args.model_shape]
    op = torch.ops.binary_kernels.marlin_nanoquant_forward

    packed_by_shape: Dict[Any, Any] = {}
    for (_, m, n) in shapes:                      # linears of one shape share a weight copy
        if (m, n) in packed_by_shape:
            continue
        r = prefill_rank(m, n, args.bpw)
        v = torch.randint(0, 2, (n, r), device=dev, generator=gen, dtype=torch.int8) * 2 - 1
        u = torch.randint(0, 2, (r, m), device=dev, generator=gen, dtype=torch.int8) * 2 - 1
        if args.constant_data:
            v, u = torch.ones_like(v), torch.ones_like(u)
        sc = lambda k: (torch.randn(k, device=dev, generator=gen).abs() * 0.02 + 1e-3).to(dtype)
        packed_by_shape[(m, n)] = (packing.marlin_nanoquant_packer(v, u, sc(n), sc(r), sc(m)), r)
        del v, u
    terms = [packed_by_shape[(m, n)][0] for (_, m, n) in shapes]

    def timed(fn) -> float:
        """Microseconds per call of fn."""
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if args.no_graph:
            e0.record()
            for _ in range(args.iters * args.reps):
                fn()
            e1.record()
        else:
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                fn()
            side.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                for _ in range(args.reps):
                    fn()
            g.replay()
            torch.cuda.synchronize()
            e0.record()
            for _ in range(args.iters):
                g.replay()
            e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (args.iters * args.reps)

    rows = []
    for tokens in parse_int_list(args.tokens, "tokens"):
        xs_by_n = {n: torch.randn(tokens, n, device=dev, generator=gen).to(dtype) for n in {n for (_, _, n) in shapes}}
        if args.constant_data:
            xs_by_n = {n: torch.zeros_like(x) for n, x in xs_by_n.items()}
        xs = [xs_by_n[n] for (_, _, n) in shapes]
        flops = sum(2.0 * tokens * packed_by_shape[(m, n)][1] * (m + n) for (_, m, n) in shapes)
        row: Dict[str, Any] = {"model_shape": args.model_shape, "tokens": tokens, "dtype": args.dtype, "panel": args.panel,
                               "data": "constant" if args.constant_data else "random", "linears": len(shapes), "GFLOP_per_layer": round(flops / 1e9, 2)}
        legs = []
        if not args.no_single:
            legs.append(("one_by_one", lambda: [op(x, *t) for x, t in zip(xs, terms)]))
        if not args.no_group:
            legs.append(("grouped", lambda: ops.gemm_group_forward(xs, terms, panel=args.panel)))
        for name, fn in legs:
            us = timed(fn)
            tf = flops / (us * 1e-6) / 1e12
            row[name] = {"us_per_layer": round(us, 2), "TFLOPs": round(tf, 1),
                         "frac_of_f16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        print(json.dumps(row), flush=True)
        rows.append(row)
    return rows


if __name__ == "__main__":
    run(sys.argv[1:])
