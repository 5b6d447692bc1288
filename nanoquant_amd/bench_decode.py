"""Decode benchmark harness over the linear layers of a decoder stack.

Counterpart of the reference's harness (src/nanoquant/kernel/test_decode.py:880-1046: sweep over batch sizes,
prompt lengths and numbers of new tokens; warm-up runs, then measured iterations; one CSV row per iteration plus
an AGGREGATE row per configuration; a summary after every configuration and a table at the end), restricted to
what this package implements: the binary low-rank linears.  A "token step" is one pass over all linears of the
stack; attention, norms, sampling and the KV cache of a real model are not part of it, so the rates are those of
the linear layers alone.  Weights are synthetic (i.i.d. signs, |N(0, 0.02)| scales) at the shapes of the chosen
model, activations are random; every linear reads its own input, as in the reference's per-layer timing.

    python -m nanoquant_amd.bench_decode --model_shape llama2-7b --layers 32 --batch_size 1,4 \
        --prompt_tokens 128 --max_new_tokens 128 --quant_kernel_type runlist --iters 3

Energy: with --profile_energy the average board power is sampled with `rocm-smi --showpower --json` in a thread
during the measured region (the reference uses Zeus, test_decode.py:288-330); blank when rocm-smi is missing.
"""
from __future__ import annotations

import argparse
import csv
import json
import os
import shutil
import subprocess
import sys
import threading
import time
from typing import Any, Dict, List, Optional

# (name, out_features, in_features); ranks follow from the bits per weight unless given
MODEL_SHAPES = {
    "llama2-7b": (("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
                  ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008)),
    "llama3-70b": (("q", 8192, 8192), ("k", 1024, 8192), ("v", 1024, 8192), ("o", 8192, 8192),
                   ("gate", 28672, 8192), ("up", 28672, 8192), ("down", 8192, 28672)),
    "qwen3-8b": (("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
                 ("gate", 12288, 4096), ("up", 12288, 4096), ("down", 4096, 12288)),
    "tiny": (("a", 256, 512), ("b", 512, 256)),
}
DEFAULT_LAYERS = {"llama2-7b": 32, "llama3-70b": 80, "qwen3-8b": 36, "tiny": 2}


def parse_int_list(text, name: str) -> List[int]:
    """'1,4,16' -> [1, 4, 16] (the reference accepts comma or space separated lists, test_decode.py:52-75)."""
    if isinstance(text, int):
        vals = [text]
    elif isinstance(text, (list, tuple)):
        vals = [int(v) for v in text]
    else:
        vals = [int(v) for v in str(text).replace(",", " ").split()]
    if not vals or any(v < 0 for v in vals):
        raise ValueError(f"{name}: expected a list of non-negative integers, got {text!r}")
    return vals


def nominal_rank(m: int, n: int, bpw: float) -> int:
    """Rank at which r (m + n) sign bits are bpw bits per weight, as a multiple of 32 (at least 32)."""
    r = int(round(bpw * m * n / (m + n)))
    return max(32, (r + 31) // 32 * 32)


def _to_float(x) -> Optional[float]:
    if x in (None, ""):
        return None
    try:
        return float(str(x).strip())
    except ValueError:
        return None


PEAK_FIELDS = ("gpu_mem_peak_alloc_bytes", "gpu_mem_peak_reserved_bytes")


def aggregate_config_rows(rows: List[Dict[str, Any]]) -> Dict[str, Any]:
    """AGGREGATE row of one configuration (test_decode.py:720-800): peaks take the maximum, rates are total tokens
    over total time, energy per token is total energy over total tokens, other numeric fields the mean."""
    if not rows:
        return {}
    agg: Dict[str, Any] = {k: "" for k in rows[0]}
    agg["iter"] = "AGGREGATE"
    for k in rows[0]:
        vals = [_to_float(r.get(k)) for r in rows]
        if k == "iter" or any(v is None for v in vals):
            if k != "iter" and all(r.get(k) == rows[0].get(k) for r in rows):
                agg[k] = rows[0].get(k)
            continue
        agg[k] = max(vals) if k in PEAK_FIELDS else sum(vals) / len(vals)
    tokens = sum(_to_float(r["decode_tokens_total"]) or 0.0 for r in rows)
    t = sum(_to_float(r["decode_time_s"]) or 0.0 for r in rows)
    agg["decode_tokens_total"] = int(tokens)
    agg["decode_time_s"] = f"{t:.6f}"
    if t > 0 and tokens > 0:
        bs = _to_float(rows[0]["batch_size"]) or 1.0
        agg["decode_tps_total"] = f"{tokens / t:.6f}"
        agg["decode_tps_per_seq"] = f"{tokens / t / bs:.6f}"
    energy = [_to_float(r.get("decode_energy_j")) for r in rows]
    if all(e is not None for e in energy) and tokens > 0:
        agg["decode_energy_j"] = f"{sum(energy):.6f}"
        agg["decode_energy_per_token_j"] = f"{sum(energy) / tokens:.9f}"
    ptime = [_to_float(r.get("prefill_time_s")) for r in rows]
    if all(p is not None for p in ptime):
        agg["prefill_time_s"] = f"{sum(ptime) / len(ptime):.6f}"
    for k in ("batch_size", "prompt_tokens", "max_new_tokens", "layers"):
        agg[k] = rows[0][k]
    return agg


def format_summary_table(summaries: List[Dict[str, Any]]) -> str:
    cols = ["batch_size", "prompt_tokens", "max_new_tokens", "prefill_time_s", "decode_tps_total", "us_per_token_step",
            "weight_GBps", "decode_energy_per_token_j", "gpu_mem_peak_alloc_gb"]
    rows = [[str(s.get(c, "")) for c in cols] for s in summaries]
    widths = [max(len(c), *(len(r[i]) for r in rows)) if rows else len(c) for i, c in enumerate(cols)]
    line = lambda cells: " | ".join(c.rjust(w) for c, w in zip(cells, widths))
    return "\n".join([line(cols), "-+-".join("-" * w for w in widths)] + [line(r) for r in rows])


class PowerSampler:
    """Average board power over a region, sampled with rocm-smi in a thread (blank when unavailable)."""

    def __init__(self, period_s: float = 0.05):
        self.period = period_s
        self.samples: List[float] = []
        self._stop = threading.Event()
        self._thread: Optional[threading.Thread] = None
        self.tool = shutil.which("rocm-smi")

    @staticmethod
    def parse(text: str) -> Optional[float]:
        try:
            data = json.loads(text)
        except ValueError:
            return None
        for card in data.values():
            if isinstance(card, dict):
                for key, val in card.items():
                    if "power" in key.lower():
                        v = _to_float(val)
                        if v is not None:
                            return v
        return None

    def _run(self) -> None:
        while not self._stop.is_set():
            try:
                out = subprocess.run([self.tool, "--showpower", "--json"], capture_output=True, text=True, timeout=5).stdout
                w = self.parse(out)
                if w is not None:
                    self.samples.append(w)
            except (OSError, subprocess.SubprocessError):
                return
            self._stop.wait(self.period)

    def __enter__(self):
        if self.tool:
            self._thread = threading.Thread(target=self._run, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self._thread:
            self._thread.join(timeout=10)

    def mean_watts(self) -> Optional[float]:
        return sum(self.samples) / len(self.samples) if self.samples else None


class LinearStack:
    """Synthetic packed weights of `layers` decoder layers and the three ways of running a token step over them."""

    def __init__(self, shape_name: str, layers: int, bpw: float, dtype, device, seed: int):
        import torch

        from . import packing
        self.torch = torch
        self.dtype, self.device = dtype, device
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        self.layers = []
        self.weight_bytes = 0
        for _ in range(layers):
            layer = []
            for name, m, n in MODEL_SHAPES[shape_name]:
                r = nominal_rank(m, n, bpw)
                rnd = lambda *s: torch.randint(-2 ** 31, 2 ** 31 - 1, s, dtype=torch.int64, device=device, generator=gen).to(torch.int32)
                sc = lambda k: (torch.randn(k, device=device, generator=gen).abs() * 0.02 + 1e-3).to(dtype)
                lin = dict(name=name, m=m, n=n, r=r, vt=rnd(r, (n + 31) // 32), u=rnd(m, (r + 31) // 32),
                           s_in=sc(n), s_mid=sc(r), s_out=sc(m))
                self.weight_bytes += (lin["vt"].numel() + lin["u"].numel()) * 4
                layer.append(lin)
            self.layers.append(layer)
        self._gemm = None
        self._packing = packing

    def inputs(self, batch: int, seed: int):
        torch = self.torch
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed)
        return [torch.randn(batch, lin["n"], device=self.device, generator=gen).to(self.dtype) for lin in self.layers[0]]

    # -- decode ----------------------------------------------------------------------------------
    def make_runlist_step(self, batch: int, xs, per_layer: bool, tiled: bool = True):
        """tiled: hand the words over in the run list's tile order (packing.tile_words; permuted once, here)."""
        from .runlist import DecodeRunList
        if tiled:
            for layer in self.layers:
                for lin in layer:
                    if "vt_tiled" not in lin:
                        lin["vt_tiled"] = self._packing.tile_words(lin["vt"])
                        lin["u_tiled"] = self._packing.tile_words(lin["u"])
        lists = []
        groups = [[layer] for layer in self.layers] if per_layer else [self.layers]
        for group in groups:
            rl = DecodeRunList(batch, self.dtype, self.device)
            for layer in group:
                for lin, x in zip(layer, xs):
                    if tiled:
                        rl.add(x, lin["s_in"], lin["vt_tiled"], lin["s_mid"], lin["u_tiled"], lin["s_out"], tiled=True)
                    else:
                        rl.add(x, lin["s_in"], lin["vt"], lin["s_mid"], lin["u"], lin["s_out"])
            rl.build()
            lists.append(rl)

        def step():
            for rl in lists:
                rl.run()
        step.status = lambda: max(rl.status() for rl in lists)
        return step

    def make_op_step(self, xs):
        torch = self.torch
        fn = torch.ops.binary_kernels.nanoquant_dyn_forward

        def step():
            for layer in self.layers:
                for lin, x in zip(layer, xs):
                    fn(x, lin["s_in"], lin["vt"], lin["s_mid"], lin["u"], lin["s_out"], 128, 128, 2, 2, 1, 1, 8, 8)
        step.status = lambda: 0
        return step

    def make_group_step(self, xs, one_launch: bool = False):
        """What a decoder with attention between its projections can issue without a run list: per layer the groups
        {q, k, v}, {o}, {gate, up}, {down} (one group per linear for other shapes), each group two launches
        (`ops.gemv_group_forward`), or one with `one_launch`."""
        from . import ops
        torch = self.torch
        nlin = len(self.layers[0])
        groups = ((0, 1, 2), (3,), (4, 5), (6,)) if nlin == 7 else tuple((i,) for i in range(nlin))
        batch = xs[0].shape[0]
        outs = [torch.empty(batch, lin["m"], dtype=self.dtype, device=self.device) for lin in self.layers[0]]

        def step():
            for layer in self.layers:
                for grp in groups:
                    ops.gemv_group_forward([xs[j] for j in grp],
                                           [(layer[j]["s_in"], layer[j]["vt"], layer[j]["s_mid"], layer[j]["u"], layer[j]["s_out"])
                                            for j in grp], outs=[outs[j] for j in grp], one_launch=one_launch)
        step.status = lambda: ops.gemv_group_status(self.device)
        return step

    # -- prefill ---------------------------------------------------------------------------------
    def prefill(self, tokens: int, seed: int) -> float:
        """One pass of `tokens` rows through the prefill (GEMM) kernels of every linear; seconds.  The prefill
        weight tiles are packed from the decode words on first use (signs unpacked once on the device)."""
        torch = self.torch
        if tokens <= 0:
            return 0.0
        if self._gemm is None:
            self._gemm = []
            for layer in self.layers:
                for lin in layer:
                    vt = self._packing.binary_unpacker(lin["vt"], (lin["r"], lin["n"]), "half2")
                    u = self._packing.binary_unpacker(lin["u"], (lin["m"], lin["r"]), "half2")
                    self._gemm.append(self._packing.marlin_nanoquant_packer(vt.T, u.T, lin["s_in"], lin["s_mid"], lin["s_out"]))
                    del vt, u
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed)
        xs = [torch.randn(tokens, lin["n"], device=self.device, generator=gen).to(self.dtype) for lin in self.layers[0]]
        fn = torch.ops.binary_kernels.marlin_nanoquant_forward
        nlin = len(self.layers[0])

        def run():
            for i, packed in enumerate(self._gemm):
                fn(xs[i % nlin], *packed)
        run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run()
        torch.cuda.synchronize()
        return time.perf_counter() - t0


def run_config(stack: LinearStack, args, bs: int, pt: int, new: int, power: bool) -> List[Dict[str, Any]]:
    torch = stack.torch
    xs = stack.inputs(bs, args.seed + 1)
    kind = args.quant_kernel_type
    if kind == "runlist":
        step = stack.make_runlist_step(bs, xs, per_layer=False, tiled=args.tiled)
    elif kind == "runlist-per-layer":
        step = stack.make_runlist_step(bs, xs, per_layer=True, tiled=args.tiled)
    elif kind in ("gemv-group", "gemv-group-one-launch"):
        step = stack.make_group_step(xs, one_launch=kind.endswith("one-launch"))
    else:
        step = stack.make_op_step(xs)
    graph = None
    if args.graph and kind != "gemv":
        step()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
    tokens_in_loop = max(new - 1, 0)          # the first new token comes out of the prefill, as in the reference
    rows = []
    for run_idx in range(1, args.warmup + args.iters + 1):
        measured = run_idx > args.warmup
        torch.cuda.reset_peak_memory_stats(stack.device)
        prefill_s = stack.prefill(pt, args.seed + 2) if (measured and pt > 0 and not args.skip_prefill) else None
        sampler = PowerSampler() if (power and measured) else None
        torch.cuda.synchronize()
        if sampler:
            sampler.__enter__()
        t0 = time.perf_counter()
        for _ in range(tokens_in_loop):
            graph.replay() if graph is not None else step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if sampler:
            sampler.__exit__(None, None, None)
        if step.status() != 0:
            raise RuntimeError("a bounded dependency wait expired inside a run-list launch")
        if not measured:
            continue
        total = bs * tokens_in_loop
        watts = sampler.mean_watts() if sampler else None
        rows.append({
            "iter": run_idx - args.warmup,
            "model_shape": args.model_shape,
            "layers": len(stack.layers),
            "bits_per_weight": args.bits,
            "batch_size": bs,
            "prompt_tokens": pt,
            "max_new_tokens": new,
            "decode_tokens_per_seq": tokens_in_loop,
            "decode_tokens_total": total,
            "decode_time_s": f"{dt:.6f}",
            "decode_tps_total": f"{total / dt:.6f}" if total > 0 and dt > 0 else "",
            "decode_tps_per_seq": f"{total / dt / bs:.6f}" if total > 0 and dt > 0 else "",
            "us_per_token_step": f"{dt / tokens_in_loop * 1e6:.3f}" if tokens_in_loop > 0 else "",
            "weight_GBps": f"{stack.weight_bytes * tokens_in_loop / dt / 1e9:.1f}" if tokens_in_loop > 0 and dt > 0 else "",
            "dtype": args.dtype,
            "graph": int(graph is not None),
            "use_quant_kernels": 1,
            "quant_kernel_type": kind,
            "prefill_time_s": f"{prefill_s:.6f}" if prefill_s is not None else "",
            "decode_energy_j": f"{watts * dt:.6f}" if watts is not None else "",
            "decode_energy_per_token_j": f"{watts * dt / total:.9f}" if watts is not None and total > 0 else "",
            "gpu_mem_peak_alloc_bytes": torch.cuda.max_memory_allocated(stack.device),
            "gpu_mem_peak_reserved_bytes": torch.cuda.max_memory_reserved(stack.device),
        })
        print(f"[iter {run_idx - args.warmup}/{args.iters}] bs={bs} pt={pt} new={new} tps={rows[-1]['decode_tps_total']}", flush=True)
    return rows


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    p.add_argument("--model_shape", default="llama2-7b", choices=sorted(MODEL_SHAPES))
    p.add_argument("--layers", type=int, default=0, help="decoder layers (0: the model's own count)")
    p.add_argument("--bits", type=float, default=1.0, help="bits per weight of the factorisation")
    p.add_argument("--quant_kernel_type", default="runlist",
                   choices=["runlist", "runlist-per-layer", "gemv", "gemv-group", "gemv-group-one-launch"],
                   help="runlist: the whole stack in one launch per token; runlist-per-layer: one launch per layer; "
                        "gemv: the reference's way, one operator call (two launches) per linear; gemv-group: per layer "
                        "the groups {q,k,v}, {o}, {gate,up}, {down}, two launches each; gemv-group-one-launch: one each")
    p.add_argument("--batch_size", default="1", help="list, e.g. 1,4,16")
    p.add_argument("--prompt_tokens", default="128", help="list of prompt lengths for the prefill pass (0: none)")
    p.add_argument("--max_new_tokens", default="128", help="list")
    p.add_argument("--warmup", type=int, default=1)
    p.add_argument("--iters", type=int, default=3)
    p.add_argument("--output_csv", default=None)
    p.add_argument("--dtype", default="float16", choices=["float16", "bfloat16"])
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--gpu_id", type=int, default=0)
    p.add_argument("--no_graph", dest="graph", action="store_false", help="launch from Python instead of replaying a graph")
    p.add_argument("--skip_prefill", action="store_true")
    p.add_argument("--row_major", dest="tiled", action="store_false",
                   help="run lists read the reference's row-major words instead of the tile order")
    p.add_argument("--profile_energy", action="store_true")
    return p


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    import torch

    import nanoquant_amd  # noqa: F401  (registers the ops, loads the library or raises)
    if not torch.cuda.is_available():
        print("bench_decode: no GPU visible", file=sys.stderr)
        return 1
    device = torch.device(f"cuda:{args.gpu_id}")
    dtype = getattr(torch, args.dtype)
    batches = parse_int_list(args.batch_size, "batch_size")
    prompts = parse_int_list(args.prompt_tokens, "prompt_tokens")
    news = parse_int_list(args.max_new_tokens, "max_new_tokens")
    layers = args.layers or DEFAULT_LAYERS[args.model_shape]
    stack = LinearStack(args.model_shape, layers, args.bits, dtype, device, args.seed)
    print(f"{args.model_shape}: {layers} layers, {stack.weight_bytes / 1e9:.2f} GB of packed signs", flush=True)
    all_rows: List[Dict[str, Any]] = []
    summaries = []
    for bs in batches:
        for pt in prompts:
            for new in news:
                rows = run_config(stack, args, bs, pt, new, args.profile_energy)
                if not rows:
                    continue
                agg = aggregate_config_rows(rows)
                gb = _to_float(agg.get("gpu_mem_peak_alloc_bytes"))
                summary = {k: agg.get(k, "") for k in ("batch_size", "prompt_tokens", "max_new_tokens", "prefill_time_s",
                                                        "decode_tps_total", "decode_energy_per_token_j")}
                t, n_steps = _to_float(agg["decode_time_s"]), args.iters * max(new - 1, 0)
                summary["us_per_token_step"] = f"{t / n_steps * 1e6:.2f}" if n_steps else ""
                summary["weight_GBps"] = f"{stack.weight_bytes * n_steps / t / 1e9:.1f}" if n_steps and t else ""
                summary["gpu_mem_peak_alloc_gb"] = f"{gb / 2 ** 30:.3f}" if gb is not None else ""
                print(f"== bs={bs} pt={pt} new={new}: {summary['decode_tps_total']} tokens/s, "
                      f"{summary['us_per_token_step']} us per token step", flush=True)
                summaries.append(summary)
                all_rows.extend(rows)
                all_rows.append(agg)
    if all_rows and args.output_csv:
        os.makedirs(os.path.dirname(args.output_csv) or ".", exist_ok=True)
        with open(args.output_csv, "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=list(all_rows[0].keys()))
            w.writeheader()
            w.writerows(all_rows)
        print(f"[OK] wrote CSV -> {args.output_csv}")
    print(format_summary_table(summaries))
    return 0


if __name__ == "__main__":
    sys.exit(main())
