#!/usr/bin/env python3
"""Benchmark of the binary low-rank linear layer on one MI355X.

Headline workload (N=1): the batch-1 decode GEMV over Llama-2-7B-shaped decoder layers at 1.0 bpw -- per layer q/k/v/o
4096x4096 (r=2048), gate/up 11008x4096 and down 4096x11008 (r = round(mn/(m+n)) = 2985) -- fp16 activations.  One
"step" is one token step over the linear layers of a whole 32-layer decoder stack (224 linears, 810 MB of packed
words, every word read once per step, so the words come from HBM and not from the 256 MB Infinity Cache), enqueued as
ONE run-list launch, one run-list launch over the whole stack of independent linears.  `value` is algorithmic bytes / time; `us_per_layer` = step time
/ 32.  The same layer as one launch per layer (rotating over the 32 weight copies) is in `extra`, with a roofline
object of its own.

Prints ONE JSON line.  Extra keys report batch 4 and 16, the prefill GEMM at 128, 512 and 4096 tokens (`roofline_prefill`
is the 128-token headline), the two-term Qwen3-8B-like layer (cfg3) and the Llama-3-70B weight stream (cfg4);
`cpu_baseline` is the reference's dense CPU path (two F.linear on unpacked +-1 factors) timed on this host.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the headline kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a
# copy kernel of known size (profiles/gemv_stream_llama2_7b_stack_b1.md); valid for the default workload only.
MEASURED_TRAFFIC_BYTES = 843630592
# The same for the two launches of the 128-token grouped layer (profiles/gemm_group_llama2_7b_layer_prefill.md):
# (18756 + 26222) KiB x 2.000 fetched + (4352 + 48686) KiB written; 38.9 MB each way of the second launch are partial
# tiles that its workgroups hand over through device-coherent memory.
MEASURED_PREFILL_TRAFFIC_BYTES = (18756 + 26222) * 2 * 1024 + (4352 + 48686) * 1024
MFMA_F16_PEAK_TFLOPS = 2500.0

LLAMA2_7B_LAYER = (("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
                   ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008))


def nominal_rank(m, n):
    return int(round(m * n / (m + n)))


def gemv_bytes(m, n, r, batch):
    """Algorithmic bytes of one decode call: packed bits at the nominal rank + fp16 scales + x + y."""
    return r * (m + n) / 8 + 2 * (n + r + m) + 2 * batch * (n + m)


def gemm_flops(m, n, r, tokens):
    return 2.0 * tokens * r * (m + n)


class SynthLinear:
    """Random packed factors of one linear, resident on the GPU (decode layout)."""

    def __init__(self, torch, dev, m, n, r, gen):
        self.m, self.n, self.r = m, n, r
        self.rp = (r + 31) // 32 * 32          # rank padded to whole words; padding has s_mid = 0
        i32 = torch.iinfo(torch.int32)
        self.vt_bits = torch.randint(i32.min, i32.max, (self.rp, n // 32), dtype=torch.int32, device=dev, generator=gen)
        self.u_bits = torch.randint(i32.min, i32.max, (m, self.rp // 32), dtype=torch.int32, device=dev, generator=gen)

        def scale(k):
            return (torch.randn(k, device=dev, generator=gen).abs() * 0.02 + 1e-3).to(torch.float16)

        self.s_in, self.s_mid, self.s_out = scale(n), scale(self.rp), scale(m)
        if self.rp > r:
            self.s_mid[r:] = 0
        self._tiled = None
        self._scales_alt = None

    def runlist_words(self, keep_row_major=True):
        """(first-stage words, second-stage words) in the tile order that run lists read fastest: a fixed
        permutation of the row-major words (nanoquant_amd.packing.tile_words), done once here, outside any timing."""
        if self._tiled is None:
            from nanoquant_amd import packing
            self._tiled = (packing.tile_words(self.vt_bits), packing.tile_words(self.u_bits))
            if not keep_row_major:
                self.vt_bits = self.u_bits = None
        return self._tiled

    def add_to(self, rl, x, keep_row_major=True, **kw):
        """Tile order at every batch size: the run-list kernels fetch an item with scalar address arithmetic there
        (Llama-2-7B stack at batch 16 13.0 against 14.1 us per layer on row-major words, one launch per layer 47 against
        53)."""
        s_in, s_mid, s_out = self.scales_as(x.dtype)
        vt, u = self.runlist_words(keep_row_major)
        return rl.add(x, s_in, vt, s_mid, u, s_out, tiled=True, **kw)

    def scales_as(self, dtype):
        """The scale vectors in the activation type (drawn as fp16; converted once for bf16 runs)."""
        if dtype == self.s_in.dtype:
            return self.s_in, self.s_mid, self.s_out
        if self._scales_alt is None or self._scales_alt[0].dtype != dtype:
            self._scales_alt = (self.s_in.to(dtype), self.s_mid.to(dtype), self.s_out.to(dtype))
        return self._scales_alt


def build_layers(torch, dev, shapes, copies, seed):
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    return [[SynthLinear(torch, dev, m, n, nominal_rank(m, n), gen) for (_, m, n) in shapes] for _ in range(copies)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--copies", type=int, default=32, help="decoder layers of the stack = distinct weight copies of the layer "
                                                           "(32 x 25.3 MB = 810 MB > 256 MB Infinity Cache)")
    ap.add_argument("--no-extra", action="store_true", help="skip batch 4/16, prefill and CPU legs")
    ap.add_argument("--cfg4-only", action="store_true",
                    help="after the headline run only the Llama-3-70B-shaped stream (cfg4) of the extra legs: the short "
                         "command that the profiles of that leg are taken with")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch the library's plain copy kernel on 256 MiB (5x): a known-traffic reference "
                         "for scaling profiler memory counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the layer is a single-GPU hot path); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import nanoquant_amd  # noqa: F401
    from nanoquant_amd import _lib, packing

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    lib = _lib.lib()
    vp = ctypes.c_void_p

    layers = build_layers(torch, dev, LLAMA2_7B_LAYER, args.copies, seed=0)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)

    def make_io(batch, dtype=torch.float16):
        xs = [torch.randn(batch, lin.n, device=dev, generator=gen).to(dtype) for lin in layers[0]]
        hs = [torch.empty(batch, lin.rp, dtype=torch.float32, device=dev) for lin in layers[0]]
        ys = [torch.empty(batch, lin.m, dtype=dtype, device=dev) for lin in layers[0]]
        return xs, hs, ys

    def layer_pass(layer, io, batch, stream):
        xs, hs, ys = io
        for lin, x, h, y in zip(layer, xs, hs, ys):
            st = lib.nq_gemv_forward(vp(x.data_ptr()), vp(lin.s_in.data_ptr()), vp(lin.vt_bits.data_ptr()),
                                     vp(lin.s_mid.data_ptr()), vp(lin.u_bits.data_ptr()), vp(lin.s_out.data_ptr()),
                                     vp(h.data_ptr()), vp(y.data_ptr()), batch, lin.n, lin.rp, lin.m, _lib.NQ_F16, stream)
            if st != 0:
                raise RuntimeError(_lib.status_message(st))

    def make_runlists(io, batch):
        """One run list (= one persistent launch) per weight copy."""
        from nanoquant_amd import DecodeRunList
        xs, _, ys = io
        lists = []
        for layer in layers:
            rl = DecodeRunList(batch, xs[0].dtype, dev)
            for lin, x, y in zip(layer, xs, ys):
                lin.add_to(rl, x, y=y)
            rl.build()
            lists.append(rl)
        return lists

    def capture_rotation(step_fns):
        """One HIP graph holding one step per weight copy, in rotation order."""
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            step_fns[0]()                      # warm (module load, function attributes)
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for fn in step_fns:
                fn()
        return g

    def timed(step_fns, steps, warmup):
        """Exactly `steps` steps: whole rotations as graph replays, the remainder as eager launches."""
        L = len(step_fns)
        g = capture_rotation(step_fns)
        for _ in range((warmup + L - 1) // L):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps // L):
            g.replay()
        for i in range(steps % L):
            step_fns[i]()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps  # ms per step

    def per_linear_steps(io, batch):
        return [(lambda layer=layer: layer_pass(layer, io, batch, vp(torch.cuda.current_stream().cuda_stream)))
                for layer in layers]

    def layer_bytes(batch):
        return sum(gemv_bytes(lin.m, lin.n, lin.r, batch) for lin in layers[0])

    # ---- headline: batch 1, one token step over the whole stack in one launch -------------------------------
    from nanoquant_amd import DecodeRunList

    def make_stack(io, batch, dtype=torch.float16, deterministic=False):
        """All linears of all layers in one list; every linear writes an output buffer of its own."""
        xs, _, _ = io
        rl = DecodeRunList(batch, dtype, dev, deterministic=deterministic)
        for layer in layers:
            for lin, x in zip(layer, xs):
                lin.add_to(rl, x)
        rl.build()
        return rl

    def stack_parity(rl, io, batch):
        """Outputs of the launch that was just timed against the dense definition (src/nanoquant/modules/linear.py:248-257
        of the reference, evaluated in fp64 by the oracle from the same packed words): 256 sampled output rows of every
        linear of the first, a middle and the last layer."""
        import numpy as np
        from oracle import nq_oracle as oracle
        xs, _, _ = io
        outs = rl.outputs
        worst_rel, worst_el = 0.0, 0.0
        c = lambda t: t.cpu().numpy()
        f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
        for li in sorted({0, len(layers) // 2, len(layers) - 1}):
            for j, (lin, x) in enumerate(zip(layers[li], xs)):
                rows = np.random.default_rng(1000 * li + j).choice(lin.m, size=256, replace=False)
                ref = oracle.layer_forward_packed(f64(x), f64(lin.s_in), c(lin.vt_bits), f64(lin.s_mid), c(lin.u_bits)[rows],
                                                  f64(lin.s_out)[rows], dtype=np.float64)
                got = outs[7 * li + j].float().cpu().numpy()[:, rows]
                worst_rel = max(worst_rel, oracle.max_rel_err(got, ref))
                worst_el = max(worst_el, oracle.elementwise_err(got, ref))
        return {"max_rel_err": float("%.3e" % worst_rel), "elementwise_err": float("%.3e" % worst_el),
                "plan_bound_flags": int(rl._plan.bound),
                "definition": "outputs of the TIMED launch (fp16, every linear its own buffer): worst of the 21 linears of the "
                              "first, a middle and the last layer, 256 sampled rows each; max|dy|/max|y_ref| and "
                              "max(|dy|/(|y_ref| + 0.1 rms(y_ref))) against the fp64 layer definition on the same packed words; "
                              "plan flags: 4 = tile order, 32 = wavefronts own row pairs"}

    def timed_launches(fn, steps, warmup):
        """Exactly `steps` launches of fn, back to back on the current stream, between two events on that stream."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps  # ms per launch

    def cfg4_leg(extra, batches=(1, 8)):
        # ---- cfg4: Llama-3-70B-shaped weight stream, 80 layers x 7 linears in one launch ----
        llama70 = (("q", 8192, 8192), ("k", 1024, 8192), ("v", 1024, 8192), ("o", 8192, 8192),
                   ("gate", 28672, 8192), ("up", 28672, 8192), ("down", 8192, 28672))
        g70 = torch.Generator(device=dev)
        g70.manual_seed(5)
        stack70 = [[SynthLinear(torch, dev, m, n, nominal_rank(m, n), g70) for (_, m, n) in llama70] for _ in range(80)]
        for b in batches:
            x70 = {n: torch.randn(b, n, device=dev, generator=g70).to(torch.float16) for n in (8192, 28672)}
            rl = DecodeRunList(b, torch.float16, dev)
            for layer in stack70:
                for lin in layer:
                    lin.add_to(rl, x70[lin.n])
            rl.build()
            ms70 = timed([rl.run], 5, 1)
            if rl.status() != 0:
                raise RuntimeError("run list reported an expired dependency wait")
            bytes70 = 80 * sum(gemv_bytes(lin.m, lin.n, lin.r, b) for lin in stack70[0])
            extra[f"cfg4_llama3_70b_stream_batch{b}"] = {
                "us_per_token_step": round(ms70 * 1e3, 1), "GBps": round(bytes70 / (ms70 * 1e-3) / 1e9, 2),
                "resident_weight_GB": round(80 * sum(lin.r * (lin.m + lin.n) / 8 for lin in stack70[0]) / 1e9, 2),
                "note": "560 linears in one run-list launch"}
            del rl
        del stack70

    io1 = make_io(1)
    stack1 = make_stack(io1, 1)
    # set-up, not part of the W warm-up steps: 300 launches (45 ms) take the device to its sustained state (the first
    # 25 ms of back-to-back launches after the weights were generated run up to 15 % slower).  The W warm-up steps and
    # the K timed steps are then launched back to back on the current stream (a launch costs the host 10 us, a step
    # takes the device 140: the queue never runs dry; replaying a one-launch graph per step leaves 4 us between steps)
    for _ in range(300):
        stack1.run()
    torch.cuda.synchronize()
    ms = timed_launches(stack1.run, args.steps, args.warmup)
    if stack1.status() != 0:
        raise RuntimeError("run list reported an expired dependency wait")
    headline_parity = stack_parity(stack1, io1, 1)
    nlayers = len(layers)
    bytes1 = layer_bytes(1)
    bytes_step = bytes1 * nlayers
    gbs = bytes_step / (ms * 1e-3) / 1e9
    result = {
        "metric": "batch-1 binary GEMV sustained GB/s over Llama-2-7B decoder layers (1.0 bpw)",
        "value": round(gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 in/out; one-bit fp4 x fp8-piece MFMA products (exact), f32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": "cfg1: batch-1 decode GEMV, one token step over the linear layers of a %d-layer Llama-2-7B-shaped "
                        "decoder stack (%d linears; per layer q/k/v/o 4096x4096 r2048, gate/up 11008x4096 and down 4096x11008 "
                        "r2985 padded to 3008 with zero mid scale; 1.0 bpw, %.0f MB of packed words, every word read once per "
                        "step, so from HBM) in ONE run-list launch; the packed words are handed over in the run list's tile "
                        "order, a fixed permutation of the reference's row-major words done once at load"
                        % (nlayers, 7 * nlayers, nlayers * sum(lin.r * (lin.m + lin.n) / 8 for lin in layers[0]) / 1e6),
            "batch": 1,
            "layers_per_step": nlayers,
            "algorithmic_bytes_per_step": int(bytes_step),
            "launches_per_step": 1,
            "setup_launches_untimed": 300,
            "step_is": "224 mutually independent linears (no link between layers, no attention or norm between them): the "
                       "sustained weight stream of the decode kernel, not a decoder's token step; decoder-shaped "
                       "launch patterns are timed in extra.decoder_pattern_*",
        },
        "us_per_layer": round(ms * 1e3 / nlayers, 3),
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_stream_kernel<fp16, batch 1, fp4 x fp8 MFMA, 1024 lanes, tile order, owned row pairs> (one launch per token step: "
                      "%d stages in 2 phases, 256 resident workgroups)" % (14 * nlayers),
            "achieved": round(gbs, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES if (args.copies == 32 and MEASURED_TRAFFIC_BYTES) else None,
            "bytes_per_launch": int(bytes_step),
            "avg_launch_us": round(ms * 1e3, 3),
        },
    }

    result["parity"] = headline_parity

    if args.calibrate_copy:
        nbytes = 256 << 20
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        for _ in range(5):
            _lib.check(lib.nq_stream_copy(vp(dst.data_ptr()), vp(src.data_ptr()), nbytes,
                                          vp(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        result["config"]["calibration_copy_bytes"] = nbytes

    if args.cfg4_only:
        extra = {}
        cfg4_leg(extra)
        result["extra"] = extra
    elif not args.no_extra:
        extra = {}
        # measured streaming ceiling of this box: the library's plain copy kernel, 256 MiB read + 256 MiB written
        nbytes = 256 << 20
        csrc_ = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_()
        cdst_ = torch.empty_like(csrc_)
        copy_fn = lambda: _lib.check(lib.nq_stream_copy(vp(cdst_.data_ptr()), vp(csrc_.data_ptr()), nbytes,
                                                        vp(torch.cuda.current_stream().cuda_stream)))
        ms_copy = timed([copy_fn], 20, 3)
        extra["hbm_copy_kernel"] = {"GBps_read_plus_write": round(2 * nbytes / (ms_copy * 1e-3) / 1e9, 1),
                                    "note": "plain 16-byte copy kernel, 256 MiB each way: a measured ceiling for streaming "
                                            "kernels on this box (vendor peak 8000 GB/s)"}
        # launch floor of this box: the same copy kernel on 16 bytes (one workgroup, nothing to do) and on 1 MiB regions
        # of the 256 MiB buffers (so that every launch reads HBM), 256 launches per graph replay
        def floor_us(nb):
            fns = [(lambda o=o: _lib.check(lib.nq_stream_copy(vp(cdst_.data_ptr() + o), vp(csrc_.data_ptr() + o), nb,
                                                              vp(torch.cuda.current_stream().cuda_stream))))
                   for o in range(0, nbytes, nbytes // 256)]
            return round(timed(fns, 1024, 256) * 1e3, 2)
        extra["launch_floor"] = {"us_per_launch_16_bytes": floor_us(16), "us_per_launch_1MiB_copy": floor_us(1 << 20),
                                 "note": "back-to-back launches in graph replay; the 1 MiB copy reads 1 MiB and writes 1 MiB"}
        del csrc_, cdst_
        for b in (4, 16):
            io = make_io(b)
            lists = make_runlists(io, b)
            msb = timed([rl.run for rl in lists], 4 * len(layers), len(layers))
            st_b = make_stack(io, b)
            ms_sb = timed_launches(st_b.run, 10, 2) / len(layers)
            if st_b.status() != 0:
                raise RuntimeError("run list reported an expired dependency wait")
            extra[f"batch{b}"] = {"parity_of_the_timed_stack": stack_parity(st_b, io, b),
                                  "us_per_layer_stack_one_launch": round(ms_sb * 1e3, 3),
                                  "GBps_stack_one_launch": round(layer_bytes(b) / (ms_sb * 1e-3) / 1e9, 2),
                                  "us_per_layer_one_launch_per_layer": round(msb * 1e3, 3),
                                  "GBps_one_launch_per_layer": round(layer_bytes(b) / (msb * 1e-3) / 1e9, 2)}
            del lists, st_b
        # bf16 activations and scales (what the reference's module defaults to), same layer and launch shape
        io_bf = make_io(1, torch.bfloat16)
        st_bf = make_stack(io_bf, 1, torch.bfloat16)
        ms_bf = timed_launches(st_bf.run, 10, 2) / len(layers)
        extra["batch1_bf16"] = {"us_per_layer": round(ms_bf * 1e3, 3), "GBps": round(bytes1 / (ms_bf * 1e-3) / 1e9, 2),
                                "note": "the headline stack with bf16 activations and scales"}
        del st_bf, io_bf
        # the headline stack with reproducible sums (every launch gives the same bits)
        st_det = make_stack(io1, 1, deterministic=True)
        ms_det = timed_launches(st_det.run, 10, 2) / len(layers)
        extra["batch1_deterministic"] = {"us_per_layer": round(ms_det * 1e3, 3),
                                         "GBps": round(bytes1 / (ms_det * 1e-3) / 1e9, 2),
                                         "note": "DecodeRunList(deterministic=True): every sum formed in a fixed order (long tile-order "
                                                 "lists: one wavefront per row pair; otherwise partial sums rounded to a "
                                                 "grid on which additions are exact)"}
        del st_det
        # the same layer as ONE launch per layer (14 stages in 2 phases), rotating over the weight copies: what a
        # caller gets who launches layer by layer; bound by the serial latencies inside a launch, not by HBM
        lists1 = make_runlists(io1, 1)
        ms_l = timed([rl.run for rl in lists1], 8 * len(layers), len(layers))
        for rl in lists1:
            if rl.status() != 0:
                raise RuntimeError("run list reported an expired dependency wait")
        extra["batch1_one_launch_per_layer"] = {
            "us_per_layer": round(ms_l * 1e3, 3), "GBps": round(bytes1 / (ms_l * 1e-3) / 1e9, 2),
            "roofline": {"bound": "hbm", "kernel": "gemv_stream_kernel, one launch per layer (14 stages in 2 phases)",
                         "achieved": round(bytes1 / (ms_l * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(bytes1 / (ms_l * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "bytes_per_launch": int(bytes1),
                         "avg_launch_us": round(ms_l * 1e3, 3)},
            "note": "graph replays of one launch per layer over %d rotating weight copies" % len(layers)}
        del lists1
        ms_pl = timed(per_linear_steps(io1, 1), 4 * len(layers), len(layers))
        extra["batch1_per_linear_launches"] = {"us_per_layer": round(ms_pl * 1e3, 3),
                                               "GBps": round(bytes1 / (ms_pl * 1e-3) / 1e9, 2),
                                               "note": "same layer through nq_gemv_forward: 14 launches per layer"}
        # ---- launch patterns with a decoder's dependency structure, over the rotating weight copies ----
        # (a) what a model with attention, norms and activations between its projections can issue: per layer four
        #     run-list launches {q,k,v}, {o}, {gate,up}, {down}, all 4 x 32 launches in one HIP graph;
        # (b) the whole stack as ONE launch whose linears are chained where the shapes allow it (v -> o -> gate/up,
        #     gate -> down -> q/k/v of the next layer): 8 dependent phases per layer instead of 2 for the whole list.
        for b in (1, 4):
            io_p = io1 if b == 1 else make_io(b)
            xs_p = io_p[0]
            per_layer = []
            for layer in layers:
                lists = []
                for group in ((0, 1, 2), (3,), (4, 5), (6,)):
                    rl = DecodeRunList(b, torch.float16, dev)
                    for j in group:
                        layer[j].add_to(rl, xs_p[j])
                    rl.build()
                    lists.append(rl)
                per_layer.append(lists)
            ms_p = timed([(lambda lists=lists: [rl.run() for rl in lists]) for lists in per_layer], 4 * len(layers), len(layers))
            for lists in per_layer:
                for rl in lists:
                    if rl.status() != 0:
                        raise RuntimeError("run list reported an expired dependency wait")
            del per_layer
            chained = DecodeRunList(b, torch.float16, dev)
            prev_down = -1
            for layer in layers:
                q, k, v, o, gate, up, down = layer
                x_in = xs_p[0] if prev_down < 0 else chained.outputs[prev_down]
                q.add_to(chained, x_in, x_from=prev_down)
                k.add_to(chained, x_in, x_from=prev_down)
                iv = v.add_to(chained, x_in, x_from=prev_down)
                io_ = o.add_to(chained, chained.outputs[iv], x_from=iv)
                ig = gate.add_to(chained, chained.outputs[io_], x_from=io_)
                up.add_to(chained, chained.outputs[io_], x_from=io_)
                prev_down = down.add_to(chained, chained.outputs[ig], x_from=ig)
            chained.build()
            ms_c = timed_launches(chained.run, 6, 2) / len(layers)
            if chained.status() != 0:
                raise RuntimeError("run list reported an expired dependency wait")
            # (c) the same four groups per layer without run lists: nq_gemv_forward_group, ordinary launches that need
            #     neither a built list nor the GPU to themselves; two launches per group (all first stages, all second
            #     stages), or one whose second stages wait inside the kernel
            from nanoquant_amd import ops as nq_ops
            ys_p = io_p[2]

            def group_step(layer, one_launch):
                for group in ((0, 1, 2), (3,), (4, 5), (6,)):
                    nq_ops.gemv_group_forward([xs_p[j] for j in group],
                                              [(layer[j].s_in, layer[j].vt_bits, layer[j].s_mid, layer[j].u_bits, layer[j].s_out)
                                               for j in group], outs=[ys_p[j] for j in group], one_launch=one_launch)

            ms_g = timed([(lambda layer=layer: group_step(layer, False)) for layer in layers], 4 * len(layers), len(layers))
            ms_g1 = timed([(lambda layer=layer: group_step(layer, True)) for layer in layers], 4 * len(layers), len(layers))
            if nq_ops.gemv_group_status(dev) != 0:
                raise RuntimeError("a group launch reported an expired wait")
            lb = layer_bytes(b)
            extra[f"decoder_pattern_batch{b}"] = {
                "four_groups_two_launches_each": {"us_per_layer": round(ms_g * 1e3, 3), "GBps": round(lb / (ms_g * 1e-3) / 1e9, 2),
                                                  "frac_of_hbm_peak": round(lb / (ms_g * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                "four_groups_one_launch_each": {"us_per_layer": round(ms_g1 * 1e3, 3), "GBps": round(lb / (ms_g1 * 1e-3) / 1e9, 2),
                                                "frac_of_hbm_peak": round(lb / (ms_g1 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                "four_launches_per_layer": {"us_per_layer": round(ms_p * 1e3, 3), "GBps": round(lb / (ms_p * 1e-3) / 1e9, 2),
                                            "frac_of_hbm_peak": round(lb / (ms_p * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                "chained_one_launch": {"us_per_layer": round(ms_c * 1e3, 3), "GBps": round(lb / (ms_c * 1e-3) / 1e9, 2),
                                       "frac_of_hbm_peak": round(lb / (ms_c * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                       "phases": int(chained._plan.nphases)},
                "note": "decoder-shaped issue patterns of the same 32 x 7 linears: per layer the launches {q,k,v}, {o}, "
                        "{gate,up}, {down} in one HIP graph: as ordinary launches of nq_gemv_forward_group, two per group "
                        "(four_groups_two_launches_each) or one per group whose second stages wait inside the kernel "
                        "(four_groups_one_launch_each), and as run-list launches (four_launches_per_layer); "
                        "chained_one_launch: one launch for the stack with v -> o -> gate/up, gate -> down -> next layer's "
                        "q/k/v linked through x_from"}
            del chained

        # ---- cfg0: one 2048 x 2048 linear of rank 1024 at batch 1 (the reference's CPU-runnable case), GPU and CPU ----
        from oracle import nq_oracle as oracle0
        g0 = torch.Generator(device=dev)
        g0.manual_seed(6)
        lin0 = SynthLinear(torch, dev, 2048, 2048, 1024, g0)
        x0 = torch.randn(1, 2048, device=dev, generator=g0).to(torch.float16)
        op0 = lambda: torch.ops.binary_kernels.nanoquant_dyn_forward(x0, lin0.s_in, lin0.vt_bits, lin0.s_mid, lin0.u_bits,
                                                                     lin0.s_out, 128, 128, 2, 2, 1, 1, 8, 8)
        us_op0 = timed([op0] * 16, 64, 16) * 1e3
        rl0 = DecodeRunList(1, torch.float16, dev)
        lin0.add_to(rl0, x0)
        rl0.build()
        us_rl0 = timed([rl0.run] * 16, 64, 16) * 1e3
        unp = lambda bits, rows, cols: torch.from_numpy(oracle0.unpack_rows(bits.cpu().numpy(), (rows, cols), "half2")).float()
        vt0, u0 = unp(lin0.vt_bits, 1024, 2048), unp(lin0.u_bits, 2048, 1024)
        c0 = [t.float().cpu() for t in (x0, lin0.s_in, lin0.s_mid, lin0.s_out)]
        y_cpu0 = oracle0.torch_dense_forward(c0[0], vt0, u0, c0[1], c0[2], c0[3])
        err0 = oracle0.max_rel_err(op0().float().cpu().numpy(), y_cpu0.numpy())
        t_cpu0 = []
        for _ in range(30):
            t0_ = time.perf_counter()
            oracle0.torch_dense_forward(c0[0], vt0, u0, c0[1], c0[2], c0[3])
            t_cpu0.append(time.perf_counter() - t0_)
        t_cpu0.sort()
        b0 = gemv_bytes(2048, 2048, 1024, 1)
        extra["cfg0_2048x2048_r1024_batch1"] = {
            "gpu_us_operator": round(us_op0, 2), "gpu_us_run_list_one_launch": round(us_rl0, 2),
            "GBps_operator": round(b0 / (us_op0 * 1e-6) / 1e9, 1), "cpu_us_dense_fp32": round(t_cpu0[len(t_cpu0) // 2] * 1e6, 1),
            "cpu_threads": torch.get_num_threads(), "max_rel_err_gpu_vs_dense_definition": float("%.3e" % err0),
            "note": "warm weights (0.5 MB, cache resident), graph replays; the CPU figure is the reference's dense path "
                    "(two F.linear on unpacked +-1 fp32 factors)"}
        del rl0, lin0

        # ---- the module interface (NanoQuantLinear prepared for decode, one call per linear), by row count ----
        from nanoquant_amd.linear import NanoQuantLinear

        def decode_module(lin):
            mod = NanoQuantLinear(lin.n, lin.m, lin.rp, dtype=torch.float16, device=dev)
            for name in ("V", "U"):
                delattr(mod, name)
            mod.do_kernel_inference, mod.kernel_type, mod.dtype = True, "gemv", torch.float16
            mod.V_int8, mod.U_int8 = lin.vt_bits, lin.u_bits
            for name, t in (("scale_pre", lin.s_in), ("scale_mid", lin.s_mid), ("scale_post", lin.s_out)):
                setattr(mod, name, torch.nn.Parameter(t, requires_grad=False))
            mod.kernel_forward = torch.ops.binary_kernels.nanoquant_dyn_forward
            mod.kernel_kwargs = {}
            return mod

        mods = [[decode_module(lin) for lin in layer] for layer in layers]
        for layer in mods:
            for mod in layer:
                mod.mfma_from_rows = 3         # opt in to the few-token MFMA tiles from 3 rows on
                mod.prepare_mfma_route()       # set-up: otherwise the first call of 3 or more rows builds the tiles
        by_rows = {}
        with torch.no_grad():
            for rows in (1, 2, 4, 16):
                xs_m = {n: torch.randn(rows, n, device=dev).to(torch.float16) for n in (4096, 11008)}
                fns = [(lambda layer=layer: [mod(xs_m[mod.in_features]) for mod in layer]) for layer in mods]
                by_rows[str(rows)] = round(timed(fns, 2 * len(layers), len(layers)) * 1e3, 1)
        extra["module_forward_us_per_layer_by_rows"] = dict(
            by_rows, note="NanoQuantLinear.forward of 7 modules prepared with kernel_type='gemv', graph replays over the "
                          "rotating weight copies: one decode launch per linear up to 2 rows, the few-token MFMA tiles "
                          "(mfma_from_rows = 3, built once from the decode words) from 3 rows on")
        del mods
        # ---- prefill GEMM over the three distinct linear shapes of the layer ----
        # Timed as HIP graph replays: through Python the two-GEMM op costs more host time than GPU time.
        op = torch.ops.binary_kernels.marlin_nanoquant_forward
        g2 = torch.Generator(device=dev)
        g2.manual_seed(2)
        packed_by_shape = {}
        for (_, m, n) in LLAMA2_7B_LAYER[3:5] + LLAMA2_7B_LAYER[6:]:   # o (4096^2), gate, down
            r = nominal_rank(m, n)
            v = (torch.randint(0, 2, (n, r), device=dev, generator=g2, dtype=torch.int8) * 2 - 1)
            u = (torch.randint(0, 2, (r, m), device=dev, generator=g2, dtype=torch.int8) * 2 - 1)
            sc = lambda k: (torch.randn(k, device=dev, generator=g2).abs() * 0.02 + 1e-3).to(torch.float16)
            packed_by_shape[(m, n, r)] = packing.marlin_nanoquant_packer(v, u, sc(n), sc(r), sc(m))
            del v, u
        for tokens in (128, 512, 4096):
            gemm_lines = {}
            for (m, n, r), packed in packed_by_shape.items():
                x = torch.randn(tokens, n, device=dev, generator=g2).to(torch.float16)
                per_graph, replays = 10, 5
                g = capture_rotation([lambda: op(x, *packed)] * per_graph)
                g.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(replays):
                    g.replay()
                e1.record()
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / (per_graph * replays)
                tf = gemm_flops(m, n, r, tokens) / (us * 1e-6) / 1e12
                gemm_lines[f"{m}x{n}_r{r}"] = {"us": round(us, 2), "TFLOPs": round(tf, 2),
                                               "frac_of_f16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
                del g, x
            extra[f"prefill_{tokens}_tokens"] = gemm_lines
        # ---- the 7 linears of the layer sharing their launches (two per group of <= 16 terms) ----
        from nanoquant_amd import ops as nq_ops
        by_mn = {(m, n): (packed, r) for (m, n, r), packed in packed_by_shape.items()}
        group = [by_mn[(m, n)] for (_, m, n) in LLAMA2_7B_LAYER]
        for tokens in (16, 128, 512, 4096):
            xs_t = {n: torch.randn(tokens, n, device=dev, generator=g2).to(torch.float16) for n in (4096, 11008)}
            group_x = [xs_t[n] for (_, _, n) in LLAMA2_7B_LAYER]
            group_flops = sum(gemm_flops(m, n, by_mn[(m, n)][1], tokens) for (_, m, n) in LLAMA2_7B_LAYER)
            g = capture_rotation([lambda: nq_ops.gemm_group_forward(group_x, [pk for pk, _ in group])] * 5)
            g.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 25
            tf = group_flops / (us * 1e-6) / 1e12
            extra[f"prefill_{tokens}_tokens_layer_grouped"] = {
                "us_per_layer": round(us, 2), "TFLOPs": round(tf, 2), "frac_of_f16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                "note": "7 linears of the layer in two launches (nq_gemm_nanoquant_group); q,k,v,o share one weight copy here"}
            del g
            if tokens == 128:
                # the second headline metric (128-token GEMM TFLOP/s) as a roofline object of its own
                result["roofline_prefill"] = {
                    "bound": "mfma", "tokens": 128,
                    "kernel": "first GEMMs of the 7 linears: gemm_kwave_group_kernel<fp16> (few-token tiles); second GEMMs: "
                              "gemm_panel_kernel<fp16> (persistent 64-token x 256-row panels, two workgroups per CU); one launch each",
                    "achieved": round(tf, 2), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4), "flops_per_layer": int(group_flops),
                    "us_per_layer": round(us, 2), "traffic": MEASURED_PREFILL_TRAFFIC_BYTES}
            if tokens == 16:
                # the same 16 rows as extra.batch16, on the prefill kernels and with cold weights as there: every
                # linear of every rotation step reads its own copy of the packed tiles (args.copies x 7 clones)
                cold = [[tuple(t.clone() for t in pk) for pk, _ in group] for _ in range(args.copies)]
                g = capture_rotation([(lambda terms=terms: nq_ops.gemm_group_forward(group_x, terms)) for terms in cold])
                g.replay()
                torch.cuda.synchronize()
                e0.record()
                for _ in range(4):
                    g.replay()
                e1.record()
                torch.cuda.synchronize()
                us_cold = e0.elapsed_time(e1) * 1e3 / (4 * args.copies)
                extra["batch16_on_prefill_kernels"] = {
                    "us_per_layer": round(us_cold, 2), "GBps": round(layer_bytes(16) / (us_cold * 1e-6) / 1e9, 2),
                    "note": "16 rows through kernel_type='gemm' + grouped launches (two per layer), rotating weight copies "
                            "as in the decode legs; GB/s counts the decode path's algorithmic bytes"}
                del g, cold
            del xs_t, group_x
        # ---- cfg3: Qwen3-8B-like layer, every weight a sum of two terms (ranks 3:1, ~0.55 bpw), batch 1 ----
        qwen = (("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
                ("gate", 12288, 4096), ("up", 12288, 4096), ("down", 4096, 12288))

        def mixture_ranks(m, n):
            total = 0.55 * m * n / (m + n)
            return (max(32, int(round(0.75 * total / 32)) * 32), max(32, int(round(0.25 * total / 32)) * 32))

        gq = torch.Generator(device=dev)
        gq.manual_seed(4)
        q_copies = 26
        q_lists, q_bytes = [], 0.0
        xq = {n: torch.randn(1, n, device=dev, generator=gq).to(torch.float16) for n in (4096, 12288)}
        for c in range(q_copies):
            rl = DecodeRunList(1, torch.float16, dev)
            for (_, m, n) in qwen:
                r0, r1 = mixture_ranks(m, n)
                t0, t1 = SynthLinear(torch, dev, m, n, r0, gq), SynthLinear(torch, dev, m, n, r1, gq)
                i0 = t0.add_to(rl, xq[n], out_f32=True)
                t1.add_to(rl, xq[n], addend=rl.outputs[i0], y_from=i0)
                if c == 0:
                    q_bytes += gemv_bytes(m, n, r0, 1) + gemv_bytes(m, n, r1, 1)
            rl.build()
            q_lists.append(rl)
        ms_q = timed([rl.run for rl in q_lists], 4 * q_copies, q_copies)
        for rl in q_lists:
            if rl.status() != 0:
                raise RuntimeError("run list reported an expired dependency wait")
        extra["cfg3_qwen3_8b_two_term_layer_batch1"] = {
            "us_per_layer": round(ms_q * 1e3, 3), "GBps": round(q_bytes / (ms_q * 1e-3) / 1e9, 2),
            "note": "14 terms in one launch, second terms add onto the fp32 output of the first inside the kernel"}
        del q_lists

        # ---- cfg3 at 128 tokens: the 14 terms of the layer in shared launches, the two terms of a weight summed ----
        q_packed = {}
        for (_, m, n) in qwen:
            if (m, n) in q_packed:
                continue
            pair = []
            for r in mixture_ranks(m, n):
                v = (torch.randint(0, 2, (n, r), device=dev, generator=gq, dtype=torch.int8) * 2 - 1)
                u = (torch.randint(0, 2, (r, m), device=dev, generator=gq, dtype=torch.int8) * 2 - 1)
                sc = lambda k: (torch.randn(k, device=dev, generator=gq).abs() * 0.02 + 1e-3).to(torch.float16)
                pair.append(packing.marlin_nanoquant_packer(v, u, sc(n), sc(r), sc(m)))
                del v, u
            q_packed[(m, n)] = pair
        xq128 = {n: torch.randn(128, n, device=dev, generator=gq).to(torch.float16) for n in (4096, 12288)}
        q_groups = [q_packed[(m, n)] for (_, m, n) in qwen]
        q_xs = [xq128[n] for (_, m, n) in qwen]
        q_flops = sum(gemm_flops(m, n, r, 128) for (_, m, n) in qwen for r in mixture_ranks(m, n))

        def qwen_prefill():
            return nq_ops.gemm_group_sum_forward(q_xs, q_groups)

        g = capture_rotation([qwen_prefill] * 5)
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / 25
        tf = q_flops / (us * 1e-6) / 1e12
        extra["cfg3_qwen3_8b_two_term_layer_128_tokens"] = {
            "us_per_layer": round(us, 2), "TFLOPs": round(tf, 2), "frac_of_f16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
            "note": "14 terms in two grouped launches (first GEMMs, second GEMMs) plus one add over all second terms; "
                    "flops at the nominal ranks"}
        del g, q_packed, q_groups

        cfg4_leg(extra)
        result["extra"] = extra

        # ---- CPU baseline: the reference's dense path on this host (bounded sample) ----
        from oracle import nq_oracle as oracle

        torch.set_num_threads(os.cpu_count() or 1)
        cpu_terms = []
        gcpu = torch.Generator().manual_seed(3)
        for (_, m, n) in LLAMA2_7B_LAYER:
            r = nominal_rank(m, n)
            vt = (torch.randint(0, 2, (r, n), generator=gcpu) * 2 - 1).float()
            u = (torch.randint(0, 2, (m, r), generator=gcpu) * 2 - 1).float()
            sc = lambda k: torch.randn(k, generator=gcpu).abs() * 0.02 + 1e-3
            cpu_terms.append((torch.randn(1, n, generator=gcpu), vt, u, sc(n), sc(r), sc(m)))

        def cpu_pass():
            for (x, vt, u, s_in, s_mid, s_out) in cpu_terms:
                oracle.torch_dense_forward(x, vt, u, s_in, s_mid, s_out)

        for _ in range(3):
            cpu_pass()
        times = []
        t_end = time.perf_counter() + args.cpu_seconds
        while len(times) < 20 or (time.perf_counter() < t_end and len(times) < 200):
            t0 = time.perf_counter()
            cpu_pass()
            times.append(time.perf_counter() - t0)
            if time.perf_counter() > t_end + 20:
                break
        times.sort()
        med = times[len(times) // 2]
        # the reference module's default dtype is bf16 (modules/linear.py:27): same pass in bf16, fewer repeats
        bf_terms = [tuple(t.to(torch.bfloat16) for t in term) for term in cpu_terms]
        bf_times = []
        for _ in range(2):
            for (x, vt, u, s_in, s_mid, s_out) in bf_terms:
                oracle.torch_dense_forward(x, vt, u, s_in, s_mid, s_out)
        t_bf_end = time.perf_counter() + max(2.0, args.cpu_seconds / 4)
        while len(bf_times) < 5 or (time.perf_counter() < t_bf_end and len(bf_times) < 50):
            t0 = time.perf_counter()
            for (x, vt, u, s_in, s_mid, s_out) in bf_terms:
                oracle.torch_dense_forward(x, vt, u, s_in, s_mid, s_out)
            bf_times.append(time.perf_counter() - t0)
            if time.perf_counter() > t_bf_end + 20:
                break
        bf_times.sort()

        result["cpu_baseline"] = {
            "value": round(bytes1 / med / 1e9, 3),
            "unit": "GB/s",
            "us_per_layer": round(med * 1e6, 1),
            "us_per_layer_bf16": round(bf_times[len(bf_times) // 2] * 1e6, 1),
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "same 7-linear layer, batch 1, fp32 dense +-1 factors through two F.linear per linear "
                      "(the reference's CPU path), median of %d passes; GB/s counts the same algorithmic bytes" % len(times),
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
