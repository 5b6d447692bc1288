"""Every workload that `bench.py` times, at its real shape, against the oracle.

The oracle is evaluated for a seeded sample of output rows (and, for the prefill cases, of tokens): every output
element is an independent function of the inputs, so a sample pins the kernels' indexing at full size while the
fp64 reference stays cheap (the first stage is always evaluated in full for the sampled tokens).  Definition
matched: src/nanoquant/modules/linear.py:248-257 of the reference.

cfg1: the 7 linears of a Llama-2-7B layer as ONE run list in tile order, ranks 2048 / 2985 padded to 3008 with a zero
      mid scale, batch 1, 4 and 16 -- the list bench.py builds.
cfg2: the three Llama-2-7B shapes at 512 tokens through the reference's op and through the grouped launches; one
      4096-token case.
cfg3: gate / down of the Qwen3-8B-like two-term layer at 128 tokens and the 14-term grouped sum.
cfg4: q/o 8192 x 8192 r4096 at batch 1 and 8.
"""
import functools

import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import DecodeRunList, ops, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu

LLAMA2_7B_LAYER = (("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
                   ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008))


@functools.lru_cache(maxsize=None)
def _term(m, n, r, seed):
    return oracle.synth_term(m, n, r, seed)


def _sampled(x, term, rows, tokens=None):
    """fp64 layer output for the sampled tokens (all when None) and output rows."""
    vt, u, s_in, s_mid, s_out = term
    xs = x if tokens is None else x[tokens]
    return oracle.layer_forward(xs.astype(np.float64), vt, u[rows], s_in, s_mid, s_out[rows], dtype=np.float64)


def _err(got, ref):
    return float(np.abs(got - ref).max() / np.abs(ref).max())


# ---- cfg1 --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch", [1, 4, 16])
def test_cfg1_layer_run_list_as_benchmarked(dev, batch):
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    rl = DecodeRunList(batch, torch.float16, dev)
    cases = []
    for i, (name, m, n) in enumerate(LLAMA2_7B_LAYER):
        r = oracle.nominal_rank(m, n)
        vt, u, s_in, s_mid, s_out = _term(m, n, r, 1000 + (i if i >= 4 else 0) * 10 + i)
        vt_p, u_p, mid_p = oracle.pad_rank(vt, u, s_mid, 32)           # 2985 -> 3008, +1 signs, zero mid scale
        x = oracle.synth_x(batch, n, 1100 + i)
        vt_bits = packing.binary_packer(torch.from_numpy(vt_p), "half2")
        u_bits = packing.binary_packer(torch.from_numpy(u_p), "half2")
        tiled = True                                                   # tile order, as in bench.py
        if tiled:
            vt_dev, u_dev = packing.tile_words(vt_bits.to(dev)), packing.tile_words(u_bits.to(dev))
        else:
            vt_dev, u_dev = vt_bits.to(dev), u_bits.to(dev)
        rl.add(f(x), f(s_in), vt_dev, f(mid_p), u_dev, f(s_out), tiled=tiled)
        rows = np.random.default_rng(i).choice(m, size=384, replace=False)
        cases.append((name, rows, _sampled(x, (vt, u, s_in, s_mid, s_out), rows)))
    print(f"cfg1 run list, 7 linears, batch {batch}", flush=True)
    for rep in range(2):                                               # the second launch reuses the counters
        ys = rl.run()
        torch.cuda.synchronize()
        assert rl.status() == 0
        for (name, rows, ref), y in zip(cases, ys):
            got = y.float().cpu().numpy()[:, rows]
            e, ee = _err(got, ref), oracle.elementwise_err(got, ref)
            if rep == 0:
                print(f"  {name}: max_rel_err {e:.2e}, element-wise (floor 0.1 rms) {ee:.2e}", flush=True)
            assert e < 1e-3, (name, batch, rep, e)
            # fp16 outputs cost 2^-11 of the element by themselves; the 16-bit arithmetic (more than 4 rows, and a list
            # as short as this one at 4 rows) also rounds x * s_in and the intermediate vector to fp16, as the
            # reference's kernels do
            assert ee < (5e-3 if batch <= 2 else 5e-2), (name, batch, rep, ee)


# ---- cfg2 --------------------------------------------------------------------------------------------
def _prefill_case(dev, m, n, seed, tokens):
    r = oracle.nominal_rank(m, n)
    term = _term(m, n, r, seed)
    vt, u, s_in, s_mid, s_out = term
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    packed = packing.marlin_nanoquant_packer(f(vt).T.contiguous(), f(u).T.contiguous(), f(s_in), f(s_mid), f(s_out))
    x = oracle.synth_x(tokens, n, seed + 1)
    rng = np.random.default_rng(seed)
    tok = np.sort(rng.choice(tokens, size=min(tokens, 48), replace=False))
    tok[0], tok[-1] = 0, tokens - 1                                    # first and last token always
    rows = rng.choice(m, size=512, replace=False)
    return packed, f(x), tok, rows, _sampled(x, term, rows, tok)


@pytest.mark.parametrize("name,m,n", [LLAMA2_7B_LAYER[0], LLAMA2_7B_LAYER[4], LLAMA2_7B_LAYER[6]])
def test_cfg2_prefill_512_tokens_single_op(dev, name, m, n):
    packed, x, tok, rows, ref = _prefill_case(dev, m, n, 1200 + m // 64 + n // 1000, 512)
    print(f"cfg2 op {name} {m}x{n} 512 tokens", flush=True)
    y = torch.ops.binary_kernels.marlin_nanoquant_forward(x, *packed)
    torch.cuda.synchronize()
    assert y.shape == (512, m)
    e = _err(y.float().cpu().numpy()[np.ix_(tok, rows)], ref)
    assert e < 1e-2, e


@pytest.mark.parametrize("tokens", [128, 512])
def test_cfg2_prefill_layer_grouped(dev, tokens):
    cases = {}
    for (name, m, n) in (LLAMA2_7B_LAYER[0], LLAMA2_7B_LAYER[4], LLAMA2_7B_LAYER[6]):
        cases[(m, n)] = _prefill_case(dev, m, n, 1300 + m // 64 + n // 1000, tokens)
    xs = [cases[(m, n)][1] for (_, m, n) in LLAMA2_7B_LAYER]           # q, k, v, o share one weight set (as bench.py)
    terms = [cases[(m, n)][0] for (_, m, n) in LLAMA2_7B_LAYER]
    print(f"cfg2 grouped layer, 7 linears, {tokens} tokens", flush=True)
    ys = ops.gemm_group_forward(xs, terms)
    torch.cuda.synchronize()
    for (name, m, n), y in zip(LLAMA2_7B_LAYER, ys):
        _, _, tok, rows, ref = cases[(m, n)]
        e = _err(y.float().cpu().numpy()[np.ix_(tok, rows)], ref)
        assert e < 1e-2, (name, e)


def test_cfg2_prefill_4096_tokens(dev):
    m, n = 11008, 4096
    packed, x, tok, rows, ref = _prefill_case(dev, m, n, 1400, 4096)
    print("cfg2 op gate 11008x4096 4096 tokens", flush=True)
    y = torch.ops.binary_kernels.marlin_nanoquant_forward(x, *packed)
    torch.cuda.synchronize()
    e = _err(y.float().cpu().numpy()[np.ix_(tok, rows)], ref)
    assert e < 1e-2, e


# ---- cfg3 --------------------------------------------------------------------------------------------
QWEN = (("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
        ("gate", 12288, 4096), ("up", 12288, 4096), ("down", 4096, 12288))


def _mixture_ranks(m, n):
    total = 0.55 * m * n / (m + n)
    return (max(32, int(round(0.75 * total / 32)) * 32), max(32, int(round(0.25 * total / 32)) * 32))


def test_cfg3_fourteen_term_grouped_sum_128_tokens(dev):
    tokens = 128
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    by_shape = {}
    for (name, m, n) in QWEN:
        if (m, n) in by_shape:
            continue
        terms = [_term(m, n, r, 1500 + m // 128 + 7 * t) for t, r in enumerate(_mixture_ranks(m, n))]
        packed = [packing.marlin_nanoquant_packer(f(vt).T.contiguous(), f(u).T.contiguous(), f(s_in), f(s_mid), f(s_out))
                  for (vt, u, s_in, s_mid, s_out) in terms]
        x = oracle.synth_x(tokens, n, 1600 + m // 128)
        rng = np.random.default_rng(m)
        tok = np.sort(rng.choice(tokens, size=32, replace=False))
        rows = rng.choice(m, size=256, replace=False)
        ref = sum(_sampled(x, t, rows, tok) for t in terms)
        by_shape[(m, n)] = (packed, f(x), tok, rows, ref)
    print("cfg3 14 terms grouped, 128 tokens", flush=True)
    ys = ops.gemm_group_sum_forward([by_shape[(m, n)][1] for (_, m, n) in QWEN], [by_shape[(m, n)][0] for (_, m, n) in QWEN])
    torch.cuda.synchronize()
    for (name, m, n), y in zip(QWEN, ys):
        _, _, tok, rows, ref = by_shape[(m, n)]
        assert y.shape == (tokens, m)
        e = _err(y.float().cpu().numpy()[np.ix_(tok, rows)], ref)
        assert e < 1e-2, (name, e)


# ---- cfg4 --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch", [1, 8])
def test_cfg4_q_o_8192_square(dev, batch):
    m = n = 8192
    r = oracle.nominal_rank(m, n)
    assert r == 4096
    term = _term(m, n, r, 1700)
    vt, u, s_in, s_mid, s_out = term
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = oracle.synth_x(batch, n, 1701)
    rows = np.random.default_rng(17).choice(m, size=384, replace=False)
    ref = _sampled(x, term, rows)
    vt_bits = packing.binary_packer(torch.from_numpy(vt), "half2").to(dev)
    u_bits = packing.binary_packer(torch.from_numpy(u), "half2").to(dev)
    print(f"cfg4 q/o 8192x8192 r4096 batch {batch}", flush=True)
    y_op = torch.ops.binary_kernels.nanoquant_dyn_forward(f(x), f(s_in), vt_bits, f(s_mid), u_bits, f(s_out), 128, 128, 2, 2,
                                                          1, 1, 8, 8)
    rl = DecodeRunList(batch, torch.float16, dev)
    tiled = batch <= 4
    if tiled:
        rl.add(f(x), f(s_in), packing.tile_words(vt_bits), f(s_mid), packing.tile_words(u_bits), f(s_out), tiled=True)
    else:
        rl.add(f(x), f(s_in), vt_bits, f(s_mid), u_bits, f(s_out))
    y_rl = rl.run()[0]
    torch.cuda.synchronize()
    assert rl.status() == 0
    for got in (y_op, y_rl):
        e = _err(got.float().cpu().numpy()[:, rows], ref)
        assert e < 1e-3, e


@pytest.mark.parametrize("batch", [1, 8])
def test_cfg4_full_stack_one_launch(dev, batch):
    """The 560 linears of the Llama-3-70B-shaped stack (8.6 GB of random words generated on the device, as bench.py
    does) in ONE run-list launch at batch 1 and 8.  No oracle fits this size; the property checked is that sampled linears
    of the stack (first, middle, last layer; every shape) equal the per-linear operator on the same words, which the
    tests above and in test_gpu_configs.py hold against the oracle at these shapes."""
    shapes = ((8192, 8192), (1024, 8192), (1024, 8192), (8192, 8192), (28672, 8192), (28672, 8192), (8192, 28672))
    gen = torch.Generator(device=dev)
    gen.manual_seed(70)
    i32 = torch.iinfo(torch.int32)
    sc = lambda k: (torch.randn(k, device=dev, generator=gen).abs() * 0.02 + 1e-3).to(torch.float16)
    xs = {n: torch.randn(batch, n, device=dev, generator=gen).to(torch.float16) for n in (8192, 28672)}
    rl = DecodeRunList(batch, torch.float16, dev)
    keep = {}
    layers = 80
    for layer in range(layers):
        for j, (m, n) in enumerate(shapes):
            r = oracle.nominal_rank(m, n)
            rp = (r + 31) // 32 * 32
            vt = torch.randint(i32.min, i32.max, (rp, n // 32), dtype=torch.int32, device=dev, generator=gen)
            u = torch.randint(i32.min, i32.max, (m, rp // 32), dtype=torch.int32, device=dev, generator=gen)
            s_in, s_mid, s_out = sc(n), sc(rp), sc(m)
            s_mid[r:] = 0
            idx = rl.add(xs[n], s_in, packing.tile_words(vt), s_mid, packing.tile_words(u), s_out, tiled=True)
            if layer in (0, 41, layers - 1):
                keep[idx] = (xs[n], s_in, vt, s_mid, u, s_out)
            else:
                del vt, u
    print(f"cfg4 full stack: {layers * len(shapes)} linears in one launch, batch {batch}", flush=True)
    ys = rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    for idx, (x, s_in, vt, s_mid, u, s_out) in keep.items():
        y_op = torch.ops.binary_kernels.nanoquant_dyn_forward(x, s_in, vt, s_mid, u, s_out, 128, 128, 2, 2, 1, 1, 8, 8)
        torch.cuda.synchronize()
        scale = float(y_op.float().abs().max())
        # batch 8 runs on 16-bit operands in the run list (x * s_in and h rounded to fp16, as the operator does too)
        tol = 2e-3 if batch == 1 else 4e-3
        assert torch.allclose(ys[idx].float(), y_op.float(), rtol=tol, atol=tol * scale), (idx, batch)
