"""The benchmark configurations at their real shapes, through the product entry points.

cfg3: Qwen3-8B-like linears as sums of two binary low-rank terms (ranks 3:1, about 0.55 bpw), batch-1 decode
      and 128-token prefill.
cfg4: Llama-3-70B-shaped linears streamed through one run list at batch 1 and 8.

Oracle cost is kept down by checking all rows of the small shapes and a seeded sample of output rows of the
large ones (the first stage is always evaluated in full).  Size-independent properties cover the rest at
full size: run list == per-linear entry point, linearity in the scale vectors.
"""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import DecodeRunList, MixtureOfRankLinear, NanoQuantLinear, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu

# (out, in, rank of term 0, rank of term 1): 0.55 bpw split 3:1, rounded to whole words
QWEN3_8B = {"q": (4096, 4096, 832, 288), "k": (1024, 4096, 320, 128),
            "gate": (12288, 4096, 1248, 416), "down": (4096, 12288, 1248, 416)}


def _pack(dev, term):
    vt, u, s_in, s_mid, s_out = term
    f = lambda a: torch.from_numpy(a).to(dev)
    return (f(s_in), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), f(s_mid),
            packing.binary_packer(torch.from_numpy(u), "half2").to(dev), f(s_out))


def _sampled_ref(x, term, rows):
    """fp64 oracle output for the given output rows only (full first stage)."""
    vt, u, s_in, s_mid, s_out = term
    sub = (vt, u[rows], s_in, s_mid, s_out[rows])
    return oracle.layer_forward(x.astype(np.float64), *sub, dtype=np.float64)


@pytest.mark.parametrize("name", list(QWEN3_8B))
def test_cfg3_mixture_decode_batch1(dev, name):
    m, n, r0, r1 = QWEN3_8B[name]
    t0, t1 = oracle.synth_term(m, n, r0, 900), oracle.synth_term(m, n, r1, 901)
    x = oracle.synth_x(1, n, 902)
    rows = np.random.default_rng(5).choice(m, size=min(m, 512), replace=False)
    ref = _sampled_ref(x, t0, rows) + _sampled_ref(x, t1, rows)
    xt = torch.from_numpy(x).to(dev)
    print(f"cfg3 decode {name} m={m} n={n} r={r0}+{r1}", flush=True)
    # (1) the fused mixture entry point behind MixtureOfRankLinear
    from nanoquant_amd import ops
    y = ops.gemv_mixture_forward(xt, [_pack(dev, t0), _pack(dev, t1)])
    # (2) the run list: term 1 adds onto the fp32 output of term 0 inside the launch
    rl = DecodeRunList(1, torch.float16, dev)
    i0 = rl.add(xt, *_pack(dev, t0), out_f32=True)
    i1 = rl.add(xt, *_pack(dev, t1), addend=rl.outputs[i0], y_from=i0)
    y_rl = rl.run()[i1]
    torch.cuda.synchronize()
    assert rl.status() == 0
    scale = np.abs(ref).max()
    for got in (y, y_rl):
        err = np.abs(got.float().cpu().numpy()[:, rows] - ref).max() / scale
        assert err < 1e-3, (name, err)


@pytest.mark.parametrize("name", ["k", "q"])
def test_cfg3_mixture_prefill_128_tokens(dev, name):
    m, n, r0, r1 = QWEN3_8B[name]
    tokens = 128
    terms = [oracle.synth_term(m, n, r0, 910), oracle.synth_term(m, n, r1, 911)]
    x = oracle.synth_x(tokens, n, 912)
    ref = oracle.mixture_forward(x.astype(np.float64), terms, dtype=np.float64)
    mods = []
    for (vt, u, s_in, s_mid, s_out) in terms:
        f = lambda a: torch.from_numpy(a.astype(np.float32))
        mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid), f(s_out), dtype=torch.float16).to(dev)
        mods.append(mod)
    mix = MixtureOfRankLinear(mods)
    mix._prepare_kernel("gemm", torch.float16)
    print(f"cfg3 prefill {name} m={m} n={n} r={r0}+{r1} tokens={tokens}", flush=True)
    y = mix(torch.from_numpy(x).to(dev))
    torch.cuda.synchronize()
    assert y.shape == (tokens, m)
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2


@pytest.mark.parametrize("batch", [1, 8])
def test_cfg4_llama3_70b_shapes_in_one_run_list(dev, batch):
    # k/v 1024x8192, gate 28672x8192, down 8192x28672 at 1.0 bpw (q/o 8192^2 are covered by smaller squares)
    shapes = [(1024, 8192), (28672, 8192), (8192, 28672)]
    rl = DecodeRunList(batch, torch.float16, dev)
    cases = []
    for i, (m, n) in enumerate(shapes):
        r = oracle.nominal_rank(m, n)
        rp = (r + 31) // 32 * 32
        term = oracle.synth_term(m, n, rp, 920 + i)
        term[3][r:] = 0                           # padded rank: zero mid scale, as the bench does
        x = oracle.synth_x(batch, n, 930 + i)
        rows = np.random.default_rng(i).choice(m, size=256, replace=False)
        print(f"cfg4 B={batch} m={m} n={n} r={r} (padded {rp})", flush=True)
        ops_dev = _pack(dev, term)
        xt = torch.from_numpy(x).to(dev)
        rl.add(xt, *ops_dev)
        cases.append((rows, _sampled_ref(x, term, rows), xt, ops_dev))
    for rep in range(2):
        ys = rl.run()
        torch.cuda.synchronize()
        assert rl.status() == 0
        for (rows, ref, xt, ops_dev), y in zip(cases, ys):
            err = np.abs(y.float().cpu().numpy()[:, rows] - ref).max() / np.abs(ref).max()
            assert err < 1e-3, err
    # full-size property: every row agrees with the per-linear entry point (other arithmetic: 16-bit staging of x
    # and h there, fp8 pieces here; each is within 1e-3 of the exact result, both errors add up here)
    for (rows, ref, xt, ops_dev), y in zip(cases, ys):
        y_op = torch.ops.binary_kernels.nanoquant_dyn_forward(xt, *ops_dev, 128, 128, 2, 2, 1, 1, 8, 8)
        torch.cuda.synchronize()
        assert torch.allclose(y.float(), y_op.float(), rtol=2e-3, atol=1e-3 * float(np.abs(ref).max()))


def test_cfg1_full_size_linearity_in_output_scale(dev):
    # doubling s_out doubles y (a power of two, so exactly, up to the order in which the row sums were
    # accumulated: LDS float atomics make that order vary by an fp32 rounding); no oracle needed at any size
    m, n = 11008, 4096
    r = 3008
    term = oracle.synth_term(m, n, r, 940)
    ops_dev = list(_pack(dev, term))
    x = torch.from_numpy(oracle.synth_x(4, n, 941)).to(dev)
    rl = DecodeRunList(4, torch.float16, dev)
    rl.add(x, *ops_dev)
    ops2 = list(ops_dev)
    ops2[4] = ops_dev[4] * 2
    rl.add(x, *ops2)
    y1, y2 = rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    assert torch.allclose(y1.float() * 2, y2.float(), rtol=1e-3, atol=1e-4 * float(y2.float().abs().max()))
    assert (y1.float() * 2 == y2.float()).float().mean() > 0.9
