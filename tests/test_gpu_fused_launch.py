"""Run lists whose input and output are bound at launch, and the module's one-launch decode path on top of them.
The reference's module spends two launches per decode call (src/nanoquant/modules/linear.py:121-130,
src/nanoquant/kernel/cuda/gemv_kernel.cu:340-425); the checks are against the dense definition and against the
same list with fixed tensors."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import DecodeRunList, NanoQuantLinear, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu


def _term(dev, m, n, r, seed):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    f = lambda a: torch.from_numpy(a).to(dev)
    ops = (f(s_in), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), f(s_mid),
           packing.binary_packer(torch.from_numpy(u), "half2").to(dev), f(s_out))
    return (vt, u, s_in, s_mid, s_out), ops


@pytest.mark.parametrize("batch", [1, 4, 8, 16])
def test_bound_tensors_change_from_launch_to_launch(dev, batch):
    m, n, r = 1376, 1056, 352
    npt, ops = _term(dev, m, n, r, seed=11)
    rl = DecodeRunList(batch, torch.float16, dev)
    rl.add(None, *ops, bind_y=True)
    rl.build()
    print(f"bound run list batch={batch}", flush=True)
    for rep in range(3):                                   # fresh tensors every time: nothing of the last call may stick
        x = oracle.synth_x(batch, n, 20 + rep)
        ref = oracle.layer_forward(x.astype(np.float64), *npt, dtype=np.float64)
        xt = torch.from_numpy(x).to(dev)
        y = torch.zeros((batch, m), dtype=torch.float16, device=dev)
        rl.run(x=xt, y=y)
        torch.cuda.synchronize()
        assert rl.status() == 0
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-3, rep
    # the same list with fixed tensors gives the same numbers as the last bound launch
    fixed = DecodeRunList(batch, torch.float16, dev)
    fixed.add(xt, *ops)
    y_fixed = fixed.run()[0]
    torch.cuda.synchronize()
    assert torch.allclose(y.float(), y_fixed.float(), rtol=2e-3, atol=1e-4 * float(y_fixed.float().abs().max()))


def test_bound_input_shared_by_three_projections(dev):
    # q, k, v of one attention block read the same activations; only one output can be left open
    n, batch = 1024, 2
    terms = [_term(dev, m, n, r, seed=40 + i) for i, (m, r) in enumerate([(1024, 512), (256, 128), (256, 160)])]
    rl = DecodeRunList(batch, torch.float16, dev)
    for i, (_, ops) in enumerate(terms):
        rl.add(None, *ops, bind_y=(i == 0))
    x = oracle.synth_x(batch, n, 44)
    y0 = torch.zeros((batch, 1024), dtype=torch.float16, device=dev)
    outs = rl.run(x=torch.from_numpy(x).to(dev), y=y0)
    torch.cuda.synchronize()
    assert rl.status() == 0 and outs[0] is None
    for (npt, _), y in zip(terms, [y0, outs[1], outs[2]]):
        ref = oracle.layer_forward(x.astype(np.float64), *npt, dtype=np.float64)
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 2e-3


def test_bound_list_refuses_what_it_cannot_run(dev):
    _, ops = _term(dev, 256, 512, 128, seed=50)
    _, ops2 = _term(dev, 256, 768, 128, seed=51)
    x = torch.zeros((1, 512), dtype=torch.float16, device=dev)
    rl = DecodeRunList(1, torch.float16, dev)
    rl.add(None, *ops, bind_y=True)
    y = torch.zeros((1, 256), dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError):
        rl.run()                                           # nothing bound
    with pytest.raises(RuntimeError):
        rl.run(x=x)                                        # output missing
    with pytest.raises(RuntimeError):
        rl.run(x=torch.zeros((1, 768), dtype=torch.float16, device=dev), y=y)
    with pytest.raises(RuntimeError):
        rl.run(x=x, y=torch.zeros((1, 256), dtype=torch.float32, device=dev))
    with pytest.raises(RuntimeError):
        rl.run(x=torch.zeros((1, 520), dtype=torch.float16, device=dev)[:, 4:516].reshape(1, 512), y=y)   # not 16-byte aligned
    two = DecodeRunList(1, torch.float16, dev)             # two open outputs would write the same tensor
    two.add(None, *ops, bind_y=True)
    two.add(None, *ops, bind_y=True)
    with pytest.raises(RuntimeError):
        two.build()
    mixed = DecodeRunList(1, torch.float16, dev)           # open inputs of different widths
    mixed.add(None, *ops)
    mixed.add(None, *ops2)
    with pytest.raises(RuntimeError):
        mixed.build()
    chained = DecodeRunList(1, torch.float16, dev)         # an open output cannot feed another entry
    first = chained.add(x, *ops, bind_y=True)
    _, ops3 = _term(dev, 128, 256, 64, seed=52)
    chained.add(torch.zeros((1, 256), dtype=torch.float16, device=dev), *ops3, x_from=first)
    with pytest.raises(RuntimeError):
        chained.build()
    with pytest.raises(RuntimeError):
        rl.add(None, *ops, x_from=0)                       # fed by an entry and left open at once
    fixed = DecodeRunList(1, torch.float16, dev)
    fixed.add(x, *ops)
    with pytest.raises(RuntimeError):
        fixed.run(x=x)                                     # nothing to bind


def test_graph_replay_of_a_bound_launch(dev):
    batch, m, n, r = 1, 2048, 1024, 512
    npt, ops = _term(dev, m, n, r, seed=60)
    rl = DecodeRunList(batch, torch.float16, dev)
    rl.add(None, *ops, bind_y=True)
    x = torch.from_numpy(oracle.synth_x(batch, n, 61)).to(dev)
    y = torch.zeros((batch, m), dtype=torch.float16, device=dev)
    rl.run(x=x, y=y)
    torch.cuda.synchronize()
    eager = y.clone()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        rl.run(x=x, y=y)
    for rep in range(3):
        x2 = oracle.synth_x(batch, n, 62 + rep)
        x.copy_(torch.from_numpy(x2).to(dev))              # the graph holds the pointers; new values go through them
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert rl.status() == 0
        ref = oracle.layer_forward(x2.astype(np.float64), *npt, dtype=np.float64)
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-3, rep
    assert not torch.equal(y, eager)


def _module(dev, m, n, r, seed, dtype, mid=True, bias=False):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    b = np.random.default_rng(seed).normal(0, 0.05, m).astype(np.float32) if bias else None
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid) if mid else None, f(s_out),
                                       bias=None if b is None else f(b), dtype=dtype).to(dev)
    if not mid:
        s_mid = np.ones_like(s_mid)
    return mod, (vt, u, s_in, s_mid, s_out), b


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 2, 4, 8, 16, 5])
def test_module_fused_launch_matches_the_op_path(dev, rows, dtype):
    m, n, r = 608, 1056, 288
    mod, term, _ = _module(dev, m, n, r, 70, dtype)
    mod._prepare_kernel("gemv", dtype)
    rnd = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype).float().numpy().astype(np.float64)
    x = oracle.synth_x(rows, n, 71)
    ref = oracle.layer_forward(rnd(x), term[0], term[1], rnd(term[2]), rnd(term[3]), rnd(term[4]), dtype=np.float64)
    xt = torch.from_numpy(x).to(dev).to(dtype)
    print(f"module fused rows={rows} {dtype}", flush=True)
    y_op = mod(xt)
    mod.fused_launch = True
    y_fused = mod(xt)
    y_again = mod(xt.clone().view(1, rows, n))             # 3-D input, the cached list, another input tensor
    torch.cuda.synchronize()
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-3
    assert y_fused.shape == (rows, m) and y_again.shape == (1, rows, m)
    assert oracle.max_rel_err(y_op.float().cpu().numpy(), ref) < tol
    assert oracle.max_rel_err(y_fused.float().cpu().numpy(), ref) < tol
    assert oracle.max_rel_err(y_again[0].float().cpu().numpy(), ref) < tol
    assert len(mod._fused_lists) == (0 if rows == 5 else 1)   # 5 rows: no list of that size, the op path serves it


def test_module_fused_launch_without_scale_mid_and_with_bias(dev):
    m, n, r, dtype = 512, 768, 160, torch.float16
    mod, term, bias = _module(dev, m, n, r, 80, dtype, mid=False, bias=True)
    mod._prepare_kernel("gemv", dtype)
    mod.fused_launch = True
    rnd = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype).float().numpy().astype(np.float64)
    for rows in (1, 8):
        x = oracle.synth_x(rows, n, 81 + rows)
        ref = oracle.layer_forward(rnd(x), term[0], term[1], rnd(term[2]), term[3].astype(np.float64), rnd(term[4]), dtype=np.float64)
        xt = torch.from_numpy(x).to(dev).to(dtype)
        mod.kernel_path_bias = False
        y0 = mod(xt)
        mod.kernel_path_bias = True
        y1 = mod(xt)
        torch.cuda.synchronize()
        assert oracle.max_rel_err(y0.float().cpu().numpy(), ref) < 2e-3, rows
        assert oracle.max_rel_err(y1.float().cpu().numpy(), ref + rnd(bias)[None, :]) < 2e-3, rows
