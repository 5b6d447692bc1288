"""Run-list decode path (one persistent launch over many linears) against the oracle and against
the per-linear entry point."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import DecodeRunList, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu
TIGHT = 1e-3   # fp16, ranks >= 256: the fp32-accumulate budget (max|y-y_ref| / max|y_ref|)


def _term(dev, m, n, r, seed):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    f = lambda a: torch.from_numpy(a).to(dev)
    ops = (f(s_in), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), f(s_mid),
           packing.binary_packer(torch.from_numpy(u), "half2").to(dev), f(s_out))
    return (vt, u, s_in, s_mid, s_out), ops


@pytest.mark.parametrize("batch", [1, 4, 16])
@pytest.mark.parametrize("interleave", [1, 2, 3])
def test_independent_linears(dev, batch, interleave):
    shapes = [(512, 1024, 256), (1376, 512, 384), (512, 1376, 352), (96, 160, 64), (2048, 2048, 1024)]
    rl = DecodeRunList(batch, torch.float16, dev, interleave=interleave)
    refs = []
    for i, (m, n, r) in enumerate(shapes):
        npt, ops = _term(dev, m, n, r, seed=100 + i)
        x = oracle.synth_x(batch, n, 100 + i)
        rl.add(torch.from_numpy(x).to(dev), *ops)
        refs.append(oracle.layer_forward(x.astype(np.float64), *npt, dtype=np.float64))
    print(f"runlist independent B={batch} interleave={interleave}", flush=True)
    for rep in range(3):                       # repeated runs: the counters must come back to zero
        for y in rl.outputs:
            y.zero_()
        ys = rl.run()
        torch.cuda.synchronize()
        assert rl.status() == 0
        for (m, n, r), y, ref in zip(shapes, ys, refs):
            err = oracle.max_rel_err(y.float().cpu().numpy(), ref)
            assert err < (TIGHT if r >= 256 else 1e-2), (rep, m, n, r, err)


def test_matches_per_linear_entry_point(dev):
    # different arithmetic (the run list stages fp8 pieces of the input, the per-linear kernel 16-bit values)
    # and different summation trees: agreement far below one fp16 ulp of the output for most elements
    m, n, r, batch = 1024, 4096, 512, 2
    npt, ops = _term(dev, m, n, r, seed=7)
    x = torch.from_numpy(oracle.synth_x(batch, n, 7)).to(dev)
    rl = DecodeRunList(batch, torch.float16, dev)
    rl.add(x, *ops)
    y_rl = rl.run()[0].float()
    y_op = torch.ops.binary_kernels.nanoquant_dyn_forward(x, *ops, 128, 128, 2, 2, 1, 1, 8, 8).float()
    torch.cuda.synchronize()
    assert torch.allclose(y_rl, y_op, rtol=2e-3, atol=2e-4 * float(y_op.abs().max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 2])
def test_small_batches_compute_exactly_on_the_fp8_pieces(dev, batch, dtype):
    # Up to batch 4 the kernel multiplies the signs with three fp8 pieces of x * s_in (resp. h * s_mid), every block of
    # 128 columns scaled by its own largest magnitude.  Restating that staging in the oracle predicts the output ten times
    # closer than the 1e-3 budget of the dense definition: a missing or misplaced piece (7e-4), a wrong column,
    # scale or class weight (O(1)) cannot hide in the tolerance.  What remains (1e-5 .. 5e-5 measured) is the
    # instruction's own 128-term sum, which keeps 13 bits below its largest product (2^5 + 2^-9 gives 2^5).
    m, n, r = 768, 1504, 416                       # ragged: 47 and 13 words per row
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 77)
    x = oracle.synth_x(batch, n, 78)
    to = lambda a: torch.from_numpy(a).to(dev).to(dtype)
    xd, sd_in, sd_mid, sd_out = to(x), to(s_in), to(s_mid), to(s_out)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)

    def stage(v, signs):
        # the kernel multiplies the signs with the staged pieces (the total it adds back for the classes that ride
        # as 0 / 1 weights is the total of the pieces, not of the exact input)
        return oracle.staged_input(v) @ signs.T.astype(np.float64)

    h = stage(f64(xd) * f64(sd_in)[None, :], vt).astype(np.float32).astype(np.float64)   # h is stored as fp32
    ref = stage(h * f64(sd_mid)[None, :], u) * f64(sd_out)[None, :]
    rl = DecodeRunList(batch, dtype, dev)
    i = rl.add(xd, sd_in, packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), sd_mid,
               packing.binary_packer(torch.from_numpy(u), "half2").to(dev), sd_out, out_f32=True)
    y = rl.run()[i]
    torch.cuda.synchronize()
    assert rl.status() == 0 and y.dtype == torch.float32
    err = np.abs(y.cpu().numpy() - ref).max() / np.abs(ref).max()
    print(f"exact-staging check batch={batch} {dtype}: {err:.3g}", flush=True)
    assert err < 1e-4, err
    # and the dense definition within the layer's budget
    dense = oracle.layer_forward(f64(xd), vt, u, f64(sd_in), f64(sd_mid), f64(sd_out), dtype=np.float64)
    assert np.abs(y.cpu().numpy() - dense).max() / np.abs(dense).max() < 1e-3


def test_chained_linears_depend_on_each_other(dev):
    # y of linear i is x of linear i+1: the in-kernel dependency counters order them
    dims = [768, 512, 1024, 256]
    batch = 2
    rl = DecodeRunList(batch, torch.float16, dev, interleave=3)
    x0 = oracle.synth_x(batch, dims[0], 3)
    cur = torch.from_numpy(x0).to(dev)
    ref = x0.astype(np.float64)
    for i in range(len(dims) - 1):
        n, m = dims[i], dims[i + 1]
        npt, ops = _term(dev, m, n, 256, seed=40 + i)
        # big scales so that values stay O(1) through the chain
        scale_up = torch.tensor(8.0, dtype=torch.float16, device=dev)
        ops = (ops[0] * scale_up, ops[1], ops[2] * scale_up, ops[3], ops[4] * scale_up)
        npt = (npt[0], npt[1], (ops[0].float().cpu().numpy()), ops[2].float().cpu().numpy(), ops[4].float().cpu().numpy())
        idx = rl.add(cur, *ops, x_from=i - 1)
        cur = rl.outputs[idx]
        ref = oracle.layer_forward(ref, *npt, dtype=np.float64)
        ref = ref.astype(np.float16).astype(np.float64)     # y is stored as fp16 between linears
    for rep in range(2):
        ys = rl.run()
        torch.cuda.synchronize()
        assert rl.status() == 0
        err = oracle.max_rel_err(ys[-1].float().cpu().numpy(), ref)
        assert err < 5e-3, err


@pytest.mark.parametrize("dtype,tiled", [(torch.float16, False), (torch.float16, True), (torch.bfloat16, True)])
def test_mixture_through_addend(dev, dtype, tiled):
    # two terms of one output at batch 4: the second adds onto the fp32 output of the first inside the launch and adds
    # a bias.  fp16: a short list, 16-bit arithmetic; bf16 in tile order: fp4 x fp8 arithmetic, wavefronts own row pairs.
    m, n, batch = 512, 1024, 4
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    words = lambda w: packing.binary_packer(torch.from_numpy(w), "half2").to(dev)
    order = (lambda w: packing.tile_words(w)) if tiled else (lambda w: w)
    xt = to(oracle.synth_x(batch, n, 5))
    terms, ops = [], []
    for r, seed in ((320, 60), (128, 61)):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
        sc = (to(s_in), to(s_mid), to(s_out))
        terms.append((vt, u, f64(sc[0]), f64(sc[1]), f64(sc[2])))
        ops.append((sc[0], order(words(vt)), sc[1], order(words(u)), sc[2]))
    bias = to(oracle.synth_x(1, m, 62)[0] * 0.01)
    rl = DecodeRunList(batch, dtype, dev, interleave=2)
    i0 = rl.add(xt, *ops[0], out_f32=True, tiled=tiled)
    i1 = rl.add(xt, *ops[1], addend=rl.outputs[i0], y_from=i0, bias=bias, tiled=tiled)
    y = rl.run()[i1]
    torch.cuda.synchronize()
    assert rl.status() == 0
    print(f"mixture {dtype} tiled={tiled}: plan flags {rl._plan.bound:#x}", flush=True)
    ref = oracle.mixture_forward(f64(xt), terms, dtype=np.float64) + f64(bias)[None, :]
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < (1e-2 if dtype == torch.bfloat16 else TIGHT)


def _weight_of_terms(dev, rl, dtype, batch, m, n, ranks, seed, tiled, links=None, x=None, x_from=-1):
    """Adds one weight = sum of len(ranks) terms to rl; term t adds onto the result of term links[t] (default: the one
    before it).  Returns (index of the last term, [per-term fp64 references], x as fp64)."""
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    words = lambda w: packing.binary_packer(torch.from_numpy(w), "half2").to(dev)
    order = (lambda w: packing.tile_words(w)) if tiled else (lambda w: w)
    xt = to(oracle.synth_x(batch, n, seed)) if x is None else x
    idx, refs = [], []
    for t, r in enumerate(ranks):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed + 1 + t)
        vt_p, u_p, mid_p = oracle.pad_rank(vt, u, s_mid, 32)
        sc = (to(s_in), to(mid_p), to(s_out))
        last = t == len(ranks) - 1
        kw = dict(tiled=tiled, out_f32=not last)
        if t == 0:
            kw["x_from"] = x_from
        else:
            src = idx[t - 1 if links is None else links[t]]
            kw.update(addend=rl.outputs[src], y_from=src)
        idx.append(rl.add(xt, sc[0], order(words(vt_p)), sc[1], order(words(u_p)), sc[2], **kw))
        refs.append(oracle.layer_forward(f64(xt), vt, u, f64(sc[0]), f64(to(s_mid)), f64(sc[2]), dtype=np.float64))
    return idx, refs, f64(xt)


@pytest.mark.parametrize("batch,dtype,tiled", [(1, torch.float16, True), (1, torch.float16, False), (4, torch.bfloat16, True),
                                               (4, torch.float16, False), (16, torch.float16, True), (8, torch.bfloat16, False)])
def test_terms_that_add_onto_the_same_rows(dev, batch, dtype, tiled):
    # Three terms of one weight in a chain, and a weight whose third term adds onto the first one's result: all second
    # stages share one phase, each workgroup runs the terms of its rows one behind the other.  A weight whose second
    # term is fed by another linear of the list cannot do that (its input is ready too late) and waits for the whole
    # first term instead.
    rl = DecodeRunList(batch, dtype, dev)
    ia, ra, _ = _weight_of_terms(dev, rl, dtype, batch, 1376, 1024, (320, 96, 64), 700, tiled)
    ib, rb, _ = _weight_of_terms(dev, rl, dtype, batch, 512, 2048, (256, 128, 40), 710, tiled, links=[None, 0, 0])
    ys = rl.run()
    assert rl._plan.nphases == 2, rl._plan.nphases
    torch.cuda.synchronize()
    assert rl.status() == 0
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-3
    print(f"families B={batch} {dtype} tiled={tiled}: plan flags {rl._plan.bound:#x}", flush=True)
    for rep in range(3):
        if rep:
            for y in rl.outputs:
                y.zero_()
            ys = rl.run()
            torch.cuda.synchronize()
            assert rl.status() == 0
        assert oracle.max_rel_err(ys[ia[2]].float().cpu().numpy(), ra[0] + ra[1] + ra[2]) < tol
        assert oracle.max_rel_err(ys[ia[1]].cpu().numpy(), ra[0] + ra[1]) < tol          # fp32 partial sums
        assert oracle.max_rel_err(ys[ib[1]].cpu().numpy(), rb[0] + rb[1]) < tol
        assert oracle.max_rel_err(ys[ib[2]].float().cpu().numpy(), rb[0] + rb[2]) < tol   # onto the first term, not the second

    # second term fed by an earlier linear's output: one phase later than the first term's second stage
    rl2 = DecodeRunList(batch, dtype, dev)
    i0, r0, _ = _weight_of_terms(dev, rl2, dtype, batch, 1024, 512, (128,), 720, tiled)
    y0 = torch.from_numpy(r0[0]).to(dtype).to(dev)
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    words = lambda w: packing.binary_packer(torch.from_numpy(w), "half2").to(dev)
    order = (lambda w: packing.tile_words(w)) if tiled else (lambda w: w)
    xa = to(oracle.synth_x(batch, 1024, 730))
    parts = []
    for t, (r, xin, kw) in enumerate(((256, xa, dict(out_f32=True)),
                                      (96, rl2.outputs[i0[0]], dict(x_from=i0[0])))):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(384, 1024, r, 731 + t)
        sc = (to(s_in), to(s_mid), to(s_out))
        if t == 1:
            kw.update(addend=rl2.outputs[first], y_from=first)
        k = rl2.add(xin, sc[0], order(words(vt)), sc[1], order(words(u)), sc[2], tiled=tiled, **kw)
        if t == 0:
            first = k
        parts.append(oracle.layer_forward(f64(xa) if t == 0 else f64(y0), vt, u, f64(sc[0]), f64(sc[1]), f64(sc[2]),
                                          dtype=np.float64))
    ys2 = rl2.run()
    torch.cuda.synchronize()
    assert rl2.status() == 0
    assert rl2._plan.nphases == 4, rl2._plan.nphases
    assert oracle.max_rel_err(ys2[k].float().cpu().numpy(), parts[0] + parts[1]) < (2e-2 if dtype == torch.bfloat16 else 5e-3)


@pytest.mark.parametrize("batch,dtype", [(1, torch.float16), (4, torch.float16), (16, torch.bfloat16)])
def test_many_weights_of_two_and_three_terms(dev, batch, dtype):
    # more families in the phase of the second stages than half the workgroups: the phase is cut by cost, a
    # workgroup's share may begin and end inside a family, and every piece carries all terms of its rows
    rng = np.random.default_rng(77 + batch)
    rl = DecodeRunList(batch, dtype, dev)
    want = []
    for w in range(300):
        m = int(rng.choice([64, 96, 160, 352]))
        n = int(rng.choice([128, 256]))
        ranks = tuple(int(v) for v in rng.choice([32, 64, 96], size=int(rng.integers(2, 4))))
        idx, refs, _ = _weight_of_terms(dev, rl, dtype, batch, m, n, ranks, 9000 + 10 * w, True)
        want.append((idx[-1], sum(refs)))
    ys = rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    assert rl._plan.nphases == 2
    print(f"many families B={batch} {dtype}: workgroups {rl._plan.workgroups} plan flags {rl._plan.bound:#x}", flush=True)
    for rep in range(2):
        if rep:
            ys = rl.run()
            torch.cuda.synchronize()
            assert rl.status() == 0
        worst = max(oracle.max_rel_err(ys[i].float().cpu().numpy(), ref) for i, ref in want)
        assert worst < (2e-2 if dtype == torch.bfloat16 else 1e-2), worst


@pytest.mark.parametrize("batch", [1, 8, 16])
def test_bf16_and_ragged_shapes(dev, batch):
    # ranks 70 and 2985 and 4100 columns: intermediate rows that allow no 16-byte loads (element-wise staging at every
    # batch size), inputs that end inside a unit, row counts that end inside a 16-row group
    rl = DecodeRunList(batch, torch.bfloat16, dev)
    refs = []
    for i, (m, n, r) in enumerate([(100, 1000, 70), (33, 4100, 2985), (300, 96, 32)]):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 200 + i)
        x = oracle.synth_x(batch, n, 200 + i)
        bf = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16)
        xt, si, sm, so = bf(x), bf(s_in), bf(s_mid), bf(s_out)
        rl.add(xt.to(dev), si.to(dev), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), sm.to(dev),
               packing.binary_packer(torch.from_numpy(u), "half2").to(dev), so.to(dev))
        refs.append(oracle.layer_forward(xt.float().numpy(), vt, u, si.float().numpy(), sm.float().numpy(),
                                         so.float().numpy(), dtype=np.float64))
    ys = rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    for y, ref in zip(ys, refs):
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < (1e-2 if batch == 1 else 2e-2)   # bf16 staging from 8 rows on


@pytest.mark.parametrize("batch,dtype,tiled", [(1, torch.float16, False), (4, torch.bfloat16, True), (4, torch.float16, True),
                                               (16, torch.float16, True)])
def test_graph_replay_of_a_run_list(dev, batch, dtype, tiled):
    # the launch allocates nothing and can be replayed; replays must equal the eager result.  Batch 4: bf16 in tile order
    # runs the kernel whose wavefronts take row pairs from a counter in LDS, the short fp16 list the 16-bit arithmetic.
    rl = DecodeRunList(batch, dtype, dev, interleave=2)
    xs = []
    for i, (m, n, r) in enumerate([(1024, 1024, 512), (1024, 2048, 512), (2048, 1024, 512)]):
        _, ops = _term(dev, m, n, r, seed=300 + i)
        ops = tuple(o.to(dtype) if o.dtype == torch.float16 else (packing.tile_words(o) if tiled else o) for o in ops)
        x = torch.from_numpy(oracle.synth_x(batch, n, 300 + i)).to(dev).to(dtype)
        xs.append(x)
        rl.add(x, *ops, tiled=tiled)
    eager = [y.clone() for y in rl.run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        rl.run()
    for rep in range(4):
        for y in rl.outputs:
            y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert rl.status() == 0
        for y, e in zip(rl.outputs, eager):
            # row sums are finished with LDS float atomics whose order varies from run to run: equal up to an
            # fp32 rounding of the sum, i.e. at most one fp16 ulp of the output here and there
            assert torch.allclose(y.float(), e.float(), rtol=2e-3, atol=1e-4 * float(e.float().abs().max())), rep
            assert (y == e).float().mean() > 0.9, rep


@pytest.mark.parametrize("batch", [2, 16])
def test_bf16_batches_on_the_mfma_path(dev, batch):
    # bf16 keeps +-1 weight operands on the MFMA units (no single-bit trick): cover it with ragged ranks too
    rl = DecodeRunList(batch, torch.bfloat16, dev)
    refs = []
    for i, (m, n, r) in enumerate([(512, 1024, 256), (200, 4096, 736), (1376, 512, 96)]):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 400 + i)
        x = oracle.synth_x(batch, n, 400 + i)
        bf = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16)
        xt, si, sm, so = bf(x), bf(s_in), bf(s_mid), bf(s_out)
        rl.add(xt.to(dev), si.to(dev), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), sm.to(dev),
               packing.binary_packer(torch.from_numpy(u), "half2").to(dev), so.to(dev))
        refs.append(oracle.layer_forward(xt.float().numpy(), vt, u, si.float().numpy(), sm.float().numpy(),
                                         so.float().numpy(), dtype=np.float64))
    print(f"bf16 run list batch={batch}", flush=True)
    ys = rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    for y, ref in zip(ys, refs):
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2


@pytest.mark.parametrize("rows,words", [(33, 17), (70, 47), (4096, 128), (5, 94)])
def test_tile_order_on_the_device(dev, rows, words):
    a = np.random.default_rng(rows + words).integers(-2 ** 31, 2 ** 31 - 1, (rows, words), dtype=np.int64).astype(np.int32)
    t = packing.tile_words(torch.from_numpy(a).to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(t.cpu().numpy(), packing.tile_words(torch.from_numpy(a)).numpy())
    back = packing.untile_words(t, (rows, words))
    torch.cuda.synchronize()
    assert np.array_equal(back.cpu().numpy(), a)


def test_tile_order_pass_checks_what_it_is_handed(dev):
    # the device pass trusts its sizes: tensors of another type, layout, size or alignment are refused on the host
    from nanoquant_amd import ops
    a = torch.zeros((70, 47), dtype=torch.int32, device=dev)
    t = packing.tile_words(a)
    for bad in (a.cpu(), a.to(torch.int64), a.t(), a.view(-1)):
        with pytest.raises(RuntimeError):
            ops.tile_words_device(bad, inverse=False)
    for bad, shape in ((t[:-4], (70, 47)), (t, (70, 48 + 16)), (t.view(2, -1), (70, 47)), (t.to(torch.int64), (70, 47))):
        with pytest.raises(RuntimeError):
            ops.tile_words_device(bad, inverse=True, shape=shape)
    longer = torch.zeros(t.numel() + 1, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="aligned"):
        ops.tile_words_device(longer[1:], inverse=True, shape=(70, 47))
    assert torch.equal(packing.untile_words(t, (70, 47)), a)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 2, 4, 16])
def test_tiled_factors_give_the_same_layer(dev, batch, dtype):
    # ragged shapes (words 47 / 13, rows not a multiple of 32) and a shape with many 32-row tiles per workgroup
    shapes = [(600, 1504, 416), (2048, 1024, 512), (96, 160, 64)]
    rl_t, rl_r = DecodeRunList(batch, dtype, dev), DecodeRunList(batch, dtype, dev)
    refs = []
    for i, (m, n, r) in enumerate(shapes):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 400 + i)
        x = oracle.synth_x(batch, n, 410 + i)
        to = lambda a: torch.from_numpy(a).to(dev).to(dtype)
        f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
        xd, sc = to(x), (to(s_in), to(s_mid), to(s_out))
        vb = packing.binary_packer(torch.from_numpy(vt), "half2").to(dev)
        ub = packing.binary_packer(torch.from_numpy(u), "half2").to(dev)
        rl_r.add(xd, sc[0], vb, sc[1], ub, sc[2])
        rl_t.add(xd, sc[0], packing.tile_words(vb), sc[1], packing.tile_words(ub), sc[2], tiled=True)
        refs.append(oracle.layer_forward(f64(xd), vt, u, f64(sc[0]), f64(sc[1]), f64(sc[2]), dtype=np.float64))
    print(f"tiled run list batch={batch} {dtype}", flush=True)
    ys_t, ys_r = rl_t.run(), rl_r.run()
    torch.cuda.synchronize()
    assert rl_t.status() == 0 and rl_r.status() == 0
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-3
    for (m, n, r), yt, yr, ref in zip(shapes, ys_t, ys_r, refs):
        assert oracle.max_rel_err(yt.float().cpu().numpy(), ref) < (tol if r >= 256 else 1e-2), (m, n, r)
        # same arithmetic, other slice boundaries: row sums differ by fp32 rounding at most
        assert torch.allclose(yt.float(), yr.float(), rtol=4e-3 if dtype == torch.float16 else 2e-2,
                              atol=2e-4 * float(yr.float().abs().max()))


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("batch,dtype", [(16, torch.float16), (8, torch.float16), (16, torch.bfloat16)])
def test_long_lists_on_the_16_bit_operands(dev, batch, dtype, tiled):
    # Batch 8 and 16: a wavefront owns whole 16-row groups of a slice and keeps their row sums in registers; in round r
    # wavefront w has group 16 r + w.  Short lists give every workgroup a few rows (one round, most wavefronts idle);
    # here 64 linears with 2000 x 8192 first factors put about 500 rows of one stage on a workgroup (a whole round, a
    # second one that only some wavefronts take part in, a last group with rows missing) and make the input two chunks
    # at batch 16.
    m, n, r, count = 520, 8192, 2000, 64
    checked = {0: 900, 31: 901, 63: 902}
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    words = (lambda w: packing.tile_words(w)) if tiled else (lambda w: w)
    terms = {}
    for seed in set(checked.values()) | {903}:
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
        dev_ops = (to(s_in), words(packing.binary_packer(torch.from_numpy(vt), "half2").to(dev)), to(s_mid),
                   words(packing.binary_packer(torch.from_numpy(u), "half2").to(dev)), to(s_out))
        terms[seed] = ((vt, u), dev_ops)
    rl = DecodeRunList(batch, dtype, dev)
    refs = {}
    for i in range(count):
        seed = checked.get(i, 903)
        (vt, u), ops = terms[seed]
        x = to(oracle.synth_x(batch, n, 950 + i))
        rl.add(x, *ops, tiled=tiled)
        if i in checked:
            refs[i] = oracle.layer_forward(f64(x), vt, u, f64(ops[0]), f64(ops[2]), f64(ops[4]), dtype=np.float64)
    print(f"long run list batch={batch} {dtype} tiled={tiled}", flush=True)
    for rep in range(2):
        ys = rl.run()
        torch.cuda.synchronize()
        assert rl.status() == 0
        for i, ref in refs.items():
            err = oracle.max_rel_err(ys[i].float().cpu().numpy(), ref)
            assert err < (1e-2 if dtype == torch.bfloat16 else 2e-3), (i, rep, err)


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("batch,dtype", [(16, torch.float16), (8, torch.bfloat16)])
def test_column_shares_of_short_slices(dev, batch, dtype, tiled):
    # Batch 8 and 16, one linear per launch: a workgroup gets a few 16-row groups of a stage, and the wavefronts
    # without a group of their own take shares of the columns (added in a fixed order through LDS).  Shapes: an input
    # of three staged chunks at batch 16 (11008 columns) with 40 rows per workgroup and fewer unit groups in the last
    # chunk than shares; a rank that leaves a last group of 8 rows; an input shorter than one unit group.
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    words = (lambda w: packing.tile_words(w)) if tiled else (lambda w: w)
    for k, (m, n, r) in enumerate([(4096, 11008, 1000), (520, 4096, 40), (64, 96, 32)]):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 7700 + k)
        vt_p, u_p, mid_p = oracle.pad_rank(vt, u, s_mid, 32)
        pack = lambda w: words(packing.binary_packer(torch.from_numpy(w), "half2").to(dev))
        x = to(oracle.synth_x(batch, n, 7800 + k))
        sc = (to(s_in), to(mid_p), to(s_out))
        rl = DecodeRunList(batch, dtype, dev)
        rl.add(x, sc[0], pack(vt_p), sc[1], pack(u_p), sc[2], tiled=tiled)
        print(f"column shares: batch {batch} {dtype} tiled={tiled} m={m} n={n} r={r}", flush=True)
        first = None
        for rep in range(3):
            y = rl.run()[0]
            torch.cuda.synchronize()
            assert rl.status() == 0
            if first is None:
                first = y.clone()
            assert torch.equal(y, first), rep                            # fixed order of the shares: bit for bit
        ref = oracle.layer_forward(f64(x), vt, u, f64(sc[0]), f64(to(s_mid)), f64(sc[2]), dtype=np.float64)
        err = oracle.max_rel_err(first.float().cpu().numpy(), ref)
        assert err < (2e-2 if dtype == torch.bfloat16 else (TIGHT if r >= 256 else 1e-2)), (m, n, r, err)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_batch_4_lists_choose_their_arithmetic_by_length(dev, dtype):
    # fp16 at batch 4: a list with little work per workgroup runs on the 16-bit arithmetic (bit 4 of the plan's flag
    # word), a long one on the fp4 x fp8 arithmetic; bf16 lists always on the latter.  The fp4 x fp8 kernel whose
    # wavefronts own whole row pairs (bit 5) takes every tile-order list at batch 4 and long ones at batch 1 and 2.  All
    # against the oracle.
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    m, n, r = 520, 8192, 2000
    for batch, count in ((4, 1), (4, 64), (2, 1), (2, 96), (1, 1), (1, 96)):
        det = (batch, count) == (1, 96)                                  # the long list at batch 1 with reproducible sums
        rl = DecodeRunList(batch, dtype, dev, deterministic=det)
        checked = {}
        for i in range(count):
            vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 8100 + (i if i in (0, count - 1) else 1))
            vt_p, u_p, mid_p = oracle.pad_rank(vt, u, s_mid, 32)
            pack = lambda w: packing.tile_words(packing.binary_packer(torch.from_numpy(w), "half2").to(dev))
            x = to(oracle.synth_x(batch, n, 8200 + i))
            sc = (to(s_in), to(mid_p), to(s_out))
            rl.add(x, sc[0], pack(vt_p), sc[1], pack(u_p), sc[2], tiled=True)
            if i in (0, count - 1):
                checked[i] = oracle.layer_forward(f64(x), vt, u, f64(sc[0]), f64(to(s_mid)), f64(sc[2]), dtype=np.float64)
        ys = rl.run()
        torch.cuda.synchronize()
        assert rl.status() == 0
        short, own = bool(rl._plan.bound & 16), bool(rl._plan.bound & 32)
        print(f"batch {batch} {dtype} list of {count}: 16-bit arithmetic = {short}, owned row pairs = {own}", flush=True)
        assert short == (batch == 4 and count == 1 and dtype == torch.float16)
        assert own == (not short and (batch == 4 or count == 96))
        for i, ref in checked.items():
            err = oracle.max_rel_err(ys[i].float().cpu().numpy(), ref)
            assert err < (1e-2 if dtype == torch.bfloat16 else TIGHT), (batch, count, i, err)
        if det:
            first = [y.clone() for y in ys]
            for rep in range(3):
                again = rl.run()
                torch.cuda.synchronize()
                assert all(torch.equal(a, b) for a, b in zip(first, again)), rep
    # a short list whose input is longer than what is staged at once at 4 rows (28672 columns, two chunks on the 16-bit
    # arithmetic) and whose rows end inside a 16-row group
    m, n, r = 100, 28672, 256
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 8300)
    x = to(oracle.synth_x(4, n, 8301))
    sc = (to(s_in), to(s_mid), to(s_out))
    pack = lambda w: packing.binary_packer(torch.from_numpy(w), "half2").to(dev)
    rl = DecodeRunList(4, dtype, dev)
    rl.add(x, sc[0], pack(vt), sc[1], pack(u), sc[2])
    y = rl.run()[0]
    torch.cuda.synchronize()
    assert rl.status() == 0
    ref = oracle.layer_forward(f64(x), vt, u, f64(sc[0]), f64(sc[1]), f64(sc[2]), dtype=np.float64)
    err = oracle.max_rel_err(y.float().cpu().numpy(), ref)
    assert err < (1e-2 if dtype == torch.bfloat16 else TIGHT), err


def test_tiled_factor_size_is_checked(dev):
    m, n, r = 64, 128, 32
    _, ops = _term(dev, m, n, r, seed=5)
    x = torch.zeros(1, n, dtype=torch.float16, device=dev)
    rl = DecodeRunList(1, torch.float16, dev)
    with pytest.raises(RuntimeError):
        rl.add(x, ops[0], ops[1].reshape(-1), ops[2], ops[3].reshape(-1), ops[4], tiled=True)   # row-major sizes


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fp8_staging_with_an_outlier_and_a_zero_row(dev, dtype):
    # batch row 0: one activation 1000x the rest (the scale of the fp8 pieces follows the outlier, the other elements
    # sit 10 binades lower); batch row 1: all zeros (its scale must stay finite and its output exactly zero)
    m, n, r = 512, 2048, 256
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 500)
    x = oracle.synth_x(2, n, 501)
    x[0, 777] = 900.0
    x[1, :] = 0.0
    to = lambda a: torch.from_numpy(a).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    xd, sc = to(x), (to(s_in), to(s_mid), to(s_out))
    rl = DecodeRunList(2, dtype, dev)
    i = rl.add(xd, sc[0], packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), sc[1],
               packing.binary_packer(torch.from_numpy(u), "half2").to(dev), sc[2], out_f32=True)
    y = rl.run()[i].cpu().numpy()
    torch.cuda.synchronize()
    assert rl.status() == 0
    ref = oracle.layer_forward(f64(xd), vt, u, f64(sc[0]), f64(sc[1]), f64(sc[2]), dtype=np.float64)
    assert np.all(np.isfinite(y))
    assert np.array_equal(y[1], np.zeros(m, dtype=np.float32))
    assert np.abs(y[0] - ref[0]).max() / np.abs(ref[0]).max() < 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 4, 8])                           # fp4 x fp8 arithmetic (<= 4 rows) and 16-bit arithmetic
def test_outlier_channels_leave_the_other_contributions_intact(dev, dtype, batch):
    """Four input channels 1000 times the rest, as LLM activations have them.  The error of the result is judged
    against the part of the output that the ORDINARY channels contribute (the outliers' own share would hide any loss
    there), element by element with an absolute floor of a tenth of that part's rms.  The yardstick is what two
    roundings to the activation type cost on the same input with everything else exact: the scaled input x * s_in and
    the intermediate vector between the two launches.  The reference makes both and, on top, accumulates in the
    activation type (kernel/cuda/gemv_kernel.cu:101-107 `__hfma2`, :283-301), so it cannot do better than that."""
    m, n, r = 1024, 4096, 512
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 510)
    x = oracle.synth_x(batch, n, 511)
    hot = [5, 1300, 2049, 4000]
    x[:, hot] = (x[:, hot] * 1000.0).astype(x.dtype)
    to = lambda a: torch.from_numpy(a).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    xd, sc = to(x), (to(s_in), to(s_mid), to(s_out))
    rl = DecodeRunList(batch, dtype, dev)
    i = rl.add(xd, sc[0], packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), sc[1],
               packing.binary_packer(torch.from_numpy(u), "half2").to(dev), sc[2], out_f32=True)
    print(f"outliers batch={batch} {dtype}", flush=True)
    y = rl.run()[i].cpu().numpy().astype(np.float64)
    torch.cuda.synchronize()
    assert rl.status() == 0
    xe, (a, b, c) = f64(xd), (f64(t) for t in sc)
    ref = oracle.layer_forward(xe, vt, u, a, b, c, dtype=np.float64)
    calm = xe.copy()
    calm[:, hot] = 0.0
    rest = oracle.layer_forward(calm, vt, u, a, b, c, dtype=np.float64)            # what the ordinary channels contribute
    rounded = lambda v: torch.from_numpy(v).to(dtype).double().numpy()
    h = (rounded(xe * a) @ vt.T.astype(np.float64)) * b
    h_rounded = rounded(h)                                                         # the reference's intermediate tensor
    ref_two_launches = (h_rounded @ u.T.astype(np.float64)) * c
    floor = 0.1 * np.sqrt(np.mean(rest * rest))
    figure = float(np.max(np.abs(y - ref) / (np.abs(rest) + floor)))
    allowed = float(np.max(np.abs(ref_two_launches - ref) / (np.abs(rest) + floor)))
    print(f"  error against the ordinary channels' share: {figure:.3e} (the two roundings alone: {allowed:.3e}); "
          f"whole tensor {oracle.max_rel_err(y, ref):.3e}", flush=True)
    assert np.all(np.isfinite(y))
    # 16-bit arithmetic (more than 4 rows) makes exactly the two roundings; in bf16 they carry 8 bits
    assert oracle.max_rel_err(y, ref) < (4e-3 if batch > 4 and dtype == torch.bfloat16 else 1e-3)
    assert figure <= 1.25 * allowed


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch,tiled", [(1, True), (1, False), (2, True), (4, True), (4, False), (8, True), (16, True), (16, False)])
def test_deterministic_lists_repeat_bit_for_bit(dev, batch, tiled, dtype):
    """`deterministic=True`: every launch of a list gives the same bits (eager launches and graph replays alike), and
    the results still meet the tolerance.  The shapes make many wavefronts add into the same row sums (few rows per
    workgroup), include an input of 16384 columns (more than one staged chunk from batch 4 on) and a ragged one, and
    the second linear reads the first one's output, so a difference anywhere upstream would show."""
    shapes = [(1024, 4096, 512), (512, 16384, 736), (1376, 1000, 96)]
    rl = DecodeRunList(batch, dtype, dev, deterministic=True)
    plain = DecodeRunList(batch, dtype, dev)
    refs = []
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    for i, (m, n, r) in enumerate(shapes):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 600 + i)
        vt_p, u_p, mid_p = oracle.pad_rank(vt, u, s_mid, 32)
        words = lambda w: packing.binary_packer(torch.from_numpy(w), "half2").to(dev)
        vt_d, u_d = words(vt_p), words(u_p)
        if tiled:
            vt_d, u_d = packing.tile_words(vt_d), packing.tile_words(u_d)
        x = to(oracle.synth_x(batch, n, 610 + i))
        sc = (to(s_in), to(mid_p), to(s_out))
        for lst in (rl, plain):
            lst.add(x, sc[0], vt_d, sc[1], u_d, sc[2], tiled=tiled, out_f32=True)
        refs.append(oracle.layer_forward(f64(x), vt, u, f64(sc[0]), f64(to(s_mid)), f64(sc[2]), dtype=np.float64))
    print(f"deterministic list batch={batch} tiled={tiled} {dtype}", flush=True)
    first = [y.clone() for y in rl.run()]
    torch.cuda.synchronize()
    assert rl.status() == 0
    # batch 8 and 16 round x * s_in and the intermediate vector to the activation type when staging
    tol = 1e-2 if (batch >= 8 and dtype == torch.bfloat16) else 1e-3
    for y, ref in zip(first, refs):
        assert oracle.max_rel_err(y.cpu().numpy(), ref) < tol
    for rep in range(20):
        for y in rl.outputs:
            y.fill_(float("nan"))
        ys = rl.run()
        torch.cuda.synchronize()
        for y, e in zip(ys, first):
            assert torch.equal(y, e), rep
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        rl.run()
    for rep in range(5):
        for y in rl.outputs:
            y.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for y, e in zip(rl.outputs, first):
            assert torch.equal(y, e), ("replay", rep)
    assert rl.status() == 0
    # for the record: how often the default mode repeats itself on the same list
    base = [y.clone() for y in plain.run()]
    torch.cuda.synchronize()
    differing = 0
    for rep in range(20):
        ys = plain.run()
        torch.cuda.synchronize()
        differing += int(any(not torch.equal(y, e) for y, e in zip(ys, base)))
    print(f"  default mode: {differing} of 20 launches differ from the first in some bit", flush=True)


def test_an_expired_wait_is_reported_and_the_list_stays_usable(dev):
    """The dependency waits inside the kernel are bounded.  With the bound lowered to one poll from the host, the first
    workgroup that finds its producers unfinished gives up and flags the launch; every kernel still runs to its end.
    The status word reports it once (reading clears it), and the same list works again with the default bound."""
    batch = 1
    rl = DecodeRunList(batch, torch.float16, dev)
    refs = []
    # rank 40: two workgroups compute the first stage, the workgroups of the second stage have nothing else to do and
    # poll while those two are still at work
    for i, (m, n, r) in enumerate([(8192, 4096, 40)]):
        term, ops = _term(dev, m, n, r, seed=800 + i)
        x = oracle.synth_x(batch, n, 810 + i)
        rl.add(torch.from_numpy(x).to(dev), *ops)
        refs.append(oracle.layer_forward(x.astype(np.float64), *term, dtype=np.float64))
    rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    print("run list with a dependency wait of one poll", flush=True)
    rl.spin_limit = 1
    rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 1                                            # reported ...
    assert rl.status() == 0                                            # ... once: reading cleared it
    rl.spin_limit = 0
    ys = rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    for y, ref in zip(ys, refs):
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2   # rank 40: the fp16-output budget


def test_periodic_status_check_raises_after_an_expired_wait(dev):
    """`status_check_every = k`: every k-th `run` reads the status word back and raises when a wait expired since the
    last check, so that a caller who never polls `status()` cannot go on using invalid outputs for long."""
    term, ops = _term(dev, 8192, 4096, 40, seed=860)
    rl = DecodeRunList(1, torch.float16, dev)
    rl.add(torch.from_numpy(oracle.synth_x(1, 4096, 861)).to(dev), *ops)
    rl.status_check_every = 3
    for _ in range(6):                                                 # two checks, both clean
        rl.run()
    rl.spin_limit = 1                                                  # the next launch gives up at its first unmet wait
    rl.run()
    rl.spin_limit = 0
    rl.run()
    with pytest.raises(RuntimeError, match="dependency wait"):
        rl.run()                                                       # the ninth launch checks
    torch.cuda.synchronize()
    assert rl.status() == 0                                            # the check cleared the flag
    for _ in range(3):
        ys = rl.run()
    ref = oracle.layer_forward(oracle.synth_x(1, 4096, 861).astype(np.float64), *term, dtype=np.float64)
    assert oracle.max_rel_err(ys[0].float().cpu().numpy(), ref) < 1e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 2, 4, 8, 16])
def test_grid_fits_every_kernel_variant(dev, batch, dtype):
    """The run-list kernel is only correct with its whole grid resident.  A plan can be launched on several kernel
    variants (word order, reproducible sums, wavefronts owning row pairs) with LDS sizes of their own, and reproducible
    sums are switched on after the grid is fixed: the grid must fit the smallest of them, and a launch whose grid does
    not fit the variant it would start is refused instead of started."""
    import ctypes
    from nanoquant_amd import _lib
    lib = _lib.lib()
    dt = _lib.NQ_F16 if dtype == torch.float16 else _lib.NQ_BF16
    for max_units in (8, 32, 86, 344, 1000):
        caps = [lib.nq_runlist_capacity(batch, dt, max_units, v) for v in range(6)]
        smallest = lib.nq_runlist_capacity(batch, dt, max_units, -1)
        print(f"capacity batch={batch} {dtype} max_units={max_units}: {caps} -> {smallest}", flush=True)
        assert all(c >= 0 for c in caps) and caps[0] > 0 and caps[2] > 0
        assert smallest == min(c for c in caps if c > 0)
    assert lib.nq_runlist_capacity(3, dt, 32, -1) == 0 and lib.nq_runlist_capacity(batch, dt, 32, 6) == 0
    # a built list: the grid fits every variant, with and without reproducible sums, and both launch
    term, ops_ = _term(dev, 512, 1024, 128, seed=850)
    x = torch.from_numpy(oracle.synth_x(batch, 1024, 851)).to(dev, dtype)
    rl = DecodeRunList(batch, dtype, dev)
    rl.add(x, *[t if t is None or t.dtype == torch.int32 else t.to(dtype) for t in ops_])
    rl.build()
    plan = rl._plan
    for v in range(6):
        c = lib.nq_runlist_capacity(batch, dt, plan.max_units, v)
        assert c == 0 or plan.workgroups <= c, (v, c, plan.workgroups)
    y0 = rl.run()[0].clone()
    assert lib.nq_runlist_set_deterministic(ctypes.byref(plan), 1) == 0     # after the grid was fixed
    y1 = rl.run()[0].clone()
    torch.cuda.synchronize()
    assert rl.status() == 0
    assert torch.allclose(y0.float(), y1.float(), rtol=2e-2, atol=2e-3 * float(y0.float().abs().max()))
    # a plan whose grid was inflated behind the library's back is refused, nothing is launched
    from nanoquant_amd.runlist import NqRunlistPlan
    bad = NqRunlistPlan.from_buffer_copy(plan)
    bad.workgroups = bad.index_words = 1 << 20
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    st = lib.nq_runlist_run(ctypes.c_void_p(rl._workspace.data_ptr()), ctypes.byref(bad), stream)
    assert st == _lib.NQ_ERR_HIP
    torch.cuda.synchronize()
    assert rl.status() == 0


@pytest.mark.parametrize("seed", range(16))
def test_random_lists_match_the_oracle(dev, seed):
    """Seeded random lists: batch, type, word order, reproducible sums, 1 to 4 linears of ragged shapes, some fed by
    the linear before them."""
    rng = np.random.default_rng(4200 + seed)
    batch = int(rng.choice([1, 2, 4, 8, 16]))
    dtype = torch.float16 if rng.random() < 0.6 else torch.bfloat16
    tiled = bool(rng.random() < 0.5)
    det = bool(rng.random() < 0.3)
    rl = DecodeRunList(batch, dtype, dev, deterministic=det)
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(dtype)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    refs, shapes, prev_m, prev_out = [], [], None, None
    for i in range(int(rng.integers(1, 5))):
        m = int(rng.choice([32, 96, 200, 512, 1376, 4096, 5000]))
        r = int(rng.choice([32, 40, 96, 256, 736, 2048]))
        chain = prev_m is not None and rng.random() < 0.3
        n = prev_m if chain else int(rng.choice([64, 256, 1000, 4096, 11008, 16384]))
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 4300 + 10 * seed + i)
        s_out = (s_out.astype(np.float32) * 30).astype(np.float16)     # keeps chained activations of order one
        vt_p, u_p, mid_p = oracle.pad_rank(vt, u, s_mid, 32)
        words = lambda w: packing.binary_packer(torch.from_numpy(w), "half2").to(dev)
        vd, ud = words(vt_p), words(u_p)
        if tiled:
            vd, ud = packing.tile_words(vd), packing.tile_words(ud)
        sc = (to(s_in), to(mid_p), to(s_out))
        if chain:
            xin = prev_out                                             # the previous output as the kernel hands it on
            rl.add(rl.outputs[-1], sc[0], vd, sc[1], ud, sc[2], tiled=tiled, x_from=i - 1)
        else:
            xin = f64(to(oracle.synth_x(batch, n, 4400 + 10 * seed + i)))
            rl.add(to(xin), sc[0], vd, sc[1], ud, sc[2], tiled=tiled)
        ref = oracle.layer_forward(xin, vt, u, f64(sc[0]), f64(to(s_mid)), f64(sc[2]), dtype=np.float64)
        refs.append(ref)
        prev_m, prev_out = m, f64(torch.from_numpy(ref).to(dtype))
        shapes.append((m, n, r, chain))
    print(f"random list {seed}: batch {batch} {dtype} tiled={tiled} deterministic={det} {shapes}", flush=True)
    ys = rl.run()
    torch.cuda.synchronize()
    assert rl.status() == 0
    for y, ref in zip(ys, refs):
        assert torch.isfinite(y.float()).all()
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < (2e-2 if dtype == torch.bfloat16 else 1e-2)
