"""Groups of independent decode linears sharing launches (nq_gemv_forward_group, `ops.gemv_group_forward`,
`decode_group`) against the dense definition (src/nanoquant/modules/linear.py:248-257 of the reference, restated in
oracle/).  The reference launches its two stage kernels per module (modules/linear.py:121-130 ->
kernel/cuda/gemv_kernel.cu:406-425); here a group takes two launches, or one whose second stages wait inside it."""
import ctypes

import numpy as np
import pytest
import torch

import nanoquant_amd
from nanoquant_amd import _lib, ops, packing
from nanoquant_amd.runlist import NqLinear
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu
TOL = {torch.float16: 2e-3, torch.bfloat16: 1e-2}


def _cast(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a).astype(np.float32)).to(dtype)


def _linear(dev, m, n, r, seed, dtype, with_mid=True):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    si, sm, so = (_cast(a, dtype) for a in (s_in, s_mid, s_out))
    if not with_mid:
        sm = None
    ops_args = (si.to(dev), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), None if sm is None else sm.to(dev),
                packing.binary_packer(torch.from_numpy(u), "half2").to(dev), so.to(dev))
    ref = lambda x: oracle.layer_forward(x, vt, u, si.float().numpy(), None if sm is None else sm.float().numpy(),
                                         so.float().numpy(), dtype=np.float64)
    return ops_args, ref


# q/k/v-like, gate/up-like and ragged shapes (n, r not multiples of 8: the element-wise staging; m not a multiple of
# the rows of a workgroup)
SHAPES = [(512, 1024, 256), (128, 1024, 96), (1376, 1024, 744), (70, 100, 50), (33, 1000, 70)]


@pytest.mark.parametrize("one_launch", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 7, 9])
def test_group_of_independent_linears(dev, batch, dtype, one_launch):
    rng = np.random.default_rng(batch)
    lins, xs, biases = [], [], []
    for i, (m, n, r) in enumerate(SHAPES):
        lins.append(_linear(dev, m, n, r, 900 + i, dtype, with_mid=i != 1))
        xs.append(_cast(oracle.synth_x(batch, n, 950 + i), dtype))
        biases.append(_cast(rng.normal(0, 0.05, m), dtype).to(dev) if i in (0, 3) else None)
    print(f"gemv group batch={batch} {dtype} one_launch={one_launch}", flush=True)
    ys = ops.gemv_group_forward([x.to(dev) for x in xs], [a for a, _ in lins], biases, one_launch=one_launch)
    torch.cuda.synchronize()
    assert ops.gemv_group_status(dev) == 0
    for (m, n, r), (args, ref), x, b, y in zip(SHAPES, lins, xs, biases, ys):
        assert y.shape == (batch, m) and y.dtype == dtype
        want = ref(x.float().numpy())
        if b is not None:
            want = want + b.float().cpu().numpy()[None, :]
        tol = TOL[dtype] if r >= 256 else 1e-2
        assert oracle.max_rel_err(y.float().cpu().numpy(), want) < tol, (m, n, r)
        # the op (one linear per launch) runs the same arithmetic in the same order
        y1 = ops.gemv_forward_with_bias(x.to(dev), *args, b)
        assert torch.equal(y1, y), (m, n, r)


@pytest.mark.parametrize("one_launch", [False, True])
def test_group_larger_than_one_launch_and_shared_input(dev, one_launch):
    # 11 linears on one input: two groups (8 + 3)
    dtype, batch, n = torch.float16, 4, 2048
    assert ops._lib.lib().nq_gemv_group_max() == 8
    shapes = [(256 + 64 * i, 128 + 32 * i) for i in range(11)]
    lins = [_linear(dev, m, n, r, 300 + i, dtype) for i, (m, r) in enumerate(shapes)]
    x = _cast(oracle.synth_x(batch, n, 77), dtype)
    print("gemv group of 11", flush=True)
    ys = ops.gemv_group_forward(x.to(dev), [a for a, _ in lins], one_launch=one_launch)
    torch.cuda.synchronize()
    assert ops.gemv_group_status(dev) == 0
    for (m, r), (_, ref), y in zip(shapes, lins, ys):
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref(x.float().numpy())) < 1e-2, (m, r)


@pytest.mark.parametrize("one_launch", [False, True])
def test_group_launches_repeat_and_replay(dev, one_launch):
    # one launch per group: the flags are put back to zero by the launch that used them: launches in a row and replays
    # of a captured launch (same slot of flags every time) must all give the first launch's result
    dtype, batch, n = torch.float16, 1, 4096
    shapes = [(4096, 1024), (1024, 256), (1024, 256)]
    lins = [_linear(dev, m, n, r, 400 + i, dtype) for i, (m, r) in enumerate(shapes)]
    x = _cast(oracle.synth_x(batch, n, 78), dtype).to(dev)
    outs = [torch.empty(batch, m, dtype=dtype, device=dev) for m, _ in shapes]
    args = [a for a, _ in lins]
    print("gemv group repeat + replay", flush=True)
    ops.gemv_group_forward(x, args, outs=outs, one_launch=one_launch)
    torch.cuda.synchronize()
    first = [o.clone() for o in outs]
    for (m, r), (_, ref), y in zip(shapes, lins, first):
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref(x.float().cpu().numpy())) < TOL[dtype]
    for _ in range(20):
        ops.gemv_group_forward(x, args, outs=outs, one_launch=one_launch)
    torch.cuda.synchronize()
    for o, f in zip(outs, first):
        assert torch.equal(o, f)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(3):                        # three launches in the graph, each with a slot of its own
                ops.gemv_group_forward(x, args, outs=outs, one_launch=one_launch)
    torch.cuda.synchronize()
    for _ in range(4):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, f in zip(outs, first):
            assert torch.equal(o, f)
    assert ops.gemv_group_status(dev) == 0


def test_an_expired_wait_of_a_one_launch_group_is_reported(dev):
    """The second-stage workgroups of a one-launch group wait a bounded number of polls.  With the bound lowered to one
    poll from the host they give up at once (the first stage has only just started), the launch still runs to its end
    and the status word says so once; with the default bound back, the next launch is right again."""
    lib = _lib.lib()
    dtype, batch, n = torch.float16, 1, 4096
    (args, ref) = _linear(dev, 4096, n, 1024, 470, dtype)
    x = _cast(oracle.synth_x(batch, n, 79), dtype).to(dev)
    good = ops.gemv_group_forward(x, [args], one_launch=True)[0].clone()
    torch.cuda.synchronize()
    assert ops.gemv_group_status(dev) == 0
    print("one-launch group with a wait of one poll", flush=True)
    assert lib.nq_gemv_group_set_spin_limit(1) == 0
    try:
        ops.gemv_group_forward(x, [args], one_launch=True)
        torch.cuda.synchronize()
        assert ops.gemv_group_status(dev) == 1                          # reported ...
        assert ops.gemv_group_status(dev) == 0                          # ... once
    finally:
        assert lib.nq_gemv_group_set_spin_limit(0) == 0
    again = ops.gemv_group_forward(x, [args], one_launch=True)[0]
    torch.cuda.synchronize()
    assert ops.gemv_group_status(dev) == 0
    assert torch.equal(again, good)
    assert oracle.max_rel_err(again.float().cpu().numpy(), ref(x.float().cpu().numpy())) < TOL[dtype]


def test_decode_group_of_modules(dev):
    dtype = torch.float16
    rng = np.random.default_rng(3)
    mods = []
    for i, (m, n, r) in enumerate([(768, 512, 192), (256, 512, 64), (256, 512, 64)]):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 40 + i)
        mod = nanoquant_amd.NanoQuantLinear.from_factors(
            torch.from_numpy(vt).float(), torch.from_numpy(u).float(), torch.from_numpy(s_in), torch.from_numpy(s_mid),
            torch.from_numpy(s_out), bias=torch.from_numpy(rng.normal(0, 0.1, m).astype(np.float32)) if i == 0 else None,
            dtype=torch.float32).to(dev)
        mod._prepare_kernel("gemv", dtype)
        mod.kernel_path_bias = True
        mods.append(mod)
    for shape in [(1, 512), (2, 2, 512), (5, 512)]:
        x = torch.from_numpy(oracle.synth_x(int(np.prod(shape[:-1])), 512, 9)).reshape(shape).to(dev, dtype)
        print(f"decode_group x={shape}", flush=True)
        ys = nanoquant_amd.decode_group(mods, x)
        torch.cuda.synchronize()
        for mod, y in zip(mods, ys):
            want = mod(x)
            assert y.shape == want.shape and torch.equal(y, want)
    with pytest.raises(ValueError):
        nanoquant_amd.decode_group(mods, [x])
    # the prepared group behind decode_group follows the modules: new factors for one of them are picked up
    assert len(mods[0].__dict__["_decode_groups"]) == 1
    vt, u, s_in, s_mid, s_out = oracle.synth_term(256, 512, 64, 99)
    fresh = nanoquant_amd.NanoQuantLinear.from_factors(torch.from_numpy(vt).float(), torch.from_numpy(u).float(), torch.from_numpy(s_in),
                                                       torch.from_numpy(s_mid), torch.from_numpy(s_out), dtype=torch.float32).to(dev)
    fresh._prepare_kernel("gemv", dtype)
    mods[2].V_int8, mods[2].U_int8 = fresh.V_int8, fresh.U_int8
    mods[2].scale_pre, mods[2].scale_mid, mods[2].scale_post = fresh.scale_pre, fresh.scale_mid, fresh.scale_post
    x = torch.from_numpy(oracle.synth_x(2, 512, 10)).to(dev, dtype)
    ys = nanoquant_amd.decode_group(mods, x)
    torch.cuda.synchronize()
    assert torch.equal(ys[2], fresh(x)) and torch.equal(ys[0], mods[0](x))


def test_prepared_group_checks_once_and_matches(dev):
    dtype = torch.float16
    lins = [_linear(dev, m, 1024, r, 480 + i, dtype) for i, (m, r) in enumerate([(512, 256), (128, 96)])]
    bias = _cast(np.linspace(-1, 1, 512), dtype).to(dev)
    group = ops.GemvGroup([a for a, _ in lins], [bias, None])
    for batch in (1, 3, 8):
        x = _cast(oracle.synth_x(batch, 1024, 490 + batch), dtype).to(dev)
        ys = group(x)
        want = ops.gemv_group_forward(x, [a for a, _ in lins], [bias, None])
        torch.cuda.synchronize()
        for y, w in zip(ys, want):
            assert torch.equal(y, w)
    with pytest.raises(RuntimeError):
        group(torch.zeros(1, 1000, dtype=dtype, device=dev))            # wrong width
    with pytest.raises(RuntimeError):
        group(torch.zeros(1, 1024, dtype=torch.float32, device=dev))     # wrong type
    with pytest.raises(RuntimeError):
        ops.GemvGroup([(lins[0][0][0], lins[0][0][1], lins[0][0][2], lins[1][0][3], lins[0][0][4])])   # factors that do not fit


def test_group_entry_point_argument_checks(dev):
    lib = _lib.lib()
    dtype = torch.float16
    (sg, ub, sl, vb, sh), _ = _linear(dev, 64, 128, 32, 1, dtype)
    x = torch.zeros(1, 128, dtype=dtype, device=dev)
    y = torch.empty(1, 64, dtype=dtype, device=dev)
    h = torch.empty(2, 32, dtype=torch.float32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: t.data_ptr()

    def entry(**kw):
        f = dict(x=p(x), s_in=p(sg), vt_bits=p(ub), s_mid=p(sl), u_bits=p(vb), s_out=p(sh), h=p(h), y=p(y), addend=None,
                 n=128, r=32, m=64, x_from=-1, y_from=-1, out_f32=0, bias=None, tiled=0)
        f.update(kw)
        return NqLinear(*[f[name] for name, _ in NqLinear._fields_])

    call = lambda entries, batch=1, dt=_lib.NQ_F16, one=0: lib.nq_gemv_forward_group((NqLinear * len(entries))(*entries),
                                                                                      len(entries), batch, dt, one, stream)
    assert call([entry()]) == 0
    assert call([entry()], one=1) == 0
    assert call([entry()], one=2) != 0                                  # not a switch value
    assert call([entry()], dt=5) != 0                                   # unknown dtype
    assert call([entry(x=None)]) != 0                                   # missing pointer
    assert call([entry(x_from=0)]) != 0                                 # links belong to run lists
    assert call([entry(out_f32=1)]) != 0
    assert call([entry(tiled=1)]) != 0
    assert call([entry(), entry()]) != 0                                # two linears on one h
    assert call([entry(), entry(h=p(h) + 4 * 32)]) == 0
    assert call([], 1) == 0
    torch.cuda.synchronize()
    st = ctypes.c_int(-1)
    assert lib.nq_gemv_group_status(ctypes.byref(st), stream) == 0 and st.value == 0
    assert lib.nq_gemv_group_status(None, stream) != 0
