"""Panel launches of the grouped prefill path (nq_gemm_nanoquant_group_ws): persistent workgroups on 128-token x
256-row panels whose k ranges are shared out evenly, partial tiles handed to the panel's owner through a workspace.
Checked against the dense definition (src/nanoquant/modules/linear.py:248-257 of the reference, restated in
oracle/) and against the launches without a workspace.  The reference's counterpart is the stripe reduction of its
prefill kernel (src/nanoquant/kernel/cuda/gemm_kernel.cu:594-640)."""
import ctypes

import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import _lib, ops, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu
TOL = {torch.float16: 2e-3, torch.bfloat16: 1e-2}


def _cast(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a).astype(np.float32)).to(dtype)


def _term(dev, m, n, r, seed, dtype):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    si, sm, so = (_cast(a, dtype) for a in (s_in, s_mid, s_out))
    packed = packing.marlin_nanoquant_packer(torch.from_numpy(vt).T.contiguous().to(dev),
                                             torch.from_numpy(u).T.contiguous().to(dev), si.to(dev), sm.to(dev), so.to(dev))
    ref = lambda x: oracle.layer_forward(x, vt, u, si.float().numpy(), sm.float().numpy(), so.float().numpy(), dtype=np.float32)
    return packed, ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tokens", [128, 100, 77, 1, 200, 300])
def test_panel_launch_on_small_shapes(dev, tokens, dtype):
    # few units for 256 workgroups: every panel is cut into single k tiles, so every output goes through the hand-over
    # of partial tiles; widths that are not multiples of 256 leave ragged last panels; 200 and 300 tokens need two and
    # three token blocks with a ragged last one
    n = 1024
    shapes = [(1024, 512), (256, 100), (320, 256), (2048, 768)]
    terms = [_term(dev, m, n, r, 500 + i, dtype) for i, (m, r) in enumerate(shapes)]
    x = _cast(oracle.synth_x(tokens, n, 9), dtype)
    print(f"panel small tokens={tokens} {dtype}", flush=True)
    ys = ops.gemm_group_forward(x.to(dev), [p for p, _ in terms], panel="always")
    torch.cuda.synchronize()
    assert ops.panel_status(dev) == 0
    plain = ops.gemm_group_forward(x.to(dev), [p for p, _ in terms], panel="never")
    torch.cuda.synchronize()
    for (m, r), (packed, ref), y, y0 in zip(shapes, terms, ys, plain):
        assert y.shape == (tokens, m) and y.dtype == dtype
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref(x.float().numpy())) < TOL[dtype], (m, r)
        # same products, another order of the fp32 additions, one rounding of h in between
        assert torch.allclose(y.float(), y0.float(), rtol=2e-2, atol=2e-3 * float(y0.float().abs().max())), (m, r)


def test_panel_launch_long_k_with_bias_and_own_inputs(dev):
    # a long k (11 tiles) over few rows: a panel is shared by many workgroups; one term with bias, inputs of their own
    dtype, tokens = torch.float16, 128
    rng = np.random.default_rng(5)
    shapes = [(512, 2816, 256), (768, 1024, 512), (256, 2816, 768)]
    terms, xs, biases = [], [], []
    for i, (m, n, r) in enumerate(shapes):
        terms.append(_term(dev, m, n, r, 640 + i, dtype))
        xs.append(_cast(oracle.synth_x(tokens, n, 740 + i), dtype))
        biases.append(_cast(rng.normal(0, 0.05, m), dtype) if i == 1 else None)
    print("panel long k + bias", flush=True)
    ys = ops.gemm_group_forward([x.to(dev) for x in xs], [p for p, _ in terms],
                                [None if b is None else b.to(dev) for b in biases], panel="always")
    torch.cuda.synchronize()
    assert ops.panel_status(dev) == 0
    for (packed, ref), x, b, y in zip(terms, xs, biases, ys):
        want = ref(x.float().numpy())
        if b is not None:
            want = want + b.float().numpy()[None, :]
        assert oracle.max_rel_err(y.float().cpu().numpy(), want) < TOL[dtype]


def test_panel_launches_repeat_and_replay(dev):
    # the hand-over flags carry the number of the launch, taken from a counter in the workspace: launches in a row
    # and replays of a captured graph (same kernel arguments every time) must all give the first launch's result
    dtype, tokens, n = torch.float16, 128, 1024
    shapes = [(1024, 512), (512, 256)]
    terms = [_term(dev, m, n, r, 560 + i, dtype) for i, (m, r) in enumerate(shapes)]
    x = _cast(oracle.synth_x(tokens, n, 19), dtype).to(dev)
    outs = [torch.empty(tokens, m, dtype=dtype, device=dev) for m, _ in shapes]
    packed = [p for p, _ in terms]
    print("panel repeat + graph replay", flush=True)
    ops.gemm_group_forward(x, packed, outs=outs, panel="always")
    torch.cuda.synchronize()
    first = [o.clone() for o in outs]
    for (m, r), (_, ref), y in zip(shapes, terms, first):
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref(x.float().cpu().numpy())) < TOL[dtype]
    for _ in range(3):
        for o in outs:
            o.zero_()
        ops.gemm_group_forward(x, packed, outs=outs, panel="always")
        torch.cuda.synchronize()
        for o, f in zip(outs, first):
            assert torch.equal(o, f)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.gemm_group_forward(x, packed, outs=outs, panel="always")      # allocates this stream's workspace outside capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            ops.gemm_group_forward(x, packed, outs=outs, panel="always")
    torch.cuda.synchronize()
    for _ in range(4):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, f in zip(outs, first):
            assert torch.equal(o, f)
    with torch.cuda.stream(side):
        assert ops.panel_status(dev) == 0
    assert ops.panel_status(dev) == 0


def test_an_expired_wait_of_a_panel_launch_is_reported(dev):
    """The workgroups that finish a shared panel wait a bounded number of polls for the others' partial tiles.  With
    the bound lowered to one poll from the host, a launch whose panels are shared by many workgroups reports an expiry,
    runs to its end, and the workspace serves the next launch (default bound) as before."""
    lib = _lib.lib()
    dtype, tokens = torch.float16, 128
    shapes = [(512, 2816, 256), (256, 2816, 768)]                    # 11 k tiles over few rows: every panel is shared
    terms = [_term(dev, m, n, r, 660 + i, dtype) for i, (m, n, r) in enumerate(shapes)]
    xs = [_cast(oracle.synth_x(tokens, n, 760 + i), dtype).to(dev) for i, (m, n, r) in enumerate(shapes)]
    packed = [p for p, _ in terms]
    good = [y.clone() for y in ops.gemm_group_forward(xs, packed, panel="always")]
    torch.cuda.synchronize()
    assert ops.panel_status(dev) == 0
    print("panel launch with waits of one poll", flush=True)
    assert lib.nq_gemm_panel_set_spin_limit(1) == 0
    try:
        ops.gemm_group_forward(xs, packed, panel="always")
        torch.cuda.synchronize()
        assert ops.panel_status(dev) == 1                               # reported ...
        assert ops.panel_status(dev) == 0                               # ... once
    finally:
        assert lib.nq_gemm_panel_set_spin_limit(0) == 0
    again = ops.gemm_group_forward(xs, packed, panel="always")
    torch.cuda.synchronize()
    assert ops.panel_status(dev) == 0
    for y, g0, (_, ref), x in zip(again, good, terms, xs):
        assert torch.equal(y, g0)
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref(x.float().cpu().numpy())) < TOL[dtype]


def test_panel_entry_point_argument_checks(dev):
    lib = _lib.lib()
    dtype, tokens, n = torch.float16, 128, 512
    packed, _ = _term(dev, 256, n, 64, 3, dtype)
    wu, wv, sg, sl, sh, _ws = packed
    rp = wu.size(1) * 2
    x = torch.zeros(tokens, n, dtype=dtype, device=dev)
    h = torch.empty(tokens, rp, dtype=dtype, device=dev)
    y = torch.empty(tokens, 256, dtype=dtype, device=dev)
    arr = (ops.NqGemmTerm * 1)(ops.NqGemmTerm(x.data_ptr(), wu.data_ptr(), wv.data_ptr(), sg.data_ptr(), sl.data_ptr(),
                                             sh.data_ptr(), None, h.data_ptr(), y.data_ptr(), n, rp, 256))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = int(lib.nq_gemm_panel_workspace_bytes())
    assert need > 128 * 256 * 4
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    call = lambda ptr, nbytes, mode: lib.nq_gemm_nanoquant_group_ws(arr, 1, tokens, _lib.NQ_F16, None, 0, ptr, nbytes, mode, stream)
    assert call(ws.data_ptr(), need, 1) == 0
    assert call(ws.data_ptr(), need - 1, 1) != 0                  # workspace too small
    assert call(ws.data_ptr() + 16, need, 1) != 0                 # not 256-byte aligned
    assert call(ws.data_ptr(), need, 7) != 0                      # unknown mode
    assert call(None, 0, 0) == 0                                  # no workspace: the launches without one
    torch.cuda.synchronize()
    st = ctypes.c_int(-1)
    assert lib.nq_gemm_panel_status(ws.data_ptr(), ctypes.byref(st), stream) == 0 and st.value == 0
    assert lib.nq_gemm_panel_status(None, ctypes.byref(st), stream) != 0
