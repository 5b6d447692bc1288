"""A module prepared for decode with `mfma_from_rows = 3` sends calls of 3 or more rows to the few-token MFMA tiles of
the prefill path (opt-in; the reference runs every batch size through its GEMV kernels, re-reading the weights per batch row:
kernel/cuda/gemv_kernel.cu:288-290).  Same interface, same result within the tolerance, tiles built from the decode
words on the device."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd.linear import NanoQuantLinear
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu


def _module(dev, m, n, r, seed, dtype):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid), f(s_out), dtype=dtype).to(dev)
    mod._prepare_kernel("gemv", dtype)
    assert mod.mfma_from_rows == 0                                     # the route is opt-in
    mod.mfma_from_rows = 3
    return mod, (vt, u, s_in, s_mid, s_out)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows", [2, 3, 8, 12, 16, 40])
def test_rows_choose_the_kernel(dev, rows, dtype):
    m, n, r = 768, 1024, 300
    mod, term = _module(dev, m, n, r, 700, dtype)
    x = torch.from_numpy(oracle.synth_x(rows, n, 701)).to(dtype)
    print(f"row routing rows={rows} {dtype}", flush=True)
    y = mod(x.to(dev))
    torch.cuda.synchronize()
    assert (mod._mfma_tiles is not None) == (rows >= 3)
    vt, u, s_in, s_mid, s_out = term
    c = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype).double().numpy()
    ref = oracle.layer_forward(x.double().numpy(), vt, u, c(s_in), c(s_mid), c(s_out), dtype=np.float64)
    assert y.shape == (rows, m) and y.dtype == dtype
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2
    if rows >= 3:
        # the tiles are the prefill packer's, bit for bit, although no dense matrix was formed
        f = lambda a: torch.from_numpy(a)
        dense = NanoQuantLinear.from_factors(f(vt.astype(np.float32)), f(u.astype(np.float32)), f(s_in.astype(np.float32)),
                                             f(s_mid.astype(np.float32)), f(s_out.astype(np.float32)), dtype=dtype)
        dense._prepare_kernel("gemm", dtype)
        for a, b in zip(mod._mfma_tiles[:2], (dense.V_int8, dense.U_int8)):
            assert torch.equal(a.cpu(), b)
        # and the decode kernels still serve the same module when the route is switched off
        mod.mfma_from_rows = 0
        y2 = mod(x.to(dev))
        torch.cuda.synchronize()
        assert oracle.max_rel_err(y2.float().cpu().numpy(), ref) < 1e-2


def test_shapes_without_prefill_tiles_stay_on_the_decode_kernels(dev):
    mod, term = _module(dev, 200, 352, 64, 710, torch.float16)       # in % 256 != 0, out % 32 != 0
    x = torch.from_numpy(oracle.synth_x(16, 352, 711))
    y = mod(x.to(dev))
    torch.cuda.synchronize()
    assert mod._mfma_tiles is None
    ref = oracle.layer_forward(x.double().numpy(), *term, dtype=np.float64)
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2
    with pytest.raises(ValueError, match="in_features % 256"):
        mod.prepare_mfma_route()


def test_bias_rides_along_on_the_routed_path(dev):
    mod, term = _module(dev, 512, 512, 128, 720, torch.float16)
    mod.bias = torch.nn.Parameter(torch.linspace(-1, 1, 512, device=dev, dtype=torch.float16), requires_grad=False)
    mod.kernel_path_bias = True
    x = torch.from_numpy(oracle.synth_x(9, 512, 721))
    y = mod(x.to(dev))
    torch.cuda.synchronize()
    ref = oracle.layer_forward(x.double().numpy(), *term, dtype=np.float64) + mod.bias.double().cpu().numpy()
    assert mod._mfma_tiles is not None
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2


def test_no_tiles_are_built_inside_a_stream_capture(dev):
    mod, term = _module(dev, 512, 512, 128, 730, torch.float16)
    x = torch.from_numpy(oracle.synth_x(8, 512, 731)).to(dev)
    ref = oracle.layer_forward(x.double().cpu().numpy(), *term, dtype=np.float64)
    mod.mfma_from_rows = 0
    mod(x)                                                             # warm the decode kernels outside the capture
    mod.mfma_from_rows = 3
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        y = mod(x)
    assert mod._mfma_tiles is None                                     # the captured call stayed on the decode kernels
    g.replay()
    torch.cuda.synchronize()
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2
    mod.prepare_mfma_route()                                           # prepared beforehand: the capture uses the tiles
    mod(x)
    torch.cuda.synchronize()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, stream=side):
        y2 = mod(x)
    g2.replay()
    torch.cuda.synchronize()
    assert oracle.max_rel_err(y2.float().cpu().numpy(), ref) < 1e-2
