"""Bias on the kernel paths.  The reference's module drops its bias once `_prepare_kernel` has run
(src/nanoquant/modules/linear.py:121-141 returns before :248-257 adds it); the default here mirrors that, and
`kernel_path_bias = True` adds the bias in the epilogue of the last kernel.  Checked against the dense definition
plus bias on every kernel that has such an epilogue: per-linear decode (lane-group kernel and 16-row pieces),
run list (fp8-piece and 16-bit arithmetic), prefill (few-token kernel, unsplit blocks, k-split + finish kernel)."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import DecodeRunList, NanoQuantLinear, ops, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu


def _module(dev, m, n, r, seed, dtype):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    bias = (np.random.default_rng(seed).normal(0, 0.05, m)).astype(np.float32)
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid), f(s_out), bias=f(bias), dtype=dtype).to(dev)
    return mod, (vt, u, s_in, s_mid, s_out), bias


def _ref(x, term, bias, dtype):
    # scales and bias as the kernels see them: rounded to the activation type
    rnd = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype).float().numpy().astype(np.float64)
    vt, u, s_in, s_mid, s_out = term
    y = oracle.layer_forward(rnd(x), vt, u, rnd(s_in), rnd(s_mid), rnd(s_out), dtype=np.float64)
    return y, y + rnd(bias)[None, :]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 3, 16])
def test_decode_module_adds_bias_only_when_asked(dev, batch, dtype):
    m, n, r = 608, 1056, 288
    mod, term, bias = _module(dev, m, n, r, 50, dtype)
    mod._prepare_kernel("gemv", dtype)
    x = oracle.synth_x(batch, n, 51)
    ref_plain, ref_bias = _ref(x, term, bias, dtype)
    xt = torch.from_numpy(x).to(dev).to(dtype)
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-3
    print(f"decode bias batch={batch} {dtype}", flush=True)
    y0 = mod(xt)                                         # the reference's behaviour: no bias on the kernel path
    mod.kernel_path_bias = True
    y1 = mod(xt)
    torch.cuda.synchronize()
    assert oracle.max_rel_err(y0.float().cpu().numpy(), ref_plain) < tol
    assert oracle.max_rel_err(y1.float().cpu().numpy(), ref_bias) < tol
    assert oracle.max_rel_err(y0.float().cpu().numpy(), ref_bias) > 0.05       # the bias is not small here


@pytest.mark.parametrize("batch", [1, 8])
def test_run_list_bias(dev, batch):
    m, n, r = 1024, 768, 352
    mod, term, bias = _module(dev, m, n, r, 60, torch.float16)
    mod._prepare_kernel("gemv", torch.float16)
    x = oracle.synth_x(batch, n, 61)
    _, ref_bias = _ref(x, term, bias, torch.float16)
    rl = DecodeRunList(batch, torch.float16, dev)
    i = rl.add(torch.from_numpy(x).to(dev), mod.scale_pre, mod.V_int8, mod.scale_mid, mod.U_int8, mod.scale_post,
               bias=mod.bias.to(torch.float16))
    print(f"run list bias batch={batch}", flush=True)
    y = rl.run()[i]
    torch.cuda.synchronize()
    assert rl.status() == 0
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref_bias) < 2e-3


@pytest.mark.parametrize("tokens,m,n,r", [(64, 512, 512, 256), (160, 2048, 1024, 512), (512, 512, 4096, 2048)])
def test_prefill_module_bias(dev, tokens, m, n, r):
    # 64 tokens: few-token kernel; 160 x 2048: unsplit blocks; 512 tokens with few row tiles: k-split + finish kernel
    mod, term, bias = _module(dev, m, n, r, 70, torch.float16)
    mod._prepare_kernel("gemm", torch.float16)
    x = oracle.synth_x(tokens, n, 71)
    ref_plain, ref_bias = _ref(x, term, bias, torch.float16)
    xt = torch.from_numpy(x).to(dev)
    print(f"prefill bias tokens={tokens} m={m} n={n} r={r}", flush=True)
    y0 = mod(xt)
    mod.kernel_path_bias = True
    y1 = mod(xt)
    torch.cuda.synchronize()
    assert oracle.max_rel_err(y0.float().cpu().numpy(), ref_plain) < 1e-2
    assert oracle.max_rel_err(y1.float().cpu().numpy(), ref_bias) < 1e-2
    assert oracle.max_rel_err(y0.float().cpu().numpy(), ref_bias) > 0.05


def test_bias_argument_errors(dev):
    mod, term, bias = _module(dev, 256, 512, 128, 80, torch.float16)
    mod._prepare_kernel("gemv", torch.float16)
    x = torch.zeros(1, 512, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError):
        ops.gemv_forward_with_bias(x, mod.scale_pre, mod.V_int8, mod.scale_mid, mod.U_int8, mod.scale_post,
                                   torch.zeros(255, dtype=torch.float16, device=dev))
    with pytest.raises(RuntimeError):
        ops.gemv_forward_with_bias(x, mod.scale_pre, mod.V_int8, mod.scale_mid, mod.U_int8, mod.scale_post,
                                   torch.zeros(256, dtype=torch.float32, device=dev))
