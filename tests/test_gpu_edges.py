"""Edge cases of the operator boundary on the GPU: empty inputs, batches that are split into pieces (16-row
pieces run on the run-list kernel in single-stage mode), 3-D module inputs, bf16 at the same shapes."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import NanoQuantLinear, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu
HINTS = (128, 128, 2, 2, 1, 1, 8, 8)


def _ops(dev, term, dtype=torch.float16):
    vt, u, s_in, s_mid, s_out = term
    f = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype).to(dev)
    return (f(s_in), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), f(s_mid),
            packing.binary_packer(torch.from_numpy(u), "half2").to(dev), f(s_out))


def test_empty_batch_and_zero_tokens(dev):
    m, n, r = 256, 512, 128
    term = oracle.synth_term(m, n, r, 1)
    s_in, vt_bits, s_mid, u_bits, s_out = _ops(dev, term)
    x = torch.empty(0, n, dtype=torch.float16, device=dev)
    print("empty decode batch", flush=True)
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(x, s_in, vt_bits, s_mid, u_bits, s_out, *HINTS)
    torch.cuda.synchronize()
    assert y.shape == (0, m)
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    mod = NanoQuantLinear.from_factors(f(term[0]), f(term[1]), f(term[2]), f(term[3]), f(term[4]), dtype=torch.float16).to(dev)
    mod._prepare_kernel("gemm", torch.float16)
    print("zero prefill tokens", flush=True)
    y = mod(torch.empty(0, n, dtype=torch.float16, device=dev))
    torch.cuda.synchronize()
    assert y.shape == (0, m)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [16, 21, 48])
def test_batches_split_into_pieces(dev, dtype, batch):
    # 16- and 8-row pieces go through the run-list kernel on a single stage, the remainder (4 + 1) through the
    # lane-group kernel; every row must come out as if computed alone
    m, n, r = 1376, 2048, 736          # 23 words per second-stage row: ragged 16-byte units
    term = oracle.synth_term(m, n, r, 50 + batch)
    x = oracle.synth_x(batch, n, 60 + batch)
    cast = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype)
    xt = cast(x)
    s_in, vt_bits, s_mid, u_bits, s_out = _ops(dev, term, dtype)
    ref = oracle.layer_forward(xt.float().numpy().astype(np.float64), term[0], term[1], s_in.float().cpu().numpy(),
                               s_mid.float().cpu().numpy(), s_out.float().cpu().numpy(), dtype=np.float64)
    print(f"pieces batch={batch} {dtype}", flush=True)
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(xt.to(dev), s_in, vt_bits, s_mid, u_bits, s_out, *HINTS)
    torch.cuda.synchronize()
    err = oracle.max_rel_err(y.float().cpu().numpy(), ref)
    assert err < (1e-3 if dtype == torch.float16 else 1e-2), err


def test_module_three_dimensional_input_both_kernels(dev):
    m, n, r = 512, 768, 256
    term = oracle.synth_term(m, n, r, 7)
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    x = oracle.synth_x(2 * 70, n, 8).reshape(2, 70, n)
    ref = oracle.layer_forward(x.reshape(-1, n).astype(np.float64), *term, dtype=np.float64).reshape(2, 70, m)
    for kind in ("gemv", "gemm"):
        mod = NanoQuantLinear.from_factors(f(term[0]), f(term[1]), f(term[2]), f(term[3]), f(term[4]), dtype=torch.float16).to(dev)
        mod._prepare_kernel(kind, torch.float16)
        print(f"3-D input through {kind}", flush=True)
        y = mod(torch.from_numpy(x).to(dev))
        torch.cuda.synchronize()
        assert y.shape == (2, 70, m) and y.dtype == torch.float16
        assert oracle.max_rel_err(y.float().cpu().numpy().reshape(-1, m), ref.reshape(-1, m)) < 1e-2
