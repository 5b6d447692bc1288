"""The allocation-free decode entry point (`nq_gemv_forward_noalloc`, intermediate in a device array inside the
library) against the entry point it is a variant of (`nq_gemv_forward_bias`, intermediate in a caller's buffer):
same kernels, so the outputs must agree bit for bit wherever the kernels are deterministic (pieces of up to 4 batch
rows; larger pieces finish their row sums with LDS float atomics, whose order varies, and are held to 1e-3 of the
output maximum).  Two calls in a row, the second on a smaller input, so that what the first left in the shared
array cannot leak into the second."""
import ctypes

import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import _lib, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu
vp = ctypes.c_void_p


def _case(dev, m, n, r, batch, seed, dtype):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a).astype(np.float32)).to(dtype).to(dev)
    x = f(oracle.synth_x(batch, n, seed))
    bias = f(oracle.synth_x(1, m, seed + 1)[0])
    vt_bits = packing.binary_packer(torch.from_numpy(vt), "half2").to(dev)
    u_bits = packing.binary_packer(torch.from_numpy(u), "half2").to(dev)
    ref = oracle.layer_forward(x.double().cpu().numpy(), vt, u, f(s_in).double().cpu().numpy(), f(s_mid).double().cpu().numpy(),
                               f(s_out).double().cpu().numpy(), dtype=np.float64) + bias.double().cpu().numpy()
    return (x, f(s_in), vt_bits, f(s_mid), u_bits, f(s_out), bias), ref


def _both(dev, args, batch, n, r, m, dtype):
    lib = _lib.lib()
    x, s_in, vt_bits, s_mid, u_bits, s_out, bias = args
    dt = _lib.NQ_F16 if dtype == torch.float16 else _lib.NQ_BF16
    stream = vp(torch.cuda.current_stream().cuda_stream)
    h = torch.empty((batch, r), dtype=torch.float32, device=dev)
    y_ref = torch.full((batch, m), float("nan"), dtype=dtype, device=dev)
    y_new = torch.full((batch, m), float("nan"), dtype=dtype, device=dev)
    p = lambda t: vp(t.data_ptr())
    st = lib.nq_gemv_forward_bias(p(x), p(s_in), p(vt_bits), p(s_mid), p(u_bits), p(s_out), p(bias), p(h), p(y_ref),
                                  batch, n, r, m, dt, stream)
    assert st == 0, _lib.status_message(st)
    st = lib.nq_gemv_forward_noalloc(p(x), p(s_in), p(vt_bits), p(s_mid), p(u_bits), p(s_out), p(bias), p(y_new),
                                     batch, n, r, m, dt, stream)
    assert st == 0, _lib.status_message(st)
    torch.cuda.synchronize()
    return y_ref, y_new


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_two_calls_in_a_row_second_smaller(dev, dtype):
    for (m, n, r, batch, seed) in ((1024, 2048, 1000, 4, 31), (512, 768, 300, 3, 32), (2048, 1024, 512, 16, 33), (256, 512, 96, 1, 34)):
        print(f"noalloc m={m} n={n} r={r} B={batch} {dtype}", flush=True)
        args, ref = _case(dev, m, n, r, batch, seed, dtype)
        y_ref, y_new = _both(dev, args, batch, n, r, m, dtype)
        assert not torch.isnan(y_new.float()).any()
        if batch <= 4:
            assert torch.equal(y_ref, y_new)
        else:
            scale = float(y_ref.float().abs().max())
            assert torch.allclose(y_ref.float(), y_new.float(), rtol=0, atol=1e-3 * scale)
        assert oracle.max_rel_err(y_new.float().cpu().numpy(), ref) < 1e-2


def test_limit_and_argument_errors(dev):
    lib = _lib.lib()
    limit = 256 * 1024
    # one float too many: refused before anything is launched (the pointers are never touched)
    assert lib.nq_gemv_forward_noalloc(None, None, None, None, None, None, None, None, 16, 64, limit // 16 + 1, 64, 0, None) == -9
    assert b"built-in scratch" in lib.nq_status_string(-9)
    assert lib.nq_gemv_forward_noalloc(None, None, None, None, None, None, None, None, 1, 64, 64, 64, 5, None) == -1
    assert lib.nq_gemv_forward_noalloc(None, None, None, None, None, None, None, None, 1, 64, 64, 64, 0, None) == -2
    assert lib.nq_gemv_forward_noalloc(None, None, None, None, None, None, None, None, 0, 64, 64, 64, 0, None) == 0
    # exactly at the limit is accepted
    m, n, r, batch = 64, 64, limit // 16, 16
    args, ref = _case(dev, m, n, r, batch, 35, torch.float16)
    y_ref, y_new = _both(dev, args, batch, n, r, m, torch.float16)
    assert oracle.max_rel_err(y_new.float().cpu().numpy(), ref) < 1e-2
