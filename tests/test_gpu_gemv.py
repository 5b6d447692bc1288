"""Decode path on the GPU against the oracle (calls go through torch.ops -> C ABI -> HIP)."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import ops, packing
from oracle import c_oracle
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu

# max|y - y_ref| / max|y_ref| against the fp32 dense reconstruction.  The stated tolerance is 1e-2 on
# 16-bit outputs.  The fp16 kernels are additionally held to the fp32-accumulate budget of 1e-3
# whenever the rank is large enough (>= 256) for the fp16 rounding of the individual operands to
# average out; below that the output's own fp16 rounding (2^-11) is a visible part of the budget.
TOL = {torch.float16: 1e-2, torch.bfloat16: 1e-2}
TIGHT = 1e-3


def _tol(dtype, r):
    return TIGHT if (dtype == torch.float16 and r >= 256) else TOL[dtype]
HINTS = dict(num_thread_stage1=128, num_thread_stage2=128, num_row_per_warp_stage1=2, num_row_per_warp_stage2=2,
             num_acc_stage1=1, num_acc_stage2=1, num_pipeline_stage1=8, num_pipeline_stage2=8)


def _np_dtype_cast(a, dtype):
    t = torch.from_numpy(np.ascontiguousarray(a).astype(np.float32))
    return t.to(dtype)


def _run(dev, m, n, r, batch, dtype, seed, with_mid=True):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    x = oracle.synth_x(batch, n, seed)
    xt, si, sm, so = (_np_dtype_cast(a, dtype) for a in (x, s_in, s_mid, s_out))
    if not with_mid:
        sm = None
    # the oracle sees exactly the rounded operands the kernel sees
    y_ref = oracle.layer_forward(xt.float().numpy(), vt, u, si.float().numpy(),
                                 None if sm is None else sm.float().numpy(), so.float().numpy(), dtype=np.float64)
    vt_bits = packing.binary_packer(torch.from_numpy(vt), "half2").to(dev)
    u_bits = packing.binary_packer(torch.from_numpy(u), "half2").to(dev)
    print(f"case m={m} n={n} r={r} B={batch} {dtype} seed={seed} mid={with_mid}", flush=True)
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(
        xt.to(dev), si.to(dev), vt_bits, None if sm is None else sm.to(dev), u_bits, so.to(dev), **HINTS)
    torch.cuda.synchronize()
    assert y.shape == (batch, m) and y.dtype == dtype
    return oracle.max_rel_err(y.float().cpu().numpy(), y_ref), y, y_ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 4, 16])
def test_config0_shape(dev, dtype, batch):
    err, _, _ = _run(dev, 2048, 2048, 1024, batch, dtype, seed=0)
    assert err < _tol(dtype, 1024), err


@pytest.mark.parametrize("m,n,r", [
    (4096, 4096, 2048),      # Llama-2-7B q/k/v/o
    (11008, 4096, 2976),     # gate/up at a rank of 93 words (not a multiple of 4 words)
    (4096, 11008, 3008),     # down
    (1024, 4096, 448),       # GQA k/v with a small rank
    (96, 160, 64),           # tiny: fewer units than lanes
    (40, 32, 32),            # rows not a multiple of anything
])
@pytest.mark.parametrize("batch", [1, 3, 8])
def test_shapes_fp16(dev, m, n, r, batch):
    err, _, _ = _run(dev, m, n, r, batch, torch.float16, seed=m + n + r + batch)
    assert err < _tol(torch.float16, r), err


def test_ragged_columns_and_rank(dev):
    # n and r not multiples of 32: the packers pad columns with +1 bits; padded columns must not count
    for (m, n, r, b) in [(64, 100, 50, 2), (33, 1000, 70, 1), (128, 4100, 2985, 5)]:
        err, _, _ = _run(dev, m, n, r, b, torch.float16, seed=n)
        assert err < _tol(torch.float16, r), (m, n, r, err)


def test_no_mid_scale_equals_ones(dev):
    err, y, _ = _run(dev, 256, 512, 128, 2, torch.float16, seed=5, with_mid=False)
    assert err < 2e-3, err


def test_batch_larger_than_16_and_1d(dev):
    err, _, _ = _run(dev, 512, 1024, 256, 37, torch.float16, seed=9)
    assert err < TIGHT, err
    vt, u, s_in, s_mid, s_out = oracle.synth_term(128, 256, 64, 3)
    x = oracle.synth_x(1, 256, 3)
    f = lambda a: torch.from_numpy(a).to(dev)
    y1 = torch.ops.binary_kernels.nanoquant_dyn_forward(
        f(x[0]), f(s_in), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), f(s_mid),
        packing.binary_packer(torch.from_numpy(u), "half2").to(dev), f(s_out), **HINTS)
    assert y1.shape == (128,)
    y_ref = oracle.layer_forward(x.astype(np.float32), vt, u, s_in, s_mid, s_out)[0]
    assert oracle.max_rel_err(y1.float().cpu().numpy(), y_ref) < 2e-3


def test_all_plus_one_closed_form(dev):
    # all-(+1) factors: y[mu] = s_out[mu] * sum(s_mid) * sum(s_in * x), independent of any bit order
    m, n, r = 64, 256, 96
    rng = np.random.default_rng(0)
    x = rng.normal(size=(2, n)).astype(np.float16)
    s_in = (np.abs(rng.normal(0, 0.02, n)) + 1e-3).astype(np.float16)
    s_mid = (np.abs(rng.normal(0, 0.02, r)) + 1e-3).astype(np.float16)
    s_out = (np.abs(rng.normal(0, 0.02, m)) + 1e-3).astype(np.float16)
    f = lambda a: torch.from_numpy(a).to(dev)
    zeros_v = torch.zeros((r, n // 32), dtype=torch.int32, device=dev)
    zeros_u = torch.zeros((m, r // 32), dtype=torch.int32, device=dev)
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(f(x), f(s_in), zeros_v, f(s_mid), zeros_u, f(s_out), **HINTS)
    expect = (x.astype(np.float64) * s_in.astype(np.float64)).sum(1, keepdims=True) * s_mid.astype(np.float64).sum() \
        * s_out.astype(np.float64)[None, :]
    # With identical signs nothing averages out: the three 16-bit roundings (x*s_in, h, y) of 2^-11
    # each add up coherently, so the bound is their sum rather than the random-sign budget of 1e-3.
    assert oracle.max_rel_err(y.float().cpu().numpy(), expect) < 3 * 2.0**-11 + 1e-4


def test_bit_index_exactness_single_minus_one(dev):
    # One -1 at (row, col) of the first factor flips exactly that column's contribution: checks the
    # kernel's bit indexing element by element against the packing definition (all 32 in-word slots).
    n, r, m = 128, 32, 32
    x = np.zeros((1, n), dtype=np.float16)
    ones = lambda k: torch.ones(k, dtype=torch.float16, device=dev)
    for col in list(range(32)) + [37, 64, 95, 127]:
        x[:] = 0
        x[0, col] = 1.0
        vt = np.ones((r, n), dtype=np.int8)
        vt[5, col] = -1
        u = np.ones((m, r), dtype=np.int8)
        vt_bits = packing.binary_packer(torch.from_numpy(vt), "half2").to(dev)
        u_bits = packing.binary_packer(torch.from_numpy(u), "half2").to(dev)
        y = torch.ops.binary_kernels.nanoquant_dyn_forward(torch.from_numpy(x).to(dev), ones(n), vt_bits, None,
                                                           u_bits, ones(m), **HINTS)
        # h = +1 everywhere except h[5] = -1  ->  y = r - 2
        assert torch.all(y == float(r - 2)), (col, y)


def test_against_c_oracle_from_packed_words(dev):
    # random words straight into the kernel; the C restatement evaluates the same words bit by bit
    rng = np.random.default_rng(11)
    m, n, r, b = 48, 96, 64, 2
    vt_bits = rng.integers(-2**31, 2**31, size=(r, n // 32), dtype=np.int64).astype(np.int32)
    u_bits = rng.integers(-2**31, 2**31, size=(m, r // 32), dtype=np.int64).astype(np.int32)
    x = rng.normal(size=(b, n)).astype(np.float16)
    s_in = (np.abs(rng.normal(0, 0.02, n)) + 1e-3).astype(np.float16)
    s_mid = (np.abs(rng.normal(0, 0.02, r)) + 1e-3).astype(np.float16)
    s_out = (np.abs(rng.normal(0, 0.02, m)) + 1e-3).astype(np.float16)
    f = lambda a: torch.from_numpy(a).to(dev)
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(f(x), f(s_in), f(vt_bits), f(s_mid), f(u_bits), f(s_out), **HINTS)
    y_ref = c_oracle.layer_forward_packed(x, s_in, vt_bits, s_mid, u_bits, s_out, "half2")
    assert oracle.max_rel_err(y.float().cpu().numpy(), y_ref) < 2e-3


def test_mixture_two_terms(dev):
    m, n = 512, 1024
    ranks = (192, 64)
    terms_np = [oracle.synth_term(m, n, r, seed=20 + i) for i, r in enumerate(ranks)]
    x = oracle.synth_x(3, n, 20)
    y_ref = oracle.mixture_forward(x.astype(np.float64), terms_np, dtype=np.float64)
    f = lambda a: torch.from_numpy(a).to(dev)
    terms = []
    for vt, u, s_in, s_mid, s_out in terms_np:
        terms.append((f(s_in), packing.binary_packer(torch.from_numpy(vt), "half2").to(dev), f(s_mid),
                      packing.binary_packer(torch.from_numpy(u), "half2").to(dev), f(s_out)))
    y = ops.gemv_mixture_forward(f(x), terms)
    assert oracle.max_rel_err(y.float().cpu().numpy(), y_ref) < 1e-3


def test_fp16_output_clamp(dev):
    # huge scales: the decode path saturates like the reference (clamp at +-64504 before rounding)
    m, n, r = 32, 64, 32
    big = torch.full((m,), 60000.0, dtype=torch.float16, device=dev)
    ones_n = torch.ones(n, dtype=torch.float16, device=dev)
    zv = torch.zeros((r, n // 32), dtype=torch.int32, device=dev)
    zu = torch.zeros((m, r // 32), dtype=torch.int32, device=dev)
    x = torch.ones((1, n), dtype=torch.float16, device=dev)
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(x, ones_n, zv, None, zu, big, **HINTS)
    assert torch.isfinite(y).all() and float(y.max()) == 64512.0
