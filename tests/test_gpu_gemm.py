"""Prefill path on the GPU against the oracle (torch.ops -> C ABI -> MFMA kernel)."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu

# max|y - y_ref| / max|y_ref| vs the fp32 dense reconstruction; the intermediate h is stored in the
# activation type between the two GEMMs (as the reference does), hence the 16-bit-output budget.
TOL = {torch.float16: 2e-3, torch.bfloat16: 1e-2}


def _cast(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a).astype(np.float32)).to(dtype)


def _run_fused(dev, m, n, r, tokens, dtype, seed):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    x = oracle.synth_x(tokens, n, seed)
    xt, si, sm, so = (_cast(a, dtype) for a in (x, s_in, s_mid, s_out))
    y_ref = oracle.layer_forward(xt.float().numpy(), vt, u, si.float().numpy(), sm.float().numpy(),
                                 so.float().numpy(), dtype=np.float32)
    print(f"case m={m} n={n} r={r} T={tokens} {dtype} seed={seed}", flush=True)
    packed = packing.marlin_nanoquant_packer(torch.from_numpy(vt).T.contiguous().to(dev),
                                             torch.from_numpy(u).T.contiguous().to(dev),
                                             si.to(dev), sm.to(dev), so.to(dev))
    y = torch.ops.binary_kernels.marlin_nanoquant_forward(xt.to(dev), *packed)
    torch.cuda.synchronize()
    assert y.shape == (tokens, m) and y.dtype == dtype
    return oracle.max_rel_err(y.float().cpu().numpy(), y_ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tokens", [128, 512])
def test_config0_shape(dev, dtype, tokens):
    err = _run_fused(dev, 2048, 2048, 1024, tokens, dtype, seed=0)
    assert err < TOL[dtype], err


@pytest.mark.parametrize("m,n,r,tokens", [
    (4096, 4096, 2048, 128),
    (11008, 4096, 2985, 128),   # rank padded to 3072 by the packer (zero mid scale on the padding)
    (4096, 11008, 2985, 128),
    (1024, 4096, 448, 128),
    (256, 256, 32, 1),          # a single token, rank padded 32 -> 256
    (320, 512, 100, 77),        # ragged tokens, rows not a multiple of 128
    (128, 768, 256, 200),
    (256, 4352, 256, 300),      # k of 17 tiles: few-token tiles beyond 256 tokens (wavefronts split k, no scratch)
    (256, 4352, 256, 1100),     # the same above 1024 tokens: block tiles with a k-split
    (384, 512, 1024, 640),      # 32-token blocks without k-split (few 64-token workgroups, short k)
])
def test_shapes_fp16(dev, m, n, r, tokens):
    err = _run_fused(dev, m, n, r, tokens, torch.float16, seed=m + r + tokens)
    assert err < TOL[torch.float16], err


def test_single_matrix_op_and_scales_optional(dev):
    rows, k, tokens = 192, 512, 40
    rng = np.random.default_rng(3)
    w = (rng.integers(0, 2, size=(rows, k), dtype=np.int8) * 2 - 1).astype(np.int8)
    x = rng.normal(size=(tokens, k)).astype(np.float16)
    s_in = (np.abs(rng.normal(0, 0.02, k)) + 1e-3).astype(np.float16)
    s_out = (np.abs(rng.normal(0, 0.02, rows)) + 1e-3).astype(np.float16)
    f = lambda a: torch.from_numpy(a).to(dev)
    bits, si, so, ws = packing.marlin_onebit_packer(f(w), f(s_in), f(s_out))
    assert bits.shape == (k // 16, rows // 2) and bits.dtype == torch.int32
    workspace = torch.zeros(max(ws, 1), dtype=torch.int32, device=dev)
    for use_in, use_out in [(True, True), (False, True), (True, False), (False, False)]:
        y = torch.ops.binary_kernels.marlin_onebit_forward(f(x), bits, si if use_in else None,
                                                           so if use_out else None, workspace)
        xs = x.astype(np.float64) * (s_in.astype(np.float64) if use_in else 1.0)
        ref = xs @ w.astype(np.float64).T * (s_out.astype(np.float64)[None, :] if use_out else 1.0)
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-3, (use_in, use_out)


def test_tile_bit_exactness_single_minus_one(dev):
    # One -1 in an otherwise all-(+1) matrix, probed with a one-hot activation: every (row, k) slot of
    # a tile must map to exactly one output element.
    rows, k = 64, 512
    ones_k = torch.ones(k, dtype=torch.float16, device=dev)
    workspace = torch.zeros(32, dtype=torch.int32, device=dev)
    rng = np.random.default_rng(0)
    probes = [(0, 0), (31, 255), (32, 256), (63, 511), (5, 8), (5, 15), (5, 16), (37, 263)]
    probes += [(int(rng.integers(rows)), int(rng.integers(k))) for _ in range(24)]
    for (row, col) in probes:
        w = np.ones((rows, k), dtype=np.int8)
        w[row, col] = -1
        bits, _, _, _ = packing.marlin_onebit_packer(torch.from_numpy(w).to(dev), None, None)
        x = torch.zeros((32, k), dtype=torch.float16, device=dev)
        x[:, col] = 1.0
        x[3, :] = 1.0   # one dense token row as well
        y = torch.ops.binary_kernels.marlin_onebit_forward(x, bits, None, None, workspace).float().cpu().numpy()
        expect = np.ones((32, rows), dtype=np.float32)
        expect[:, row] = -1.0
        expect[3, :] = k
        expect[3, row] = k - 2
        assert np.array_equal(y, expect), (row, col)


def test_k_split_matches_single_pass(dev):
    # small row count forces a k-split (atomic fp32 partial sums); large row count does not
    for (m, n, r) in [(128, 4096, 256), (4096, 512, 256)]:
        err = _run_fused(dev, m, n, r, 128, torch.float16, seed=m)
        assert err < TOL[torch.float16], (m, n, r, err)


def test_graph_replay_of_the_split_k_path(dev):
    # k-split partial sums live in a scratch that the finish kernel re-zeroes: replays of a captured call
    # must equal the eager result every time (no memset nodes involved, the scratch is never cleared by the host)
    m, n, r, tokens = 512, 4096, 512, 300
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 77)
    x = torch.from_numpy(oracle.synth_x(tokens, n, 78)).to(dev)
    f = lambda a: torch.from_numpy(a).to(dev)
    packed = packing.marlin_nanoquant_packer(torch.from_numpy(vt.T.copy()).to(dev), torch.from_numpy(u.T.copy()).to(dev),
                                             f(s_in), f(s_mid), f(s_out))
    op = torch.ops.binary_kernels.marlin_nanoquant_forward
    print("graph replay of marlin_nanoquant_forward", flush=True)
    eager = op(x, *packed).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        op(x, *packed)                       # the side stream's scratch exists before the capture
    side.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        y = op(x, *packed)
    for rep in range(4):
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager) or oracle.max_rel_err(y.float().cpu().numpy(), eager.float().cpu().numpy()) < 1e-3, rep
        op(x, *packed)                       # eager work between the replays
        torch.cuda.synchronize()
