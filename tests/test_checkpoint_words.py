"""Checkpoint words -> kernel formats without a dense matrix.

The reference stores a layer as `lsb_first` words (src/nanoquant/modules/linear.py:288-321) and its loader unpacks
them to dense +-1 before packing again (src/nanoquant/utils/load_utils.py:269-293).  Here the words go straight to
the decode order (one bit permutation per word) and to the prefill tiles (one pass over the words); both must be
bit-identical to packing the unpacked factors.  The CPU tests pin the torch paths against the oracle, the GPU tests
pin the device kernels (`nq_repack_words`, `nq_pack_gemm_tiles`, `nq_gemv_stage`) against the same.
"""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import ops, packing
from nanoquant_amd.linear import NanoQuantLinear
from oracle import nq_oracle as oracle


def _signs(rows, cols, seed):
    return (np.random.default_rng(seed).integers(0, 2, (rows, cols)) * 2 - 1).astype(np.int8)


# ---- CPU: the torch paths -----------------------------------------------------------------------
@pytest.mark.parametrize("rows,cols,rows_p,k_p", [(32, 256, 32, 256), (40, 300, 64, 512), (96, 512, 256, 512),
                                                  (64, 200, 64, 256), (1, 1, 32, 256)])
@pytest.mark.parametrize("method", ["lsb_first", "half2"])
def test_tiles_from_words_equal_tiles_from_dense(rows, cols, rows_p, k_p, method):
    w = _signs(rows, cols, rows * 7 + cols)
    words = torch.from_numpy(oracle.pack_rows(w, method))
    dense = np.ones((rows_p, k_p), dtype=np.int8)
    dense[:rows, :cols] = w
    want = packing.pack_gemm_tiles(torch.from_numpy(dense))
    got = packing.pack_gemm_tiles_from_words(words, rows_p, k_p, method)
    assert got.dtype == torch.int32 and torch.equal(got, want)


def test_tiles_from_words_argument_errors():
    words = torch.zeros((32, 8), dtype=torch.int32)
    with pytest.raises(ValueError, match="prefill packing needs"):
        packing.pack_gemm_tiles_from_words(words, 32, 128)            # k_padded below the source
    with pytest.raises(ValueError, match="prefill packing needs"):
        packing.pack_gemm_tiles_from_words(words, 48, 256)            # rows_padded % 32
    with pytest.raises(ValueError, match="Unsupported method"):
        packing.pack_gemm_tiles_from_words(words, 32, 256, "msb_first")
    with pytest.raises(TypeError):
        packing.pack_gemm_tiles_from_words(words.to(torch.int64), 32, 256)


@pytest.mark.parametrize("m,n,r", [(64, 256, 32), (96, 512, 300), (128, 256, 256)])
def test_fused_packer_from_words_is_the_fused_packer(m, n, r):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed=m + r)
    f = torch.from_numpy
    want = packing.marlin_nanoquant_packer(f(vt).T.contiguous(), f(u).T.contiguous(), f(s_in), f(s_mid), f(s_out))
    got = packing.pack_binary_marlin_fused_from_words(f(oracle.pack_rows(vt, "lsb_first")), f(oracle.pack_rows(u, "lsb_first")),
                                                      r, f(s_in), f(s_mid), f(s_out))
    assert len(got) == 6
    for a, b in zip(got, want):
        assert a.shape == b.shape and a.dtype == b.dtype and torch.equal(a, b)


def _checkpoint_module(m, n, r, seed):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    f = torch.from_numpy
    mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in).float(), f(s_mid).float(), f(s_out).float(), dtype=torch.float32)
    return mod, (vt, u, s_in, s_mid, s_out)


def test_load_packed_for_the_prefill_path_never_unpacks():
    mod, (vt, u, s_in, s_mid, s_out) = _checkpoint_module(64, 256, 40, seed=3)
    sd = mod.state_dict()
    fresh = NanoQuantLinear(256, 64, 40, dtype=torch.float32)
    fresh.load_packed(sd, kernel_type="gemm", dtype=torch.float16)
    dense = NanoQuantLinear.from_factors(torch.from_numpy(vt), torch.from_numpy(u), torch.from_numpy(s_in).float(),
                                         torch.from_numpy(s_mid).float(), torch.from_numpy(s_out).float(), dtype=torch.float32)
    dense._prepare_kernel("gemm", torch.float16)
    assert fresh.kernel_type == "gemm" and not hasattr(fresh, "V") and not hasattr(fresh, "scale_pre")
    for name in ("V_int8", "U_int8", "s1", "s2", "s3", "workspace"):
        a, b = getattr(fresh, name), getattr(dense, name)
        assert a.shape == b.shape and a.dtype == b.dtype and torch.equal(a, b), name
    assert fresh.kernel_forward is torch.ops.binary_kernels.marlin_nanoquant_forward
    with pytest.raises(ValueError, match="in_features % 256"):
        other, _ = _checkpoint_module(64, 96, 32, seed=4)
        NanoQuantLinear(96, 64, 32, dtype=torch.float32).load_packed(other.state_dict(), kernel_type="gemm")


def test_load_packed_drops_lists_built_on_the_old_words():
    mod, _ = _checkpoint_module(64, 96, 32, seed=5)
    fresh = NanoQuantLinear(96, 64, 32, dtype=torch.float32)
    fresh._fused_lists, fresh._fused_tiled = {"stale": object()}, (None, None)
    fresh.load_packed(mod.state_dict(), kernel_type="gemv", dtype=torch.float16)
    assert fresh._fused_lists == {} and fresh._fused_tiled is None


# ---- GPU: the device kernels ----------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("nwords", [1, 3, 255, 257, 1 << 20, (1 << 20) + 17])
def test_device_repack_words(dev, nwords):
    rng = np.random.default_rng(nwords)
    words = rng.integers(-2**31, 2**31, nwords, dtype=np.int64).astype(np.int32)
    t = torch.from_numpy(words).to(dev)
    print(f"repack {nwords} words", flush=True)
    for src, dst in (("lsb_first", "half2"), ("half2", "lsb_first")):
        want = oracle.repack(words.reshape(1, -1), src, dst).reshape(-1)
        out = packing.repack_words(t, src, dst)                       # out of place
        assert out.data_ptr() != t.data_ptr()
        assert np.array_equal(out.cpu().numpy(), want)
        inplace = t.clone()                                           # in place through the C ABI
        from nanoquant_amd import _lib
        import ctypes
        st = _lib.lib().nq_repack_words(ctypes.c_void_p(inplace.data_ptr()), ctypes.c_void_p(inplace.data_ptr()), nwords,
                                        _lib.ORDER_IDS[src], _lib.ORDER_IDS[dst],
                                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == 0
        torch.cuda.synchronize()
        assert np.array_equal(inplace.cpu().numpy(), want)
    assert np.array_equal(t.cpu().numpy(), words)                     # the source is untouched


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols,rows_p,k_p", [(40, 300, 64, 512), (2985, 4096, 3072, 4096), (4096, 2985, 4096, 3072),
                                                  (32, 256, 32, 256)])
@pytest.mark.parametrize("method", ["lsb_first", "half2"])
def test_device_tiles_from_words(dev, rows, cols, rows_p, k_p, method):
    w = _signs(rows, cols, rows + cols)
    words = torch.from_numpy(oracle.pack_rows(w, method))
    want = packing.pack_gemm_tiles_from_words(words, rows_p, k_p, method)           # CPU path, pinned above
    print(f"tiles from words {rows}x{cols} -> {rows_p}x{k_p} {method}", flush=True)
    got = packing.pack_gemm_tiles_from_words(words.to(dev), rows_p, k_p, method)
    assert got.is_cuda and torch.equal(got.cpu(), want)
    if rows == rows_p and cols == k_p:
        assert torch.equal(got.cpu(), packing.pack_gemm_tiles(torch.from_numpy(w)))


@pytest.mark.gpu
@pytest.mark.parametrize("kernel_type,batch", [("gemv", 3), ("gemm", 130)])
def test_load_packed_on_the_device_serves_the_checkpoint(dev, kernel_type, batch):
    m, n, r = 512, 768, 300
    mod, term = _checkpoint_module(m, n, r, seed=11)
    sd = {k: v.to(dev) for k, v in mod.state_dict().items()}
    fresh = NanoQuantLinear(n, m, r, dtype=torch.float32, device=dev)
    fresh.load_packed(sd, kernel_type=kernel_type, dtype=torch.float16)
    assert not hasattr(fresh, "V") and fresh.V_int8.is_cuda
    x = oracle.synth_x(batch, n, seed=12)
    print(f"load_packed {kernel_type} m={m} n={n} r={r} rows={batch}", flush=True)
    y = fresh(torch.from_numpy(x).to(dev))
    torch.cuda.synchronize()
    ref = oracle.layer_forward(x.astype(np.float64), *term, dtype=np.float64)
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch,rows,cols", [(1, 256, 512), (3, 300, 1000), (16, 2048, 4096)])
def test_single_stage_entry_point(dev, dtype, batch, rows, cols):
    """`nq_gemv_stage`: one launch of the reference's two (kernel/cuda/gemv_kernel.cu:283-301)."""
    rng = np.random.default_rng(rows + cols)
    w = _signs(rows, cols, rows * 3 + cols)
    x = torch.from_numpy(rng.standard_normal((batch, cols)).astype(np.float32)).to(dtype)
    s_col = torch.from_numpy((np.abs(rng.standard_normal(cols)) * 0.02 + 1e-3).astype(np.float32)).to(dtype)
    s_row = torch.from_numpy((np.abs(rng.standard_normal(rows)) * 0.02 + 1e-3).astype(np.float32)).to(dtype)
    bits = packing.binary_packer(torch.from_numpy(w), "half2").to(dev)
    print(f"stage rows={rows} cols={cols} B={batch} {dtype}", flush=True)
    y = ops.gemv_stage_forward(x.to(dev), s_col.to(dev), bits, s_row.to(dev))
    y_plain = ops.gemv_stage_forward(x.to(dev), None, bits, None)
    torch.cuda.synchronize()
    xs = x.double().numpy() * s_col.double().numpy()
    ref = (xs @ w.astype(np.float64).T) * s_row.double().numpy()
    ref_plain = x.double().numpy() @ w.astype(np.float64).T
    assert y.shape == (batch, rows) and y.dtype == dtype
    assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < 1e-2
    assert oracle.max_rel_err(y_plain.float().cpu().numpy(), ref_plain) < 1e-2
