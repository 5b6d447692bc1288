"""Host side of the drop-in boundary, no GPU: the C-ABI library loads and exports what the header
declares, the operator schemas/meta kernels/error behaviour match the reference's, the prefill
packer's tile layout is what the kernel documentation says, and the module mirror keeps the
reference's protocol.  No compute entry point is called."""
import ctypes

import numpy as np
import pytest
import torch

import binary_kernels  # noqa: F401  (the name the reference imports)
import nanoquant_amd
from nanoquant_amd import _lib, ops, packing
from nanoquant_amd.linear import MixtureOfRankLinear, NanoQuantLinear
from oracle import nq_oracle as oracle


# ---- C ABI -------------------------------------------------------------------------------------
def test_library_exports_every_declared_symbol():
    names = _lib.declared_symbols()
    assert {"nq_gemv_forward", "nq_gemv_mixture", "nq_gemm_onebit", "nq_gemm_nanoquant", "nq_repack_words",
            "nq_status_string", "nq_stream_copy"} <= set(names)
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(handle, name), f"{name} declared in include/nq_gfx950.h but not exported"
    assert set(_lib._SIGNATURES) == set(names)


def test_status_strings_are_the_reference_messages():
    lib = _lib.lib()
    assert lib.nq_abi_version() >= 1
    assert lib.nq_status_string(0) == b"ok"
    assert lib.nq_status_string(-1) == b"Support only Half or BFloat16"       # cuda/gemv_kernel.cu:318
    assert lib.nq_status_string(-4) == b"k dimension mismatch"                # cuda/gemm.cpp:48
    assert lib.nq_status_string(-5) == b"Problem shape incompatible"          # cuda/gemm.cpp:93
    assert lib.nq_status_string(-6) == b"workspace too small"                 # cuda/gemm.cpp:52
    with pytest.raises(RuntimeError, match="k dimension mismatch"):
        _lib.check(-4)


def test_argument_errors_need_no_gpu():
    lib = _lib.lib()
    # dtype and size checks come before any HIP call
    assert lib.nq_gemv_forward(None, None, None, None, None, None, None, None, 1, 32, 32, 32, 7, None) == -1
    assert lib.nq_gemv_forward(None, None, None, None, None, None, None, None, 1, 32, 32, 32, 0, None) == -2
    assert lib.nq_gemv_forward(None, None, None, None, None, None, None, None, -1, 32, 32, 32, 0, None) == -3
    assert lib.nq_gemv_forward(None, None, None, None, None, None, None, None, 0, 32, 32, 32, 0, None) == 0
    assert lib.nq_gemm_onebit(None, None, None, None, None, None, 0, 8, 100, 64, 0, None) == -5   # k % 256
    assert lib.nq_gemm_onebit(None, None, None, None, None, None, 0, 8, 256, 48, 0, None) == -5   # rows % 32
    assert lib.nq_repack_words(None, None, 4, 0, 5, None) == -7
    assert lib.nq_stream_copy(None, None, 24, None) == -3
    assert lib.nq_gemm_scratch_bytes(128, 4096, 4096) in (0, 128 * 4096 * 4)


# ---- operator registration ------------------------------------------------------------------------
def test_schemas_are_the_reference_schemas():
    s = str(torch.ops.binary_kernels.nanoquant_dyn_forward.default._schema)
    assert "Tensor x, Tensor scale_g, Tensor Ubits, Tensor? scale_l, Tensor Vbits, Tensor scale_h" in s
    for frag in ("int num_thread_stage1=128", "int num_row_per_warp_stage2=2", "int num_acc_stage1=4",
                 "int num_pipeline_stage2=2"):
        assert frag in s
    s = str(torch.ops.binary_kernels.marlin_onebit_forward.default._schema)
    assert "Tensor x, Tensor weight, Tensor? scale_g, Tensor? scale_h, Tensor(a!) workspace" in s
    s = str(torch.ops.binary_kernels.marlin_nanoquant_forward.default._schema)
    assert "Tensor x, Tensor weight_u, Tensor weight_v, Tensor? scale_g, Tensor? scale_l, Tensor? scale_h, Tensor(a!) workspace" in s
    assert ops.get_kernel_function("nanoquant", torch.float16, "dynamic") is torch.ops.binary_kernels.nanoquant_dyn_forward
    with pytest.raises(AttributeError, match="Dispatcher op `nope::nope_dyn_forward` not found"):
        ops.get_kernel_function("nope", torch.float16, "dynamic")


def test_meta_kernels_give_output_shapes():
    mt = lambda *shape, dtype=torch.float16: torch.empty(*shape, dtype=dtype, device="meta")
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(mt(3, 64), mt(64), mt(32, 2, dtype=torch.int32), None,
                                                       mt(96, 1, dtype=torch.int32), mt(96))
    assert y.shape == (3, 96) and y.dtype == torch.float16
    y = torch.ops.binary_kernels.nanoquant_dyn_forward(mt(64), mt(64), mt(32, 2, dtype=torch.int32), mt(32),
                                                       mt(96, 1, dtype=torch.int32), mt(96))
    assert y.shape == (96,)
    ws = mt(64, dtype=torch.int32)
    y = torch.ops.binary_kernels.marlin_onebit_forward(mt(5, 512), mt(32, 128, dtype=torch.int32), mt(512), mt(256), ws)
    assert y.shape == (5, 256)
    y = torch.ops.binary_kernels.marlin_nanoquant_forward(mt(5, 512), mt(32, 128, dtype=torch.int32),
                                                          mt(16, 64, dtype=torch.int32), mt(512), mt(256), mt(128), ws)
    assert y.shape == (5, 128)
    with pytest.raises(RuntimeError, match="k dimension mismatch"):
        torch.ops.binary_kernels.marlin_onebit_forward(mt(5, 500), mt(32, 128, dtype=torch.int32), None, None, ws)
    with pytest.raises(RuntimeError, match="s_in size mismatch"):
        torch.ops.binary_kernels.marlin_onebit_forward(mt(5, 512), mt(32, 128, dtype=torch.int32), mt(511), None, ws)
    with pytest.raises(RuntimeError, match="s_out size mismatch"):
        torch.ops.binary_kernels.marlin_onebit_forward(mt(5, 512), mt(32, 128, dtype=torch.int32), None, mt(255), ws)
    with pytest.raises(RuntimeError, match="workspace too small"):
        torch.ops.binary_kernels.marlin_onebit_forward(mt(5, 512), mt(32, 128, dtype=torch.int32), None, None,
                                                       mt(63, dtype=torch.int32))


def test_decode_op_argument_checks():
    f16 = lambda *s: torch.zeros(*s, dtype=torch.float16)
    i32 = lambda *s: torch.zeros(*s, dtype=torch.int32)
    args = (f16(1, 64), f16(64), i32(32, 2), None, i32(96, 1), f16(96))
    with pytest.raises(RuntimeError, match="Support only Half or BFloat16"):
        ops.nanoquant_dyn_forward(torch.zeros(1, 64), *args[1:])
    with pytest.raises(RuntimeError, match="x must be a CUDA tensor"):
        ops.nanoquant_dyn_forward(*args)
    # the CPU dispatch key has no kernel: there is no host fallback
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.binary_kernels.nanoquant_dyn_forward(*args)
    # legal sets of the tuning hints (cuda/gemv_kernel.cu:351-354); message format of cuda/meta_utils.h:36
    with pytest.raises(ValueError, match=r"n_th1 should be one of \[64, 128, 256\], but 96 was given"):
        ops._sweep("n_th1", 96)
    with pytest.raises(ValueError, match=r"n_pipe2 should be one of \[1, 2, 4, 8, 16\], but 3 was given"):
        ops._sweep("n_pipe2", 3)
    with pytest.raises(ValueError, match="n_rpw1 should be one of"):
        ops._sweep("n_rpw1", 16)
    for ok in (1, 2, 4):
        ops._sweep("n_acc1", ok)


# ---- prefill packer --------------------------------------------------------------------------------
def test_gemm_tile_layout_element_by_element():
    rng = np.random.default_rng(0)
    out, k = 64, 512
    w = (rng.integers(0, 2, size=(out, k), dtype=np.int8) * 2 - 1).astype(np.int8)
    words = packing.pack_gemm_tiles(torch.from_numpy(w)).numpy().view(np.uint32)
    assert words.shape == (out * k // 32,)
    ktiles = k // 256
    for _ in range(400):
        row, col = int(rng.integers(out)), int(rng.integers(k))
        rt, kt = row // 32, col // 256
        kk = col % 256
        t, half, e = kk // 16, (kk % 16) // 8, kk % 8      # MFMA k-step, lane half, element in the lane's 8
        lane = 32 * half + row % 32
        q, tp = t // 4, t % 4
        word = int(words[((rt * ktiles + kt) * 64 + lane) * 4 + q])
        bit = 15 - (4 * tp + e // 2) + 16 * (e % 2)
        assert ((word >> bit) & 1) == (1 if w[row, col] == -1 else 0)
    back = packing.unpack_gemm_tiles(torch.from_numpy(words.view(np.int32)), out, k).numpy()
    assert np.array_equal(back, w)


def test_prefill_packer_interface():
    n, r, m = 512, 100, 128
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 1)
    t = torch.from_numpy
    V_bits, U_bits, s1, s2, s3, ws = packing.marlin_nanoquant_packer(t(vt).T.contiguous(), t(u).T.contiguous(),
                                                                    t(s_in), t(s_mid), t(s_out))
    rp = 256                                               # rank padded to a multiple of 256
    assert V_bits.shape == (n // 16, rp // 2) and U_bits.shape == (rp // 16, m // 2)
    assert V_bits.dtype == torch.int32 and ws.dtype == torch.int32 and ws.numel() == max(rp, m) // 128 * 32
    assert s2.numel() == rp and torch.all(s2[r:] == 0) and torch.equal(s2[:r], t(s_mid))
    # padded ranks carry +1 signs
    v_back = packing.unpack_gemm_tiles(V_bits, rp, n)
    assert torch.equal(v_back[:r], t(vt)) and torch.all(v_back[r:] == 1)
    u_back = packing.unpack_gemm_tiles(U_bits, m, rp)
    assert torch.equal(u_back[:, :r], t(u)) and torch.all(u_back[:, r:] == 1)
    with pytest.raises(ValueError, match="prefill packing needs"):
        packing.marlin_onebit_packer(torch.ones(48, 256, dtype=torch.int8), None, None)


# ---- module mirror -----------------------------------------------------------------------------------
def _module(m=64, n=96, r=32, seed=0, mid=True):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    t = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32))
    mod = NanoQuantLinear.from_factors(t(vt), t(u), t(s_in), t(s_mid) if mid else None, t(s_out), dtype=torch.float32)
    return mod, (vt, u, s_in, s_mid if mid else None, s_out)


def test_dense_forward_is_the_oracle_definition():
    mod, (vt, u, s_in, s_mid, s_out) = _module()
    x = oracle.synth_x(3, 96, 0).astype(np.float32)
    y = mod(torch.from_numpy(x)).numpy()
    assert np.allclose(y, oracle.layer_forward(x, vt, u, s_in, s_mid, s_out), rtol=1e-5, atol=1e-7)
    mod2, (vt, u, s_in, _, s_out) = _module(mid=False)
    assert not hasattr(mod2, "scale_mid")
    assert np.allclose(mod2(torch.from_numpy(x)).numpy(), oracle.layer_forward(x, vt, u, s_in, None, s_out),
                       rtol=1e-5, atol=1e-7)


def test_state_dict_uses_the_packed_checkpoint_format():
    mod, (vt, u, *_rest) = _module()
    sd = mod.state_dict()
    assert "V" not in sd and "U" not in sd
    assert sd["V_packed"].dtype == torch.int32 and tuple(sd["V_shape"]) == (32, 96) and tuple(sd["U_shape"]) == (64, 32)
    assert np.array_equal(sd["V_packed"].numpy(), oracle.pack_rows(vt, "lsb_first"))
    assert np.array_equal(sd["U_packed"].numpy(), oracle.pack_rows(u, "lsb_first"))
    assert sd["scale_pre"].shape == (1, 96) and sd["scale_mid"].shape == (1, 32)


def test_prepare_kernel_protocol_and_no_cpu_fallback():
    mod, (vt, u, *_rest) = _module()
    mod._prepare_kernel("gemv", torch.float16)
    assert mod.do_kernel_inference and mod.kernel_type == "gemv" and not hasattr(mod, "V") and not hasattr(mod, "U")
    assert np.array_equal(mod.V_int8.numpy(), oracle.pack_rows(vt, "half2"))
    assert np.array_equal(mod.U_int8.numpy(), oracle.pack_rows(u, "half2"))
    assert mod.scale_pre.shape == (96,) and mod.scale_pre.dtype == torch.float16
    assert mod.kernel_kwargs["num_acc_stage1"] == 1 and mod.kernel_kwargs["num_pipeline_stage2"] == 8
    assert mod.kernel_forward is torch.ops.binary_kernels.nanoquant_dyn_forward
    with pytest.raises(ValueError, match="Expected 2D or 3D input tensor"):
        mod(torch.zeros(96))
    with pytest.raises((NotImplementedError, RuntimeError)):   # CPU tensors: no kernel, no fallback
        mod(torch.zeros(1, 96))
    with pytest.raises(ValueError, match="kernel_type must be one of"):
        _module()[0]._prepare_kernel("fast")
    g, _ = _module(m=64, n=256, r=32)
    g._prepare_kernel("gemm", torch.float16)
    assert g.kernel_type == "gemm" and g.s2.numel() == 256 and not hasattr(g, "scale_pre")
    assert g.kernel_forward is torch.ops.binary_kernels.marlin_nanoquant_forward


def test_load_packed_goes_straight_to_kernel_words():
    mod, (vt, u, *_rest) = _module()
    sd = mod.state_dict()
    fresh = NanoQuantLinear(96, 64, 32, dtype=torch.float32)
    fresh.load_packed(sd, kernel_type="gemv", dtype=torch.float16)
    assert np.array_equal(fresh.V_int8.numpy(), oracle.pack_rows(vt, "half2"))
    assert np.array_equal(fresh.U_int8.numpy(), oracle.pack_rows(u, "half2"))
    assert fresh.kernel_type == "gemv" and fresh.scale_mid.shape == (32,)


def test_mixture_dense_path_is_the_sum():
    a, ta = _module(seed=1)
    b, tb = _module(r=64, seed=2)
    mix = MixtureOfRankLinear([a, b])
    x = oracle.synth_x(2, 96, 5).astype(np.float32)
    y = mix(torch.from_numpy(x)).numpy()
    assert np.allclose(y, oracle.mixture_forward(x, [ta, tb]), rtol=1e-5, atol=1e-7)


def test_ops_trace_under_fake_tensors_and_make_fx():
    # What torch.compile needs from a custom op: it runs on fake tensors of the device the real kernel serves,
    # and a traced graph holds the op itself (no decomposition, no host fallback).  No GPU is touched.
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.fx.experimental.proxy_tensor import make_fx

    def layer(x, s_in, vt_bits, s_mid, u_bits, s_out):
        return torch.ops.binary_kernels.nanoquant_dyn_forward(x, s_in, vt_bits, s_mid, u_bits, s_out, 128, 128, 2, 2,
                                                              1, 1, 8, 8)

    with FakeTensorMode(allow_non_fake_inputs=False) as mode:
        ft = lambda *shape, dtype=torch.float16: torch.empty(*shape, dtype=dtype, device="cuda")
        args = (ft(4, 256), ft(256), ft(128, 8, dtype=torch.int32), ft(128), ft(512, 4, dtype=torch.int32), ft(512))
        y = layer(*args)
        assert y.shape == (4, 512) and y.dtype == torch.float16 and y.device.type == "cuda"
        g = make_fx(layer, tracing_mode="real")(*args)
    targets = [n.target for n in g.graph.nodes if n.op == "call_function"]
    assert targets == [torch.ops.binary_kernels.nanoquant_dyn_forward.default]


def test_row_routing_and_run_list_options_need_no_gpu():
    """Host logic of the options added to the module and the run list: defaults, state checks, plan mirror."""
    import ctypes
    from nanoquant_amd.runlist import DecodeRunList, NqRunlistPlan
    vt, u, s_in, s_mid, s_out = oracle.synth_term(64, 256, 32, seed=9)
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid), f(s_out), dtype=torch.float32)
    assert mod.mfma_from_rows == 0 and mod._mfma_tiles is None
    with pytest.raises(RuntimeError, match="kernel_type='gemv'"):
        mod.prepare_mfma_route()                                       # not prepared for decode yet
    mod._prepare_kernel("gemv", torch.float16)
    mod.mfma_from_rows = 3
    assert not mod._routes_to_mfma(torch.zeros(8, 256))                # CPU tensors never route (and never build tiles)
    assert mod._mfma_tiles is None
    mod.prepare_mfma_route()                                           # the packing pass itself runs on any device
    dense = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid), f(s_out), dtype=torch.float32)
    dense._prepare_kernel("gemm", torch.float16)
    assert torch.equal(mod._mfma_tiles[0], dense.V_int8) and torch.equal(mod._mfma_tiles[1], dense.U_int8)
    odd = NanoQuantLinear.from_factors(f(vt[:, :96]), f(u), f(s_in[:96]), f(s_mid), f(s_out), dtype=torch.float32)
    odd._prepare_kernel("gemv", torch.float16)
    with pytest.raises(ValueError, match="in_features % 256"):
        odd.prepare_mfma_route()
    # the plan mirror has the library's layout (the library fills it; a mismatch would shift every field)
    names = [n for n, _ in NqRunlistPlan._fields_]
    assert names == ["nlinears", "nstages", "nphases", "workgroups", "max_units", "batch", "dtype", "index_words", "bound",
                     "spin_limit"]
    assert ctypes.sizeof(NqRunlistPlan) == 10 * ctypes.sizeof(ctypes.c_int)
    rl = DecodeRunList(4, torch.float16, "cpu", deterministic=True)
    assert rl.deterministic and rl.spin_limit == 0
    with pytest.raises(ValueError):
        DecodeRunList(3, torch.float16, "cpu")
    plan = NqRunlistPlan(batch=3, dtype=_lib.NQ_F16)
    assert _lib.lib().nq_runlist_set_deterministic(ctypes.byref(plan), 1) != 0      # no run-list kernel for 3 rows
    for b in (8, 16):
        plan = NqRunlistPlan(batch=b, dtype=_lib.NQ_BF16)
        assert _lib.lib().nq_runlist_set_deterministic(ctypes.byref(plan), 1) == 0 and plan.bound & 8
    plan = NqRunlistPlan(batch=4, dtype=_lib.NQ_F16)
    assert _lib.lib().nq_runlist_set_deterministic(ctypes.byref(plan), 1) == 0 and plan.bound & 8
    assert _lib.lib().nq_runlist_set_deterministic(ctypes.byref(plan), 0) == 0 and not plan.bound & 8
