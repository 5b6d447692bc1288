"""Grouped prefill: several linears on the same tokens sharing their launches (nq_gemm_nanoquant_group), against
the dense definition and against the one-linear operator.  The reference launches each linear by itself
(src/nanoquant/modules/linear.py:131-133, src/nanoquant/kernel/cuda/gemm.cpp:112-122)."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import MixtureOfRankLinear, NanoQuantLinear, ops, packing, prefill_group
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
@pytest.mark.parametrize("tokens", [128, 77, 1, 150, 200, 320, 512])
def test_group_on_shared_tokens(dev, tokens, dtype):
    # q, k, v-like: one input, different widths and ranks (one rank padded by the packer); above 128 tokens the
    # group runs on block tiles (64 tokens; 200 leaves a ragged last block), every workgroup walking the whole k
    n = 1024
    shapes = [(1024, 512), (256, 100), (320, 256), (2048, 768)]
    terms = [_term(dev, m, n, r, 500 + i, dtype) for i, (m, r) in enumerate(shapes)]
    x = _cast(oracle.synth_x(tokens, n, 9), dtype)
    print(f"group shared tokens={tokens} {dtype}", flush=True)
    ys = ops.gemm_group_forward(x.to(dev), [p for p, _ in terms])
    torch.cuda.synchronize()
    for (m, r), (packed, ref), y in zip(shapes, terms, ys):
        assert y.shape == (tokens, m) and y.dtype == dtype
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref(x.float().numpy())) < TOL[dtype], (m, r)
        single = torch.ops.binary_kernels.marlin_nanoquant_forward(x.to(dev), *packed)
        if tokens <= 128:
            assert torch.equal(y, single), (m, r)          # the same tiles in the same order: bit-identical
        else:
            assert torch.allclose(y.float(), single.float(), rtol=1e-2, atol=1e-3 * float(single.float().abs().max()))


def test_group_with_own_inputs_bias_and_more_terms_than_one_launch_takes(dev):
    dtype, tokens = torch.float16, 96
    rng = np.random.default_rng(4)
    shapes = [(256 + 32 * (i % 3), 512 if i % 2 else 768, 64 + 32 * i) for i in range(19)]   # 19 > 16 terms per launch
    terms, xs, biases = [], [], []
    for i, (m, n, r) in enumerate(shapes):
        terms.append(_term(dev, m, n, r, 600 + i, dtype))
        xs.append(_cast(oracle.synth_x(tokens, n, 700 + i), dtype))
        biases.append(_cast(rng.normal(0, 0.05, m), dtype) if i % 2 == 0 else None)
    ys = ops.gemm_group_forward([x.to(dev) for x in xs], [p for p, _ in terms],
                                [None if b is None else b.to(dev) for b in biases])
    torch.cuda.synchronize()
    for (packed, ref), x, b, y in zip(terms, xs, biases, ys):
        want = ref(x.float().numpy())
        if b is not None:
            want = want + b.float().numpy()[None, :]
        assert oracle.max_rel_err(y.float().cpu().numpy(), want) < TOL[dtype]


def test_group_rejects_mismatched_inputs(dev):
    dtype = torch.float16
    (p0, _), (p1, _) = _term(dev, 256, 512, 64, 1, dtype), _term(dev, 256, 768, 64, 2, dtype)
    x512 = torch.zeros((64, 512), dtype=dtype, device=dev)
    with pytest.raises(RuntimeError):
        ops.gemm_group_forward(x512, [p0, p1])                               # second term reads 768 columns
    with pytest.raises(RuntimeError):
        ops.gemm_group_forward([x512, torch.zeros((32, 768), dtype=dtype, device=dev)], [p0, p1])   # token counts differ
    with pytest.raises(RuntimeError):
        ops.gemm_group_forward([x512], [p0, p1])
    assert ops.gemm_group_forward(x512, []) == []


@pytest.mark.parametrize("ndim", [2, 3])
def test_prefill_group_of_modules(dev, ndim):
    dtype, n = torch.float16, 1024
    mods, refs = [], []
    for i, (m, r) in enumerate([(1024, 512), (512, 256), (512, 300)]):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 800 + i)
        bias = np.random.default_rng(i).normal(0, 0.05, m).astype(np.float32)
        f = lambda a: torch.from_numpy(a.astype(np.float32))
        mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid), f(s_out), bias=f(bias), dtype=dtype).to(dev)
        mod._prepare_kernel("gemm", dtype)
        mod.kernel_path_bias = (i == 1)
        mods.append(mod)
    x = _cast(oracle.synth_x(2 * 60, n, 12), dtype).to(dev)
    if ndim == 3:
        x = x.view(2, 60, n)
    ys = prefill_group(mods, x)
    torch.cuda.synchronize()
    for mod, y in zip(mods, ys):
        single = mod(x)
        assert y.shape == single.shape and torch.equal(y, single)
    unprepared = NanoQuantLinear(256, 256, 64, dtype=dtype)
    with pytest.raises(ValueError):
        prefill_group([mods[0], unprepared], x)


@pytest.mark.parametrize("tokens", [96, 200])
def test_prefill_group_with_a_mixture_module(dev, tokens):
    # a two-term weight and a plain linear on the same tokens: all three terms share the launches, the mixture's
    # output is the sum of its terms (the dense definition of a sum of low-rank terms)
    dtype, n = torch.float16, 768
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    make = lambda m, r, seed: (oracle.synth_term(m, n, r, seed))
    t0, t1, t2 = make(512, 192, 820), make(512, 64, 821), make(1024, 256, 822)
    mods = [NanoQuantLinear.from_factors(*(f(a) for a in t), dtype=dtype).to(dev) for t in (t0, t1, t2)]
    mix = MixtureOfRankLinear(mods[:2])
    mix._prepare_kernel("gemm", dtype)
    mods[2]._prepare_kernel("gemm", dtype)
    x = oracle.synth_x(tokens, n, 13)
    xt = _cast(x, dtype).to(dev)
    print(f"group with mixture tokens={tokens}", flush=True)
    y_mix, y_plain = prefill_group([mix, mods[2]], xt)
    y_fwd = mix(xt)
    torch.cuda.synchronize()
    xf = xt.float().cpu().numpy()
    ref_mix = oracle.mixture_forward(xf.astype(np.float64), [t0, t1], dtype=np.float64)
    ref_plain = oracle.layer_forward(xf.astype(np.float64), *t2, dtype=np.float64)
    assert y_mix.shape == (tokens, 512) and y_plain.shape == (tokens, 1024)
    assert oracle.max_rel_err(y_mix.float().cpu().numpy(), ref_mix) < TOL[dtype]
    assert oracle.max_rel_err(y_fwd.float().cpu().numpy(), ref_mix) < TOL[dtype]
    assert oracle.max_rel_err(y_plain.float().cpu().numpy(), ref_plain) < TOL[dtype]


def test_prefill_harness_on_a_tiny_layer(dev):
    from nanoquant_amd import bench_prefill
    rows = bench_prefill.run(["--model_shape", "tiny", "--tokens", "32,160", "--iters", "2", "--reps", "2"])
    assert [r["tokens"] for r in rows] == [32, 160]
    for r in rows:
        assert r["one_by_one"]["us_per_layer"] > 0 and r["grouped"]["us_per_layer"] > 0


def test_group_sum_with_uneven_term_counts_and_bias(dev):
    # three weights with 2, 1 and 3 terms: the flat output buffers put weights with more terms first; every weight
    # must still come back in its own position and equal the sum of its terms (dense definition, fp64)
    dtype, tokens, n = torch.float16, 100, 512
    spec = [(256, [64, 32]), (512, [128]), (320, [96, 64, 32])]
    rng = np.random.default_rng(8)
    groups, refs, bias_groups = [], [], []
    x = _cast(oracle.synth_x(tokens, n, 21), dtype)
    for w, (m, ranks) in enumerate(spec):
        terms, ref, biases = [], 0.0, []
        for t, r in enumerate(ranks):
            packed, f = _term(dev, m, n, r, 900 + 10 * w + t, dtype)
            terms.append(packed)
            ref = ref + f(x.float().numpy().astype(np.float64))
            if w == 2 and t == 1:
                b = _cast(rng.normal(0, 0.05, m), dtype)
                biases.append(b.to(dev))
                ref = ref + b.float().numpy()[None, :]
            else:
                biases.append(None)
        groups.append(terms)
        refs.append(ref)
        bias_groups.append(biases)
    print("group sum 2/1/3 terms", flush=True)
    ys = ops.gemm_group_sum_forward(x.to(dev), groups, bias_groups)
    torch.cuda.synchronize()
    for (m, _), y, ref in zip(spec, ys, refs):
        assert y.shape == (tokens, m) and y.dtype == dtype
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref) < TOL[dtype]
    with pytest.raises(RuntimeError):
        ops.gemm_group_sum_forward(x.to(dev), [groups[0], []])


@pytest.mark.parametrize("tokens", [64, 300])
def test_group_through_the_c_abi_without_scratch(dev, tokens):
    # nq_gemm_nanoquant_group called directly with raw pointers and scratch = NULL: groups whose terms all have input
    # scales need no scratch at any token count; null pointers, duplicate outputs and oversized groups are refused
    import ctypes
    from nanoquant_amd import _lib
    lib = _lib.lib()
    dtype, n = torch.float16, 512
    shapes = [(256, 64), (512, 128)]
    x = _cast(oracle.synth_x(tokens, n, 31), dtype).to(dev)
    items, keep, refs = [], [], []
    for i, (m, r) in enumerate(shapes):
        packed, ref = _term(dev, m, n, r, 950 + i, dtype)
        wu, wv, sg, sl, sh, _ = packed
        rp = wu.size(1) * 2                                   # rank as padded by the packer
        h = torch.empty(tokens, rp, dtype=dtype, device=dev)
        y = torch.empty(tokens, m, dtype=dtype, device=dev)
        keep += [packed, h, y]
        refs.append((y, ref))
        items.append(ops.NqGemmTerm(x.data_ptr(), wu.data_ptr(), wv.data_ptr(), sg.data_ptr(), sl.data_ptr(), sh.data_ptr(),
                                    None, h.data_ptr(), y.data_ptr(), n, rp, m))
    arr = (ops.NqGemmTerm * len(items))(*items)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    print(f"group via C ABI tokens={tokens}", flush=True)
    assert lib.nq_gemm_nanoquant_group(arr, len(items), tokens, _lib.NQ_F16, None, 0, stream) == 0
    torch.cuda.synchronize()
    for y, ref in refs:
        assert oracle.max_rel_err(y.float().cpu().numpy(), ref(x.float().cpu().numpy())) < TOL[dtype]
    dup = (ops.NqGemmTerm * 2)(items[0], items[0])            # same h / y twice
    assert lib.nq_gemm_nanoquant_group(dup, 2, tokens, _lib.NQ_F16, None, 0, stream) != 0
    assert lib.nq_gemm_nanoquant_group(None, 2, tokens, _lib.NQ_F16, None, 0, stream) != 0
    assert lib.nq_gemm_nanoquant_group(arr, int(lib.nq_gemm_group_max()) + 1, tokens, _lib.NQ_F16, None, 0, stream) != 0
    assert lib.nq_gemm_nanoquant_group(arr, 0, tokens, _lib.NQ_F16, None, 0, stream) == 0
