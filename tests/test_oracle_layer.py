"""Pins the oracle's layer mathematics against what the mathematics fixes (no GPU).

A dropped scale, a wrong multiplication order, a transposed factor or a wrong sign convention fails
at least one of: the all-(+1) closed form, the one-hot rank-1 case, a pure-Python triple loop on tiny
shapes, the dense-weight closed form evaluated in float64, the bit-by-bit C restatement, exact
neutrality of rank padding, linearity and the multi-term sum.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import nq_oracle as oracle


def _rand_layer(m, n, r, seed, batch=2):
    vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, seed)
    x = oracle.synth_x(batch, n, seed)
    f64 = lambda a: a.astype(np.float64)
    return f64(x), vt, u, f64(s_in), f64(s_mid), f64(s_out)


def test_all_plus_one_closed_form():
    rng = np.random.default_rng(0)
    m, n, r = 5, 7, 3
    x = rng.normal(size=(2, n))
    s_in, s_mid, s_out = rng.uniform(0.5, 2, n), rng.uniform(0.5, 2, r), rng.uniform(0.5, 2, m)
    y = oracle.layer_forward(x, np.ones((r, n), np.int8), np.ones((m, r), np.int8), s_in, s_mid, s_out, np.float64)
    expect = (x * s_in).sum(1, keepdims=True) * s_mid.sum() * s_out[None, :]
    assert np.allclose(y, expect, rtol=1e-13)


def test_one_hot_mid_scale_is_rank_one():
    rng = np.random.default_rng(1)
    m, n, r = 6, 9, 32
    x, vt, u, s_in, _, s_out = _rand_layer(m, n, r, 4)
    s_mid = np.zeros(r)
    s_mid[11] = 1.7
    y = oracle.layer_forward(x, vt, u, s_in, s_mid, s_out, np.float64)
    expect = 1.7 * ((x * s_in) @ vt[11].astype(np.float64))[:, None] * (u[:, 11].astype(np.float64) * s_out)[None, :]
    assert np.allclose(y, expect, rtol=1e-12, atol=1e-15)


@pytest.mark.parametrize("m,n,r,batch", [(3, 4, 2, 1), (8, 5, 6, 3), (33, 40, 17, 2)])
def test_triple_loop(m, n, r, batch):
    x, vt, u, s_in, s_mid, s_out = _rand_layer(m, n, r, 7 + m, batch)
    y = oracle.layer_forward(x, vt, u, s_in, s_mid, s_out, np.float64)
    for b in range(batch):
        for j in range(m):
            acc = 0.0
            for i in range(r):
                h = 0.0
                for c in range(n):
                    h += float(vt[i, c]) * s_in[c] * x[b, c]
                acc += float(u[j, i]) * s_mid[i] * h
            assert abs(y[b, j] - s_out[j] * acc) <= 1e-12 * (1 + abs(y[b, j]))


def test_dense_weight_closed_form_and_none_mid():
    x, vt, u, s_in, s_mid, s_out = _rand_layer(24, 40, 16, 3)
    w = oracle.dense_weight(vt, u, s_in, s_mid, s_out)
    assert w.shape == (24, 40)
    assert np.allclose(oracle.layer_forward(x, vt, u, s_in, s_mid, s_out, np.float64), x @ w.T, rtol=1e-12)
    y_none = oracle.layer_forward(x, vt, u, s_in, None, s_out, np.float64)
    y_ones = oracle.layer_forward(x, vt, u, s_in, np.ones(16), s_out, np.float64)
    assert np.array_equal(y_none, y_ones)


def test_packed_path_equals_dense_and_c_restatement():
    m, n, r = 20, 70, 45        # ragged: n and r not multiples of 32
    x, vt, u, s_in, s_mid, s_out = _rand_layer(m, n, r, 5)
    y = oracle.layer_forward(x, vt, u, s_in, s_mid, s_out, np.float64)
    for method in ("half2", "lsb_first"):
        vb, ub = oracle.pack_rows(vt, method), oracle.pack_rows(u, method)
        y_p = oracle.layer_forward_packed(x, s_in, vb, s_mid, ub, s_out, n=n, method=method, dtype=np.float64)
        assert np.allclose(y_p, y, rtol=1e-12)
        # the C code reads the words bit by bit; padded columns/ranks carry no input so they vanish
        xp = np.zeros((x.shape[0], vb.shape[1] * 32))
        xp[:, :n] = x
        sp = np.zeros(vb.shape[1] * 32)
        sp[:n] = s_in
        y_c = c_oracle.layer_forward_packed(xp, sp, vb, s_mid, ub, s_out, method)
        assert np.allclose(y_c, y, rtol=1e-12)


def test_rank_padding_is_exactly_neutral():
    x, vt, u, s_in, s_mid, s_out = _rand_layer(16, 64, 37, 9)
    y = oracle.layer_forward(x, vt, u, s_in, s_mid, s_out, np.float64)
    for mult in (32, 128, 256):
        vt_p, u_p, mid_p = oracle.pad_rank(vt, u, s_mid, mult)
        assert vt_p.shape[0] % mult == 0 and u_p.shape[1] == vt_p.shape[0]
        assert np.all(vt_p[37:] == 1) and np.all(u_p[:, 37:] == 1) and np.all(mid_p[37:] == 0)
        assert np.array_equal(oracle.layer_forward(x, vt_p, u_p, s_in, mid_p, s_out, np.float64), y)


def test_linearity_and_mixture_sum():
    x, vt, u, s_in, s_mid, s_out = _rand_layer(12, 48, 20, 11)
    x2 = oracle.synth_x(2, 48, 99).astype(np.float64)
    f = lambda v: oracle.layer_forward(v, vt, u, s_in, s_mid, s_out, np.float64)
    assert np.allclose(f(2.5 * x - x2), 2.5 * f(x) - f(x2), rtol=1e-11, atol=1e-14)
    t2 = oracle.synth_term(12, 48, 8, 12)
    y_mix = oracle.mixture_forward(x, [(vt, u, s_in, s_mid, s_out), t2], np.float64)
    assert np.allclose(y_mix, f(x) + oracle.layer_forward(x, *t2, dtype=np.float64), rtol=1e-12)
    # a mixture equals one layer over the concatenated rank when the outer scales are shared
    vt_b, u_b, _, mid_b, _ = t2
    y_cat = oracle.layer_forward(x, np.concatenate([vt, vt_b]), np.concatenate([u, u_b], 1), s_in,
                                 np.concatenate([s_mid, mid_b.astype(np.float64)]), s_out, np.float64)
    y_two = oracle.mixture_forward(x, [(vt, u, s_in, s_mid, s_out), (vt_b, u_b, s_in, mid_b, s_out)], np.float64)
    assert np.allclose(y_cat, y_two, rtol=1e-12)


def test_torch_dense_path_equals_oracle():
    x, vt, u, s_in, s_mid, s_out = _rand_layer(32, 64, 24, 13)
    t = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float64))
    y_t = oracle.torch_dense_forward(t(x), t(vt), t(u), t(s_in), t(s_mid), t(s_out)).numpy()
    assert np.allclose(y_t, oracle.layer_forward(x, vt, u, s_in, s_mid, s_out, np.float64), rtol=1e-12)


def test_rank_rules():
    assert oracle.nominal_rank(2048, 2048) == 1024
    assert oracle.nominal_rank(4096, 4096) == 2048
    assert oracle.nominal_rank(11008, 4096) == 2985
    assert oracle.nominal_rank(8192, 28672) == 6372 and oracle.nominal_rank(1024, 8192) == 910
    # checkpoint rule: budget / (a + b) - 16, floored to a multiple of 32 (utils/utils.py:132-159)
    assert oracle.checkpoint_rank(4096, 4096, 1.0) == 2016
    assert oracle.checkpoint_rank(4096, 11008, 1.0) == 2944
    assert oracle.checkpoint_rank(4096, 4096, 1.0, num_scales=3) == ((4096 * 4096 - 16 * 8192) // (8192 + 16)) // 32 * 32
    assert oracle.checkpoint_rank(64, 64, 0.1) == 32


def test_max_rel_err_metric():
    ref = np.array([[1.0, -4.0]])
    assert oracle.max_rel_err(ref + np.array([[0.02, 0.0]]), ref) == pytest.approx(0.005)


# ---- the fp8 input format of the run-list kernel ------------------------------------------------------
def test_fp8_rounding_matches_the_library_type():
    # every finite e4m3 number is a fixed point; random values and all midpoints round as torch's type does
    bits = torch.arange(256, dtype=torch.uint8)
    vals = bits.view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    vals = vals[np.isfinite(vals)]
    assert len(vals) == 254 and np.abs(vals).max() == 448.0
    assert np.array_equal(oracle.fp8_e4m3_round(vals), vals)
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(0, 50, 20000), rng.normal(0, 0.01, 20000), rng.uniform(-448, 448, 20000)])
    x = x[np.abs(x) <= 448].astype(np.float32).astype(np.float64)
    t = torch.from_numpy(x).float().to(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    assert np.array_equal(oracle.fp8_e4m3_round(x), t)
    grid = np.unique(np.abs(vals))
    mid = (grid[:-1] + grid[1:]) / 2            # ties go to the even mantissa
    t = torch.from_numpy(mid).float().to(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    assert np.array_equal(oracle.fp8_e4m3_round(mid), t)


def test_three_fp8_pieces_reproduce_the_input():
    # q0 + q1 + q2 = u up to 2^-12 relative, or the subnormal floor 2^-10 absolute (2^-17 of a maximum >= 128)
    rng = np.random.default_rng(1)
    u = np.concatenate([rng.uniform(-255.9, 255.9, 100000), rng.normal(0, 1e-2, 20000), [0.0, 255.99, -128.0, 2.0 ** -9]])
    q = oracle.fp8_pieces(u, 3)
    assert np.abs(q).max() <= 256               # never near the format's 448
    err = np.abs(q.sum(axis=0) - u)
    assert np.all(err <= np.maximum(2.0 ** -12 * np.abs(u), 2.0 ** -10))
    # two pieces are not enough for the 1e-3 budget of the layer (worst element 2^-9), three are
    assert np.max(np.abs(oracle.fp8_pieces(u, 2).sum(axis=0) - u) / np.maximum(np.abs(u), 1.0)) > 1e-3
    # a whole vector: scaled by a power of two, so the decomposition of v is that of v * S
    v = rng.normal(0, 0.02, (2, 512))
    sv = oracle.staged_input(v)
    assert np.all(np.abs(sv - v) <= np.maximum(2.0 ** -12 * np.abs(v), 2.0 ** -17 * np.abs(v).max(axis=1, keepdims=True)))
    assert np.array_equal(oracle.staged_input(v * 8.0), sv * 8.0)
    assert np.array_equal(oracle.staged_input(np.zeros((1, 64))), np.zeros((1, 64)))


def test_error_figures_known_answers():
    ref = np.array([3.0, -4.0, 0.0, 5.0])                              # rms = sqrt(50 / 4)
    y = ref + np.array([0.0, 0.5, 0.25, -1.0])
    floor = 0.1 * np.sqrt(12.5)
    assert oracle.max_rel_err(y, ref) == pytest.approx(1.0 / 5.0)
    assert oracle.elementwise_err(y, ref) == pytest.approx(max(0.5 / (4 + floor), 0.25 / floor, 1.0 / (5 + floor)))
    assert oracle.elementwise_err(y, ref, floor_frac=1.0) == pytest.approx(1.0 / (5 + np.sqrt(12.5)))
    assert oracle.elementwise_err(ref, ref) == 0.0
    assert oracle.elementwise_err(np.array([0.5]), np.zeros(1)) == 0.5   # a zero reference: the absolute error
