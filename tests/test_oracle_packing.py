"""Pins the oracle's packing (and the product packers) without any GPU.

Checks, chosen so that a wrong bit table, a flipped sign convention, a transposed index or a wrong
padding value fails at least one of them:
  * hand-derived known-answer words and the committed fixture (tests/golden/packing_kat.json, written
    by a script that uses neither the oracle nor the package);
  * a brute-force per-element Python loop on seeded matrices;
  * invariants: unpack(pack(w)) == w, popcount(word) == number of -1 in the group, the two orders are
    related by a fixed bit permutation;
  * the scalar restatement of the device-side decode (kernel/cuda/cuda_utils.cuh:93-102) over all 2^8
    sign patterns of an 8-element slice at each of the 4 lane offsets;
  * the independent C restatement (oracle/nq_oracle.c).
"""
import json
import os

import numpy as np
import pytest
import torch

from nanoquant_amd import packing
from oracle import c_oracle
from oracle import nq_oracle as oracle

HERE = os.path.dirname(os.path.abspath(__file__))
METHODS = ("lsb_first", "half2")


def _u32(a):
    return np.asarray(a, dtype=np.int64) & 0xFFFFFFFF


def test_hand_derived_words():
    ones = np.ones((1, 32), dtype=np.int8)
    for method in METHODS:
        assert _u32(oracle.pack_rows(ones, method))[0, 0] == 0x00000000
        assert _u32(oracle.pack_rows(-ones, method))[0, 0] == 0xFFFFFFFF
        assert oracle.pack_rows(-ones, method)[0, 0] == -1
    expect = {0: (0x00000001, 0x00008000), 1: (0x00000002, 0x80000000), 31: (0x80000000, 0x00010000),
              2: (0x00000004, 0x00004000), 30: (0x40000000, 0x00000001)}
    for k, (lsb, h2) in expect.items():
        w = ones.copy()
        w[0, k] = -1
        assert _u32(oracle.pack_rows(w, "lsb_first"))[0, 0] == lsb
        assert _u32(oracle.pack_rows(w, "half2"))[0, 0] == h2
    w = np.ones((1, 32), dtype=np.int8)
    w[0, 1] = -1
    assert oracle.pack_rows(w, "half2")[0, 0] == -2147483648   # wraps into the int32 sign bit
    w40 = -np.ones((1, 40), dtype=np.int8)
    assert list(_u32(oracle.pack_rows(w40, "lsb_first"))[0]) == [0xFFFFFFFF, 0x000000FF]
    assert list(_u32(oracle.pack_rows(w40, "half2"))[0]) == [0xFFFFFFFF, 0xF000F000]


def test_bit_tables_match_reference_lists():
    # the `powers` lists of kernel/utils.py:99-104, written out
    assert [oracle.bit_position(k, "lsb_first") for k in range(32)] == list(range(32))
    h2 = [j for i in reversed(range(16)) for j in (i, i + 16)]
    assert h2[:6] == [15, 31, 14, 30, 13, 29] and h2[-2:] == [0, 16]
    assert [oracle.bit_position(k, "half2") for k in range(32)] == h2
    assert sorted(h2) == list(range(32))


@pytest.mark.parametrize("impl", ["oracle", "c", "product"])
def test_golden_fixture(impl):
    with open(os.path.join(HERE, "golden", "packing_kat.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 40
    for case in cases:
        signs = np.array(case["signs"], dtype=np.int8)
        for method in METHODS:
            want = np.array(case[method], dtype=np.int64).astype(np.int32)
            if impl == "oracle":
                got = oracle.pack_rows(signs, method)
                back = oracle.unpack_rows(want, signs.shape, method)
            elif impl == "c":
                got = c_oracle.pack_rows(signs, method)
                back = c_oracle.unpack_rows(want, signs.shape, method)
            else:
                got = packing.pack_binary_gemv(torch.from_numpy(signs), method).numpy()
                back = packing.unpack_binary_gemv(torch.from_numpy(want), signs.shape, method).numpy()
            assert got.dtype == np.int32 and np.array_equal(got, want), (case["name"], method, impl)
            assert np.array_equal(back, signs), (case["name"], method, impl)


def _brute_pack(signs, method):
    rows, cols = signs.shape
    words = (cols + 31) // 32
    out = np.zeros((rows, words), dtype=np.uint32)
    for r in range(rows):
        for c in range(cols):
            if signs[r, c] == -1:
                k = c % 32
                pos = k if method == "lsb_first" else 15 - k // 2 + 16 * (k % 2)
                out[r, c // 32] |= np.uint32(1 << pos)
    return out.view(np.int32)


@pytest.mark.parametrize("shape", [(1, 1), (3, 31), (4, 32), (5, 33), (7, 200), (2, 1024)])
def test_brute_force_and_invariants(shape):
    rng = np.random.default_rng(shape[0] * 1000 + shape[1])
    signs = (rng.integers(0, 2, size=shape, dtype=np.int8) * 2 - 1).astype(np.int8)
    packed = {}
    for method in METHODS:
        got = oracle.pack_rows(signs, method)
        assert np.array_equal(got, _brute_pack(signs, method))
        assert np.array_equal(c_oracle.pack_rows(signs, method), got)
        assert np.array_equal(packing.pack_binary_gemv(torch.from_numpy(signs), method).numpy(), got)
        assert np.array_equal(oracle.unpack_rows(got, shape, method), signs)
        assert np.array_equal(packing.unpack_binary_gemv(torch.from_numpy(got), shape, method).numpy(), signs)
        # popcount of each word = number of -1 in its group (padding contributes none)
        pop = np.array([[bin(int(v) & 0xFFFFFFFF).count("1") for v in row] for row in got])
        padded = np.ones((shape[0], got.shape[1] * 32), dtype=np.int8)
        padded[:, :shape[1]] = signs
        assert np.array_equal(pop, (padded.reshape(shape[0], -1, 32) == -1).sum(-1))
        packed[method] = got
    # the two orders differ by a fixed bit permutation
    assert np.array_equal(oracle.repack(packed["lsb_first"], "lsb_first", "half2"), packed["half2"])
    assert np.array_equal(oracle.repack(packed["half2"], "half2", "lsb_first"), packed["lsb_first"])
    assert np.array_equal(packing.repack_words(torch.from_numpy(packed["lsb_first"]), "lsb_first", "half2").numpy(),
                          packed["half2"])


def test_device_decode_restatement_all_patterns():
    # 8 consecutive elements, all 256 sign patterns, each of the 4 positions inside the 32-group
    x = np.arange(1, 9, dtype=np.float16)                # 8 distinct positive values
    xbits = x.view(np.uint16).astype(np.uint32)
    x4 = np.array([xbits[2 * c] | (xbits[2 * c + 1] << 16) for c in range(4)], dtype=np.uint32)
    for quad in range(4):
        for pattern in range(256):
            signs = np.ones((1, 32), dtype=np.int8)
            for e in range(8):
                if (pattern >> e) & 1:
                    signs[0, 8 * quad + e] = -1
            word = int(oracle.pack_rows(signs, "half2")[0, 0]) & 0xFFFFFFFF
            flipped = oracle.device_sign_flip_fp16(x4, word, quad)
            vals = []
            for c in range(4):
                vals.append(np.array([flipped[c] & 0xFFFF], dtype=np.uint16).view(np.float16)[0])
                vals.append(np.array([flipped[c] >> 16], dtype=np.uint16).view(np.float16)[0])
            want = x * signs[0, 8 * quad:8 * quad + 8].astype(np.float16)
            assert np.array_equal(np.array(vals, dtype=np.float16), want), (quad, pattern)


def test_errors_match_reference_behaviour():
    with pytest.raises(TypeError, match="Input tensor must be int8"):
        oracle.pack_rows(np.ones((2, 2), dtype=np.int32))
    with pytest.raises(TypeError, match="Input tensor must be int8"):
        packing.pack_binary_gemv(torch.ones(2, 2, dtype=torch.int32))
    with pytest.raises(ValueError, match="Unsupported method"):
        packing.pack_binary_gemv(torch.ones(2, 32, dtype=torch.int8), method="msb")
    with pytest.raises(ValueError, match="Expected 2D tensor"):
        packing.unpack_binary_gemv(torch.zeros(4, dtype=torch.int32), (1, 128))
    with pytest.raises(ValueError, match="Unsupported packed tensor shape"):
        packing.unpack_binary_gemv(torch.zeros(2, 3, dtype=torch.int32), (2, 128))
    with pytest.raises(ValueError, match="Unsupported packed tensor shape"):
        oracle.unpack_rows(np.zeros((2, 3), dtype=np.int32), (2, 128))


def test_empty_inputs():
    e = np.ones((0, 64), dtype=np.int8)
    assert oracle.pack_rows(e, "half2").shape == (0, 2)
    assert packing.pack_binary_gemv(torch.from_numpy(e), "half2").shape == (0, 2)
    z = np.ones((3, 0), dtype=np.int8)
    assert oracle.pack_rows(z, "half2").shape == (3, 0)
    assert packing.pack_binary_gemv(torch.from_numpy(z), "half2").shape == (3, 0)


# ---- tile order of the run list -----------------------------------------------------------------------
@pytest.mark.parametrize("rows,words", [(1, 1), (16, 4), (33, 17), (70, 47), (64, 16), (5, 94)])
def test_tile_order_matches_the_index_formula_and_round_trips(rows, words):
    import torch

    from nanoquant_amd import packing
    rng = np.random.default_rng(rows * 131 + words)
    a = rng.integers(-2 ** 31, 2 ** 31 - 1, (rows, words), dtype=np.int64).astype(np.int32)
    t = packing.tile_words(torch.from_numpy(a))
    groups = (words + 15) // 16
    assert t.numel() == (rows + 31) // 32 * groups * 512
    assert np.array_equal(t.numpy(), oracle.tile_words(a))           # reshape/permute == per-element formula
    assert np.array_equal(packing.untile_words(t, (rows, words)).numpy(), a)
    # a wave-load (16 rows x 4 units of one 32-row tile) is 256 consecutive words
    if rows >= 16 and words >= 16:
        blk = t.numpy()[:256].reshape(4, 16, 4)                      # [unit, row, word]
        assert np.array_equal(blk[2, 5], a[5, 8:12])
