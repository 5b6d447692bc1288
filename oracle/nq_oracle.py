"""CPU oracle for the binary low-rank linear layer.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import it.  Nothing under nanoquant_amd/ or
binary_kernels/ imports it, and the product path raises when the HIP library is missing
instead of falling back to anything here.

Each function restates one piece of the reference (paths relative to the reference
checkout):

  bit_position            src/nanoquant/kernel/utils.py:99-104   (the `powers` tables)
  pack_rows               src/nanoquant/kernel/utils.py:51-113   (pack_binary_gemv)
  unpack_rows             src/nanoquant/kernel/utils.py:116-183  (unpack_binary_gemv)
  device_sign_flip_fp16   src/nanoquant/kernel/cuda/cuda_utils.cuh:93-102 (apply_sign) with
                          shift_base = 4*(lane%4) as used at cuda/gemv_kernel.cu:114
  layer_forward           src/nanoquant/modules/linear.py:248-257 (_compute_forward)
  dense_weight            the closed form W = diag(s_out) U diag(s_mid) V diag(s_in)
  layer_forward_packed    unpack -> layer_forward (what the kernels must equal)
  mixture_forward         sum of single-term layer_forward results (the multi-term layer has
                          no code in the reference; it is defined as this sum)
  pad_rank                src/nanoquant/kernel/utils.py:262-271 (+1 signs, zero mid scale)
  nominal_rank / checkpoint_rank   round(mn/(m+n)) and src/nanoquant/utils/utils.py:132-159
  torch_dense_forward     the same _compute_forward with torch.nn.functional.linear on dense
                          +-1 factors: the reference's CPU path, timed as the CPU baseline
  fp8_e4m3_round / fp8_pieces / staged_input   no counterpart in the reference: the number format (OCP e4m3,
                          round to nearest even) and the three-piece decomposition, with one power-of-two scale
                          per block of 128 columns, in which the gfx950 run-list kernel stages its input; lets a
                          test state exactly what that kernel must compute
  max_rel_err / elementwise_err   the two error figures of the tests: max|dy| / max|y_ref| (the tolerance
                          metric) and max(|dy| / (|y_ref| + 0.1 rms(y_ref))) (every element judged on its own)

Pinning of the fp8 helpers: against torch.float8_e4m3fn conversion on every finite fp8 value, on midpoints and on
random inputs, and against the closed-form error bound of the decomposition (tests/test_oracle_layer.py).

Pinning (tests/test_oracle_*.py): pack/unpack against hand-derived known-answer words and the
committed fixtures in tests/golden/, a brute-force per-bit Python loop, the popcount and
round-trip invariants and the scalar restatement of the device decode; layer_forward against
the all-(+1) closed form, the rank-1 outer-product case, a pure-Python triple loop on tiny
shapes, the C restatement in nq_oracle.c, and float64 evaluation of dense_weight.

Bit convention (follows the code, not prose): packed bit 1 means -1, bit 0 means +1.
Naming: `vt` is the first-stage factor [r, n] (module attribute `V`), `u` the second-stage
factor [m, r] (module attribute `U`).
"""
from __future__ import annotations

import numpy as np

METHODS = ("lsb_first", "half2")


# --------------------------------------------------------------------------------------
# packing
# --------------------------------------------------------------------------------------
def bit_position(k: int, method: str) -> int:
    """Bit index inside the 32-bit word that holds element k (0..31) of a 32-group."""
    if not 0 <= k < 32:
        raise ValueError("k must be in [0, 32)")
    if method == "lsb_first":
        return k
    if method == "half2":
        # even elements fill bits 15..0 downwards, odd elements bits 31..16 downwards
        return 15 - (k >> 1) + 16 * (k & 1)
    raise ValueError(f"Unsupported method: '{method}'. Supported methods are 'lsb_first', 'half2'.")


def _positions(method: str) -> np.ndarray:
    return np.array([bit_position(k, method) for k in range(32)], dtype=np.uint64)


def pack_rows(signs: np.ndarray, method: str = "lsb_first") -> np.ndarray:
    """int8 {-1,+1} [rows, cols] -> int32 [rows, ceil(cols/32)].  Column padding is +1 (bit 0)."""
    signs = np.asarray(signs)
    if signs.dtype != np.int8:
        raise TypeError("Input tensor must be int8.")
    if signs.ndim != 2:
        raise ValueError("expected a 2-D matrix")
    rows, cols = signs.shape
    words = (cols + 31) // 32
    padded = np.ones((rows, words * 32), dtype=np.int8)
    padded[:, :cols] = signs
    bits = ((1 - padded.astype(np.int64)) // 2).astype(np.uint64).reshape(rows, words, 32)
    pos = _positions(method)
    packed = (bits << pos).sum(axis=2, dtype=np.uint64)
    return packed.astype(np.uint32).view(np.int32)


def unpack_rows(packed: np.ndarray, shape: tuple[int, int], method: str = "lsb_first") -> np.ndarray:
    """Inverse of pack_rows; trims the column padding."""
    packed = np.asarray(packed)
    if packed.ndim != 2:
        raise ValueError(f"Unsupported packed tensor format. Expected 2D tensor, got {packed.ndim} dimensions.")
    rows, cols = int(shape[0]), int(shape[1])
    words = (cols + 31) // 32
    if tuple(packed.shape) != (rows, words):
        raise ValueError(f"Unsupported packed tensor shape. Expected ({rows}, {words}), got {tuple(packed.shape)}.")
    pos = _positions(method)
    w = packed.astype(np.int32).view(np.uint32).astype(np.uint64)
    bits = (w[:, :, None] >> pos) & np.uint64(1)
    bits = bits.reshape(rows, words * 32)[:, :cols].astype(np.int8)
    return (1 - 2 * bits).astype(np.int8)


def repack(packed: np.ndarray, src: str, dst: str) -> np.ndarray:
    """Fixed per-word bit permutation between the two row-major orders."""
    w = np.asarray(packed).astype(np.int32).view(np.uint32).astype(np.uint64)
    out = np.zeros_like(w)
    for k in range(32):
        out |= ((w >> np.uint64(bit_position(k, src))) & np.uint64(1)) << np.uint64(bit_position(k, dst))
    return out.astype(np.uint32).view(np.int32)


def device_sign_flip_fp16(x8_bits: np.ndarray, word: int, quad: int) -> np.ndarray:
    """Scalar restatement of the device decode of the 'half2' order.

    x8_bits: 4 uint32, each holding two fp16 bit patterns (low half = even element).  They are
    the 8 consecutive elements 8*quad .. 8*quad+7 of a 32-group; `word` is that group's packed
    word.  Returns the 4 uint32 with sign bits flipped where the element's packed bit is 1.
    """
    mask = 0x80008000
    shifted = (int(word) & 0xFFFFFFFF) << (4 * quad)
    out = []
    for c in range(4):
        out.append((int(x8_bits[c]) ^ ((shifted << c) & mask)) & 0xFFFFFFFF)
    return np.array(out, dtype=np.uint32)


# --------------------------------------------------------------------------------------
# layer mathematics
# --------------------------------------------------------------------------------------
def layer_forward(x, vt, u, s_in, s_mid, s_out, dtype=np.float32) -> np.ndarray:
    """y = ((x * s_in) @ vt.T [* s_mid]) @ u.T * s_out, evaluated in `dtype` in that order.

    x [B, n]; vt [r, n] and u [m, r] dense +-1; s_in [n], s_mid [r] or None, s_out [m].
    """
    x = np.asarray(x, dtype=dtype)
    vt = np.asarray(vt, dtype=dtype)
    u = np.asarray(u, dtype=dtype)
    y = (x * np.asarray(s_in, dtype=dtype).reshape(1, -1)) @ vt.T
    if s_mid is not None:
        y = y * np.asarray(s_mid, dtype=dtype).reshape(1, -1)
    y = y @ u.T
    return y * np.asarray(s_out, dtype=dtype).reshape(1, -1)


def dense_weight(vt, u, s_in, s_mid, s_out, dtype=np.float64) -> np.ndarray:
    """W [m, n] = diag(s_out) . u . diag(s_mid) . vt . diag(s_in)."""
    vt = np.asarray(vt, dtype=dtype)
    u = np.asarray(u, dtype=dtype)
    mid = np.ones(vt.shape[0], dtype=dtype) if s_mid is None else np.asarray(s_mid, dtype=dtype)
    w = (u * mid.reshape(1, -1)) @ vt
    return np.asarray(s_out, dtype=dtype).reshape(-1, 1) * w * np.asarray(s_in, dtype=dtype).reshape(1, -1)


def layer_forward_packed(x, s_in, vt_bits, s_mid, u_bits, s_out, n=None, r=None, m=None,
                         method="half2", dtype=np.float32) -> np.ndarray:
    """Reference result for the kernel-side operands: unpack the words, then layer_forward."""
    vt_bits = np.asarray(vt_bits)
    u_bits = np.asarray(u_bits)
    r_rows = vt_bits.shape[0]
    n = int(np.asarray(x).shape[-1]) if n is None else n
    m = u_bits.shape[0] if m is None else m
    r = r_rows if r is None else r
    vt = unpack_rows(vt_bits, (r_rows, n), method)
    u = unpack_rows(u_bits, (m, u_bits.shape[1] * 32), method)[:, :r_rows]
    x2 = np.asarray(x, dtype=dtype).reshape(-1, n)
    return layer_forward(x2, vt, u, s_in, s_mid, s_out, dtype=dtype)


def mixture_forward(x, terms, dtype=np.float32) -> np.ndarray:
    """Sum of single-term layers.  terms: iterable of (vt, u, s_in, s_mid, s_out)."""
    acc = None
    for vt, u, s_in, s_mid, s_out in terms:
        y = layer_forward(x, vt, u, s_in, s_mid, s_out, dtype=dtype)
        acc = y if acc is None else acc + y
    return acc


def pad_rank(vt, u, s_mid, multiple: int):
    """Pad the rank axis to a multiple with +1 signs and a zero mid scale (exactly neutral)."""
    vt = np.asarray(vt)
    u = np.asarray(u)
    r = vt.shape[0]
    rp = (r + multiple - 1) // multiple * multiple
    if s_mid is None:
        s_mid = np.ones(r, dtype=np.float32)
    s_mid = np.asarray(s_mid)
    if rp == r:
        return vt, u, s_mid
    vt_p = np.concatenate([vt, np.ones((rp - r, vt.shape[1]), dtype=vt.dtype)], axis=0)
    u_p = np.concatenate([u, np.ones((u.shape[0], rp - r), dtype=u.dtype)], axis=1)
    mid_p = np.concatenate([s_mid, np.zeros(rp - r, dtype=s_mid.dtype)])
    return vt_p, u_p, mid_p


def nominal_rank(m: int, n: int, bpw: float = 1.0) -> int:
    """Rank at which r*(m+n) sign bits equal bpw bits per weight of the m x n matrix."""
    return int(round(bpw * m * n / (m + n)))


def checkpoint_rank(in_features: int, out_features: int, bits: float, num_scales: int = 2, min_rank: int = 32) -> int:
    """Rank rule of real checkpoints (accounts for the scale overhead, floors to a multiple of 32)."""
    a, b = in_features, out_features
    if a * b == 0:
        rank = None
    else:
        budget = a * b * bits
        s = a + b
        rank = (budget - 16 * s) / (s + 16) if num_scales == 3 else budget / s - 16
    cur = int(rank) if rank is not None else 0
    cur = (cur // 32) * 32
    if cur == 0:
        cur = min_rank
    cur = max(cur, min_rank)
    if cur <= 0:
        return max(min(a, b) // 32, 32)
    return min(cur, min(a, b))


def max_rel_err(y, y_ref) -> float:
    """max|y - y_ref| / max|y_ref| per output tensor (the tolerance metric)."""
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    denom = float(np.max(np.abs(y_ref)))
    if denom == 0.0:
        return float(np.max(np.abs(y)))
    return float(np.max(np.abs(y - y_ref)) / denom)


def elementwise_err(y, y_ref, floor_frac: float = 0.1) -> float:
    """max over elements of |y - y_ref| / (|y_ref| + floor), floor = floor_frac * rms(y_ref) per output tensor.
    The absolute floor keeps outputs that happen to lie near zero from deciding the figure; everything above the
    floor is judged relative to itself, which `max_rel_err` (one denominator for the whole tensor) does not do."""
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    floor = floor_frac * float(np.sqrt(np.mean(y_ref * y_ref)))
    if floor == 0.0:
        return float(np.max(np.abs(y)))
    return float(np.max(np.abs(y - y_ref) / (np.abs(y_ref) + floor)))


# --------------------------------------------------------------------------------------
# seeded synthetic operands (same recipe for tests, smoke and bench)
# --------------------------------------------------------------------------------------
def synth_term(m: int, n: int, r: int, seed: int, scale_dtype=np.float16):
    """i.i.d. fair-coin signs, scales |N(0,0.02)|+1e-3 in fp16; returns (vt, u, s_in, s_mid, s_out)."""
    rng = np.random.default_rng(seed)
    vt = (rng.integers(0, 2, size=(r, n), dtype=np.int8) * 2 - 1).astype(np.int8)
    u = (rng.integers(0, 2, size=(m, r), dtype=np.int8) * 2 - 1).astype(np.int8)

    def scale(k):
        return (np.abs(rng.normal(0.0, 0.02, size=k)) + 1e-3).astype(scale_dtype)

    return vt, u, scale(n), scale(r), scale(m)


def synth_x(batch: int, n: int, seed: int, dtype=np.float16):
    rng = np.random.default_rng(seed + 7919)
    return rng.normal(0.0, 1.0, size=(batch, n)).astype(dtype)


# --------------------------------------------------------------------------------------
# the reference's CPU path (dense +-1 factors through torch.nn.functional.linear)
# --------------------------------------------------------------------------------------
def torch_dense_forward(x, vt, u, s_in, s_mid, s_out):
    """Two F.linear calls on dense +-1 factors plus three scale multiplies; all torch tensors of
    one dtype on the CPU.  This is what bench.py times as the CPU baseline."""
    import torch.nn.functional as F

    y = F.linear(x * s_in, vt)
    if s_mid is not None:
        y = y * s_mid
    y = F.linear(y, u)
    return y * s_out


# ---- the input format of the gfx950 run-list kernel (batch <= 2) --------------------------------------
def fp8_e4m3_round(v) -> np.ndarray:
    """Round float64 values to the nearest OCP e4m3 number (ties to even, subnormals down to 2^-9, |v| <= 448
    expected).  Returned as float64."""
    v = np.asarray(v, dtype=np.float64)
    a = np.abs(v)
    e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.clip(e, -6, 8)                       # binade of the value; below 2^-6 the spacing stays 2^-9
    q = np.exp2(e - 3)                          # spacing: 3 mantissa bits
    r = np.round(a / q) * q                     # numpy rounds halves to even
    return np.sign(v) * np.minimum(r, 448.0)


def fp8_pieces(u, pieces: int = 3) -> np.ndarray:
    """[pieces, ...]: q_k = fp8(u - q_0 - ... - q_{k-1})."""
    u = np.asarray(u, dtype=np.float64)
    out = []
    rest = u.copy()
    for _ in range(pieces):
        q = fp8_e4m3_round(rest)
        out.append(q)
        rest = rest - q
    return np.stack(out)


def staged_input(v, pieces: int = 3, block: int = 128) -> np.ndarray:
    """What the run-list kernel multiplies the signs with, per row of v [batch, K]: every block of 128 consecutive
    columns (one 16-byte unit of packed signs) scaled by the power of two S that brings its max |v| into [128, 256),
    cut into fp8 pieces, summed and scaled back."""
    v = np.asarray(v, dtype=np.float64)
    out = np.zeros_like(v)
    for b in range(v.shape[0]):
        for c in range(0, v.shape[1], block):
            seg = v[b, c:c + block]
            mx = np.abs(seg).max()
            if mx == 0:
                continue
            s = np.exp2(7 - np.floor(np.log2(mx)))
            out[b, c:c + block] = fp8_pieces(seg * s, pieces).sum(axis=0) / s
    return out


# ---- tile order of the gfx950 run-list kernel ---------------------------------------------------------
def tile_words(packed: np.ndarray) -> np.ndarray:
    """Row-major words [rows, words] -> flat tile order, by the index formula itself (no counterpart in the
    reference): 16-byte unit (row, unit) goes to unit index
    ((((row // 32) * G + unit // 4) * 2 + (row // 16) % 2) * 4 + unit % 4) * 16 + row % 16, G = ceil(words / 16);
    padding rows / words are zero."""
    rows, words = packed.shape
    groups = (words + 15) // 16
    out = np.zeros(((rows + 31) // 32) * groups * 128 * 4, dtype=packed.dtype)
    for row in range(rows):
        for c in range(words):
            unit = c // 4
            idx = ((((row // 32) * groups + unit // 4) * 2 + (row // 16) % 2) * 4 + unit % 4) * 16 + row % 16
            out[idx * 4 + c % 4] = packed[row, c]
    return out

