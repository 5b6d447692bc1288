"""Host-side packers for the binary factors (torch, any device).

Mirrors the packer interface of the reference (src/nanoquant/kernel/utils.py): the same function
names, argument meaning and error behaviour, so model code written against it keeps working.

Row-major formats (bit-exact with the reference; bit 1 encodes -1, column padding is +1):
  * ``lsb_first``: element k of a 32-group at bit k                      (utils.py:99)  checkpoints
  * ``half2``:     element k at bit 15 - (k >> 1) + 16 * (k & 1)         (utils.py:104) decode kernels

Prefill format (``pack_binary_marlin`` / ``pack_binary_marlin_fused``): the reference emits Marlin's
tensor-core fragment layout (utils.py:186-214), which is private to its packer/kernel pair.  The gfx950
prefill kernel has its own private layout instead, shaped for 64-lane MFMA operands ("tile32x256",
see ``pack_gemm_tiles``); tensor shapes, dtypes, padding rules and the returned tuple are the
reference's, so callers cannot tell the difference.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

MARLIN_MIN_MAX_PAR = 32  # workspace sizing rule kept from the reference (utils.py:21, :212)
GEMM_TILE_ROWS = 32
GEMM_TILE_K = 256
RANK_MULTIPLE_GEMM = 256  # utils.py:261


def _bit_positions(method: str, device) -> torch.Tensor:
    k = torch.arange(32, device=device)
    if method == "lsb_first":
        return k
    if method == "half2":
        return 15 - (k >> 1) + 16 * (k & 1)
    raise ValueError(f"Unsupported method: '{method}'. Supported methods are 'lsb_first', 'half2'.")


def _bits_to_words(bits_by_position: torch.Tensor) -> torch.Tensor:
    """uint8 {0,1} [..., 32] indexed by bit position -> int32 [...] (little-endian byte assembly)."""
    lead = bits_by_position.shape[:-1]
    b = bits_by_position.reshape(*lead, 4, 8)
    weights = torch.tensor([1, 2, 4, 8, 16, 32, 64, 128], dtype=torch.uint8, device=b.device)
    by = (b * weights).sum(dim=-1, dtype=torch.uint8)  # [..., 4] bytes, byte 0 = bits 0..7
    return by.contiguous().view(torch.int32).reshape(lead)


def _words_to_bits(words: torch.Tensor) -> torch.Tensor:
    """int32 [...] -> uint8 {0,1} [..., 32] indexed by bit position."""
    by = words.contiguous().view(torch.uint8).reshape(*words.shape, 4)
    shifts = torch.arange(8, dtype=torch.uint8, device=words.device)
    bits = (by.unsqueeze(-1) >> shifts) & 1
    return bits.reshape(*words.shape, 32)


def pack_binary_gemv(tensor: torch.Tensor, method: str = "lsb_first") -> torch.Tensor:
    """int8 {-1,+1} [rows, cols] -> int32 [rows, ceil(cols/32)]  (reference: utils.py:51-113)."""
    if tensor.dtype != torch.int8:
        raise TypeError("Input tensor must be int8.")
    n_rows, n_cols = tensor.shape
    pos = _bit_positions(method, tensor.device)
    words = (n_cols + 31) // 32
    neg = torch.zeros((n_rows, words * 32), dtype=torch.uint8, device=tensor.device)
    neg[:, :n_cols] = (tensor < 0).to(torch.uint8)
    neg = neg.view(n_rows, words, 32)
    by_position = torch.empty_like(neg)
    by_position[..., pos] = neg  # element k lands on its bit position
    return _bits_to_words(by_position).contiguous()


def unpack_binary_gemv(packed_tensor: torch.Tensor, original_shape: Tuple[int, int],
                       method: str = "lsb_first") -> torch.Tensor:
    """Inverse of pack_binary_gemv (reference: utils.py:116-183)."""
    if packed_tensor.dim() != 2:
        raise ValueError(
            f"Unsupported packed tensor format. Expected 2D tensor, got {packed_tensor.dim()} dimensions.")
    n_rows, n_cols = int(original_shape[0]), int(original_shape[1])
    words = (n_cols + 31) // 32
    if tuple(packed_tensor.shape) != (n_rows, words):
        raise ValueError(
            f"Unsupported packed tensor shape. Expected ({n_rows}, {words}), got {packed_tensor.shape}.")
    pos = _bit_positions(method, packed_tensor.device)
    bits = _words_to_bits(packed_tensor.to(torch.int32))[..., pos]  # element order
    bits = bits.reshape(n_rows, words * 32)[:, :n_cols].to(torch.int8)
    return (1 - 2 * bits).to(torch.int8)


def repack_words(packed: torch.Tensor, src: str = "lsb_first", dst: str = "half2") -> torch.Tensor:
    """Convert packed words between the two row-major orders without unpacking to a dense matrix.
    On a ROCm tensor this is one pass of the device kernel; on the CPU a bit gather in torch."""
    if packed.dtype != torch.int32:
        raise TypeError("packed words must be int32")
    if packed.is_cuda:
        from . import ops
        return ops.repack_words_device(packed, src, dst)
    src_pos = _bit_positions(src, packed.device)
    dst_pos = _bit_positions(dst, packed.device)
    bits = _words_to_bits(packed)[..., src_pos]
    by_position = torch.empty_like(bits)
    by_position[..., dst_pos] = bits
    return _bits_to_words(by_position).contiguous()


# ---------------------------------------------------------------------------------------------
# tile order of the decode run list
# ---------------------------------------------------------------------------------------------
def tile_words(packed: torch.Tensor) -> torch.Tensor:
    """Row-major words [rows, words] ("half2" order) -> flat int32 buffer in the tile order of the run-list kernel:
    16-byte units (4 words) indexed [row // 32][unit // 4][(row // 16) & 1][unit & 3][row & 15], rows padded to a
    multiple of 32 and units to a multiple of 4 with zero words.  The 64 units that a wavefront fetches for one MFMA
    operand (16 rows x 4 units) become 1 KiB contiguous.  The reference has no such layout (its kernels read the
    row-major words, kernel/utils.py:51-113); this is a fixed permutation done once at load time."""
    if packed.dtype != torch.int32 or packed.dim() != 2:
        raise TypeError("packed words must be a 2-D int32 tensor")
    rows, words = packed.shape
    if packed.is_cuda:
        from . import ops
        return ops.tile_words_device(packed.contiguous(), inverse=False)
    groups = (words + 15) // 16
    r32 = (rows + 31) // 32 * 32
    pad = torch.zeros((r32, groups * 16), dtype=torch.int32)
    pad[:rows, :words] = packed
    # [rp, half, r16, ub, g, word] -> [rp, ub, half, g, r16, word]
    t = pad.view(r32 // 32, 2, 16, groups, 4, 4).permute(0, 3, 1, 4, 2, 5)
    return t.contiguous().view(-1)


def untile_words(tiled: torch.Tensor, shape: Tuple[int, int]) -> torch.Tensor:
    """Inverse of tile_words for a matrix of `shape` = (rows, words)."""
    rows, words = int(shape[0]), int(shape[1])
    if tiled.dtype != torch.int32 or tiled.dim() != 1:
        raise TypeError("tiled words must be a flat int32 tensor")
    groups = (words + 15) // 16
    r32 = (rows + 31) // 32 * 32
    if tiled.numel() != r32 * groups * 16:
        raise ValueError(f"expected {r32 * groups * 16} words for shape {(rows, words)}, got {tiled.numel()}")
    if tiled.is_cuda:
        from . import ops
        return ops.tile_words_device(tiled.contiguous(), inverse=True, shape=(rows, words))
    t = tiled.view(r32 // 32, groups, 2, 4, 16, 4).permute(0, 2, 4, 1, 3, 5)
    return t.contiguous().view(r32, groups * 16)[:rows, :words].contiguous()


# ---------------------------------------------------------------------------------------------
# prefill (MFMA) layout
# ---------------------------------------------------------------------------------------------
def pack_gemm_tiles(weight: torch.Tensor) -> torch.Tensor:
    """int8 {-1,+1} [out, in] -> int32 flat tile buffer of out*in/32 words ("tile32x256").

    The matrix is cut into tiles of 32 output rows x 256 input columns, stored [out/32][in/256] with
    the in-tile index fastest; one tile is 1 KiB = 64 lanes x 16 bytes, so a wavefront fetches a tile
    with a single 128-bit load per lane.  Lane l owns output row 32*rt + (l & 31); its word q (0..3)
    holds the four MFMA k-steps t = 4q .. 4q+3, and within a word the 32 elements
    k = 256*kt + 16*t + 8*(l >> 5) + e (t' = t & 3, e = 0..7, in-word index 8*t' + e) sit in the
    "half2" bit order, so `(word << (4*t' + c)) & 0x80008000` is the sign mask of the 16-bit pair
    (e = 2c, 2c+1) -- exactly the 8 consecutive k values a lane feeds to v_mfma_f32_32x32x16.
    """
    if weight.dtype != torch.int8:
        raise TypeError("Input tensor must be int8.")
    out, k = weight.shape
    if out % GEMM_TILE_ROWS != 0 or k % GEMM_TILE_K != 0:
        raise ValueError(f"prefill packing needs out % {GEMM_TILE_ROWS} == 0 and in % {GEMM_TILE_K} == 0, "
                         f"got out={out}, in={k}")
    neg = (weight < 0).to(torch.uint8)
    # axes: rt, row(32), kt, q(4), t'(4), half(2) [= l >> 5], e(8)
    neg = neg.view(out // 32, 32, k // 256, 4, 4, 2, 8)
    # -> rt, kt, half, row, q, t', e : lane = 32*half + row, word q, in-word element 8*t' + e
    neg = neg.permute(0, 2, 5, 1, 3, 4, 6).reshape(-1, 32)
    pos = _bit_positions("half2", weight.device)
    by_position = torch.empty_like(neg)
    by_position[..., pos] = neg
    return _bits_to_words(by_position).contiguous()


def pack_gemm_tiles_from_words(words: torch.Tensor, rows_padded: int, k_padded: int, method: str = "lsb_first") -> torch.Tensor:
    """Row-major packed words [rows, ceil(cols/32)] (either word order) -> the "tile32x256" buffer of
    pack_gemm_tiles for the matrix padded with +1 signs to [rows_padded, k_padded], without a dense +-1 matrix
    on the device: one pass of `nq_pack_gemm_tiles` over the words (on CPU tensors a bit gather in torch).
    This is what lets a packed checkpoint (`lsb_first` words, modules/linear.py:288-321 of the reference) be
    served by the prefill kernels directly; the reference's loader unpacks to dense first
    (utils/load_utils.py:269-293)."""
    if words.dtype != torch.int32 or words.dim() != 2:
        raise TypeError("packed words must be a 2-D int32 tensor")
    rows, nwords = words.shape
    if rows_padded % GEMM_TILE_ROWS != 0 or k_padded % GEMM_TILE_K != 0 or rows_padded < rows or k_padded < 32 * nwords:
        raise ValueError(f"prefill packing needs rows_padded % {GEMM_TILE_ROWS} == 0, k_padded % {GEMM_TILE_K} == 0 and "
                         f"both at least the source's size, got {rows_padded} x {k_padded} for {rows} x {32 * nwords}")
    pos = _bit_positions(method, words.device)      # also validates the method name
    if words.is_cuda:
        from . import ops
        return ops.pack_gemm_tiles_device(words.contiguous(), rows_padded, k_padded, method)
    neg = torch.zeros((rows_padded, k_padded), dtype=torch.uint8)
    neg[:rows, :32 * nwords] = _words_to_bits(words)[..., pos].reshape(rows, 32 * nwords)
    neg = neg.view(rows_padded // 32, 32, k_padded // 256, 4, 4, 2, 8).permute(0, 2, 5, 1, 3, 4, 6).reshape(-1, 32)
    by_position = torch.empty_like(neg)
    by_position[..., _bit_positions("half2", words.device)] = neg
    return _bits_to_words(by_position).contiguous()


def unpack_gemm_tiles(packed: torch.Tensor, out: int, k: int) -> torch.Tensor:
    """Inverse of pack_gemm_tiles -> int8 {-1,+1} [out, k]."""
    pos = _bit_positions("half2", packed.device)
    bits = _words_to_bits(packed.reshape(-1).to(torch.int32))[..., pos]
    bits = bits.view(out // 32, k // 256, 2, 32, 4, 4, 8).permute(0, 3, 1, 4, 5, 2, 6).reshape(out, k)
    return (1 - 2 * bits.to(torch.int8)).to(torch.int8)


def pack_binary_marlin(weight: torch.Tensor, scale_in: Optional[torch.Tensor], scale_out: Optional[torch.Tensor]):
    """weight int8 {-1,+1} [out, in] -> (bits int32 [in/16, out/2], scale_in, scale_out, workspace_size).

    Interface of the reference's single-matrix prefill packer (utils.py:186-214).  The bit layout inside
    the returned tensor is the gfx950 tile layout; the scale vectors stay in natural order (the
    reference permutes them for its fragment layout)."""
    out, k = weight.shape
    bits = pack_gemm_tiles(weight.to(torch.int8)).view(k // 16, out // 2)
    workspace_size = out // 128 * MARLIN_MIN_MAX_PAR
    s_in = None if scale_in is None else scale_in.reshape(-1).contiguous()
    s_out = None if scale_out is None else scale_out.reshape(-1).contiguous()
    return bits, s_in, s_out, workspace_size


def pack_binary_marlin_fused(V_sign: torch.Tensor, U_sign: torch.Tensor, scale_g: torch.Tensor,
                             scale_l: Optional[torch.Tensor], scale_h: torch.Tensor):
    """Two-stage prefill packing (reference: utils.py:217-284).

    V_sign int8 [N, R], U_sign int8 [R, M]; scale_g [N], scale_l [R] or None, scale_h [M].  The rank is
    padded to a multiple of 256 with +1 signs and a zero mid scale, which makes the padding exactly
    neutral.  Returns (V_bits, U_bits, scale_g, scale_l_padded, scale_h, workspace)."""
    dev = V_sign.device
    r = U_sign.shape[0]
    if scale_l is None:
        scale_l = torch.ones(r, device=dev, dtype=scale_g.dtype)
    rank_p = (r + RANK_MULTIPLE_GEMM - 1) // RANK_MULTIPLE_GEMM * RANK_MULTIPLE_GEMM
    if rank_p > r:
        pad = rank_p - r
        V_sign = torch.cat([V_sign, torch.ones(V_sign.shape[0], pad, device=dev, dtype=torch.int8)], dim=1)
        U_sign = torch.cat([U_sign, torch.ones(pad, U_sign.shape[1], device=dev, dtype=torch.int8)], dim=0)
        scale_l = torch.cat([scale_l, torch.zeros(pad, device=dev, dtype=scale_l.dtype)], dim=0)
    V_bits, s_g, s_l, ws_v = pack_binary_marlin(V_sign.T.contiguous(), scale_g, scale_l)
    U_bits, _, s_h, ws_u = pack_binary_marlin(U_sign.T.contiguous(), scale_l, scale_h)
    workspace = torch.zeros(max(ws_v, ws_u), device=dev, dtype=torch.int32)
    return V_bits.contiguous(), U_bits.contiguous(), s_g, s_l, s_h, workspace


def pack_binary_marlin_fused_from_words(V_words: torch.Tensor, U_words: torch.Tensor, rank: int, scale_g: torch.Tensor,
                                        scale_l: Optional[torch.Tensor], scale_h: torch.Tensor, method: str = "lsb_first"):
    """pack_binary_marlin_fused for factors that are already packed row-major words, as a checkpoint holds them
    (modules/linear.py:288-321): V_words [rank, in/32] (module V, the first stage), U_words [out, ceil(rank/32)]
    (module U, the second stage).  Same 6-tuple, same rank padding (+1 signs, zero mid scale), bit-identical to
    packing the unpacked factors -- but the dense +-1 matrices are never formed."""
    dev = V_words.device
    n, m = 32 * V_words.shape[1], U_words.shape[0]
    if V_words.shape[0] != rank or U_words.shape[1] != (rank + 31) // 32:
        raise ValueError("packed factor shapes do not match the rank")
    if scale_l is None:
        scale_l = torch.ones(rank, device=dev, dtype=scale_g.dtype)
    rank_p = (rank + RANK_MULTIPLE_GEMM - 1) // RANK_MULTIPLE_GEMM * RANK_MULTIPLE_GEMM
    if rank_p > rank:
        scale_l = torch.cat([scale_l, torch.zeros(rank_p - rank, device=dev, dtype=scale_l.dtype)], dim=0)
    V_bits = pack_gemm_tiles_from_words(V_words, rank_p, n, method).view(n // 16, rank_p // 2)
    U_bits = pack_gemm_tiles_from_words(U_words, m, rank_p, method).view(rank_p // 16, m // 2)
    workspace = torch.zeros(max(rank_p, m) // 128 * MARLIN_MIN_MAX_PAR, device=dev, dtype=torch.int32)
    return (V_bits.contiguous(), U_bits.contiguous(), scale_g.reshape(-1).contiguous(), scale_l.reshape(-1).contiguous(),
            scale_h.reshape(-1).contiguous(), workspace)


# aliases used by the reference's callers (utils.py:503-507)
binary_packer = pack_binary_gemv
binary_unpacker = unpack_binary_gemv
marlin_onebit_packer = pack_binary_marlin
marlin_nanoquant_packer = pack_binary_marlin_fused
