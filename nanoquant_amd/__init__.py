"""MI355X (gfx950) implementation of the binary low-rank linear layer.

Importing this package registers the `torch.ops.binary_kernels.*` operators.
"""
from . import ops  # noqa: F401  (registers torch.ops.binary_kernels)
from .linear import MixtureOfRankLinear, NanoQuantLinear, decode_group, prefill_group
from .packing import (binary_packer, binary_unpacker, marlin_nanoquant_packer, marlin_onebit_packer,
                      pack_binary_gemv, pack_binary_marlin, pack_binary_marlin_fused, repack_words,
                      unpack_binary_gemv)
from .ops import get_kernel_function
from .runlist import DecodeRunList

__all__ = [
    "NanoQuantLinear", "MixtureOfRankLinear", "binary_packer", "binary_unpacker", "marlin_nanoquant_packer",
    "marlin_onebit_packer", "pack_binary_gemv", "unpack_binary_gemv", "pack_binary_marlin",
    "pack_binary_marlin_fused", "repack_words", "get_kernel_function", "DecodeRunList", "prefill_group", "decode_group",
]
