"""ctypes binding of libnq_gfx950.so.  There is no fallback: if the library is missing, loading
raises, and every op of the package raises with it."""
from __future__ import annotations

import ctypes
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnq_gfx950.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "nq_gfx950.h")

NQ_F16, NQ_BF16 = 0, 1
ORDER_IDS = {"lsb_first": 0, "half2": 1}

NQ_ERR_DTYPE = -1
NQ_ERR_HIP = -100

_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
_SIGNATURES = {
    "nq_status_string": (ctypes.c_char_p, [_i]),
    "nq_last_hip_error": (_i, []),
    "nq_abi_version": (_i, []),
    "nq_device_query": (_i, [_i, ctypes.POINTER(_i)]),
    "nq_gemv_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "nq_gemv_forward_bias": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "nq_gemv_forward_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "nq_gemv_group_max": (_i, []),
    "nq_gemv_forward_group": (_i, [_vp, _i, _i, _i, _i, _vp]),
    "nq_gemv_group_status": (_i, [ctypes.POINTER(_i), _vp]),
    "nq_gemv_group_set_spin_limit": (_i, [ctypes.c_uint]),
    "nq_gemv_mixture": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "nq_runlist_workspace_bytes": (_sz, [_vp, _i]),
    "nq_runlist_build": (_i, [_vp, _i, _i, _i, _i, _vp, _sz, _vp, _vp]),
    "nq_runlist_run": (_i, [_vp, _vp, _vp]),
    "nq_runlist_run_bound": (_i, [_vp, _vp, _vp, _vp, _vp]),
    "nq_runlist_status": (_i, [_vp, ctypes.POINTER(_i), _vp]),
    "nq_runlist_set_deterministic": (_i, [_vp, _i]),
    "nq_runlist_capacity": (_i, [_i, _i, _i, _i]),
    "nq_gemv_stage": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "nq_gemm_scratch_bytes": (_sz, [_i, _i, _i]),
    "nq_gemm_onebit": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _vp]),
    "nq_gemm_nanoquant": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "nq_gemm_onebit_bias": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _vp]),
    "nq_gemm_nanoquant_bias": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "nq_repack_words": (_i, [_vp, _vp, _sz, _i, _i, _vp]),
    "nq_gemm_group_max": (_i, []),
    "nq_gemm_nanoquant_group": (_i, [_vp, _i, _i, _i, _vp, _sz, _vp]),
    "nq_gemm_panel_workspace_bytes": (_sz, []),
    "nq_gemm_nanoquant_group_ws": (_i, [_vp, _i, _i, _i, _vp, _sz, _vp, _sz, _i, _vp]),
    "nq_gemm_panel_status": (_i, [_vp, ctypes.POINTER(_i), _vp]),
    "nq_gemm_panel_set_spin_limit": (_i, [ctypes.c_uint]),
    "nq_pack_gemm_tiles": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "nq_tiled_words": (_sz, [_i, _i]),
    "nq_tile_words": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "nq_stream_copy": (_i, [_vp, _vp, _sz, _vp]),
}

_lib = None


def declared_symbols() -> list[str]:
    """Entry points declared in include/nq_gfx950.h (used by the load test)."""
    with open(HEADER_PATH) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nq_[a-z0-9_]+)\s*\(", text)))


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: the gfx950 kernels are not built. "
                "Run `python -c 'import __graft_entry__ as g; g.build()'` (or nanoquant_amd/build.py).")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def status_message(status: int) -> str:
    msg = lib().nq_status_string(status).decode()
    if status == NQ_ERR_HIP:
        msg += f" (hipError {lib().nq_last_hip_error()})"
    return msg


def check(status: int) -> None:
    """Map a C-ABI status to the exception type the reference's host wrappers raise (RuntimeError)."""
    if status != 0:
        raise RuntimeError(status_message(status))
