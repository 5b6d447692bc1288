"""ctypes binding of the C restatement (oracle/nq_oracle.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libnq_oracle.so")


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.nqo_bit_position.restype = ctypes.c_int
        _lib.nqo_layer_forward_packed.restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def pack_rows(signs: np.ndarray, method: str) -> np.ndarray:
    signs = np.ascontiguousarray(signs, dtype=np.int8)
    rows, cols = signs.shape
    out = np.zeros((rows, (cols + 31) // 32), dtype=np.uint32)
    lib().nqo_pack_rows(_p(signs), ctypes.c_int64(rows), ctypes.c_int64(cols), int(method == "half2"), _p(out))
    return out.view(np.int32)


def unpack_rows(packed: np.ndarray, shape, method: str) -> np.ndarray:
    packed = np.ascontiguousarray(packed).view(np.uint32)
    rows, cols = shape
    out = np.zeros((rows, cols), dtype=np.int8)
    lib().nqo_unpack_rows(_p(packed), ctypes.c_int64(rows), ctypes.c_int64(cols), int(method == "half2"), _p(out))
    return out


def layer_forward_packed(x, s_in, vt_bits, s_mid, u_bits, s_out, method="half2") -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float64)
    B, n = x.shape
    vt_bits = np.ascontiguousarray(vt_bits).view(np.uint32)
    u_bits = np.ascontiguousarray(u_bits).view(np.uint32)
    r, m = vt_bits.shape[0], u_bits.shape[0]
    s_in = np.ascontiguousarray(s_in, dtype=np.float64)
    s_out = np.ascontiguousarray(s_out, dtype=np.float64)
    mid = None if s_mid is None else np.ascontiguousarray(s_mid, dtype=np.float64)
    y = np.zeros((B, m), dtype=np.float64)
    rc = lib().nqo_layer_forward_packed(_p(x), _p(s_in), _p(vt_bits), None if mid is None else _p(mid), _p(u_bits),
                                        _p(s_out), ctypes.c_int64(B), ctypes.c_int64(n), ctypes.c_int64(r),
                                        ctypes.c_int64(m), int(method == "half2"), _p(y))
    if rc != 0:
        raise MemoryError("nqo_layer_forward_packed failed")
    return y
