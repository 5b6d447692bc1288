"""`torch.ops.binary_kernels.*`: the operator boundary of the reference, served by libnq_gfx950.so.

Schemas are the reference's, character for character (src/nanoquant/kernel/pybind.cpp:83-105).  The
device implementations are registered under the CUDA dispatch key (ROCm tensors dispatch there) and
shape-only implementations under Meta, as the reference does (pybind.cpp:108-124), so the ops trace
under torch.compile(fullgraph=True).  There is no CPU registration and no fallback: without the
built library, or on CPU tensors, the ops raise.

Argument checks and their messages follow the reference's host wrappers:
  nanoquant_dyn_forward     src/nanoquant/kernel/cuda/gemv_kernel.cu:308-346, cuda/meta_utils.h:14-38
  marlin_onebit_forward     src/nanoquant/kernel/cuda/gemm.cpp:36-98
  marlin_nanoquant_forward  src/nanoquant/kernel/cuda/gemm.cpp:112-122
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib

_NS = "binary_kernels"

_SCHEMAS = (
    "nanoquant_dyn_forward("
    "Tensor x, Tensor scale_g, Tensor Ubits, Tensor? scale_l, Tensor Vbits, Tensor scale_h, "
    "int num_thread_stage1=128, int num_thread_stage2=128, int num_row_per_warp_stage1=2, "
    "int num_row_per_warp_stage2=2, int num_acc_stage1=4, int num_acc_stage2=4, "
    "int num_pipeline_stage1=2, int num_pipeline_stage2=2) -> Tensor",
    "marlin_onebit_forward("
    "Tensor x, "
    "Tensor weight, "
    "Tensor? scale_g, Tensor? scale_h, "
    "Tensor(a!) workspace) -> Tensor",
    "marlin_nanoquant_forward("
    "Tensor x, "
    "Tensor weight_u, Tensor weight_v, "
    "Tensor? scale_g, Tensor? scale_l, Tensor? scale_h, "
    "Tensor(a!) workspace) -> Tensor",
)

MARLIN_MIN_MAX_PAR = 32

# Legal values of the CUDA tuning hints (gemv_kernel.cu:351-354).  They select template instances in
# the reference; here they are validated and otherwise ignored -- the gfx950 launch shape is derived
# from the problem.  4 is added to the accumulator set because it is the schema's own default.
_SWEEPS = {
    "n_th": (64, 128, 256),
    "n_rpw": (1, 2, 4, 8),
    "n_acc": (1, 2, 4),
    "n_pipe": (1, 2, 4, 8, 16),
}


def _dtype_id(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return _lib.NQ_F16
    if t.dtype == torch.bfloat16:
        return _lib.NQ_BF16
    raise RuntimeError("Support only Half or BFloat16")


def _check_dev_cont(t: torch.Tensor, name: str, dtype: torch.dtype, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} {what}")


_FLOAT_WHAT = {torch.float16: "must be float16 tensor", torch.bfloat16: "must be bfloat16 tensor"}


def _sweep(name: str, value: int) -> None:
    legal = _SWEEPS[name.rstrip("12")]
    if value not in legal:
        choices = ", ".join(str(v) for v in legal)
        raise ValueError(f"{name} should be one of [{choices}], but {value} was given")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev: torch.device):
    """The current stream of `dev` as the C ABI takes it.  The raw-handle query costs a tenth of building a
    `torch.cuda.Stream` object, which counts on a decode call that the GPU finishes in microseconds."""
    if _raw_stream is not None and dev.index is not None:
        return ctypes.c_void_p(_raw_stream(dev.index))
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


class _on_device:
    """`torch.cuda.device(dev)` that does nothing when `dev` is already the current device (the usual case)."""
    __slots__ = ("ctx",)

    def __init__(self, dev: torch.device):
        self.ctx = None if (dev.index is None or dev.index == torch.cuda.current_device()) else torch.cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


# ---------------------------------------------------------------------------------------------
# decode op
# ---------------------------------------------------------------------------------------------
def _check_gemv_args(x, scale_g, Ubits, scale_l, Vbits, scale_h):
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("Support only Half or BFloat16")
    what = _FLOAT_WHAT[x.dtype]
    _check_dev_cont(x, "x", x.dtype, what)
    _check_dev_cont(scale_g, "scale_g", x.dtype, what)
    _check_dev_cont(scale_h, "scale_h", x.dtype, what)
    _check_dev_cont(Ubits, "Ubits", torch.int32, "tensor dtype must be int32")
    _check_dev_cont(Vbits, "Vbits", torch.int32, "tensor dtype must be int32")
    if scale_l is not None:
        _check_dev_cont(scale_l, "(*scale_l)", x.dtype, what)
        if scale_l.size(0) != Ubits.size(0):
            raise RuntimeError("scale_l size mismatch")
    if x.dim() < 1:
        raise RuntimeError("x must have at least one dimension")
    n = x.size(-1)
    r = Ubits.size(0)
    m = scale_h.size(0)
    # The reference trusts these and indexes out of bounds otherwise; the launch needs them to hold.
    if Ubits.dim() != 2 or Vbits.dim() != 2:
        raise RuntimeError("Ubits and Vbits must be 2-D packed word matrices")
    if Ubits.size(1) != (n + 31) // 32:
        raise RuntimeError(f"Ubits has {Ubits.size(1)} words per row, expected {(n + 31) // 32} for {n} input columns")
    if scale_g.numel() != n:
        raise RuntimeError("scale_g size mismatch")
    if Vbits.size(0) != m or Vbits.size(1) != (r + 31) // 32:
        raise RuntimeError(f"Vbits must be [{m}, {(r + 31) // 32}], got {list(Vbits.shape)}")
    return n, r, m


def _check_bias(bias, m, x):
    if bias is None:
        return
    _check_dev_cont(bias, "bias", x.dtype, "Bias")
    if bias.dim() != 1 or bias.size(0) != m:
        raise RuntimeError(f"bias must be [{m}], got {list(bias.shape)}")


def _gemv_forward(x, scale_g, Ubits, scale_l, Vbits, scale_h, bias=None, dims=None):
    n, r, m = dims if dims is not None else _check_gemv_args(x, scale_g, Ubits, scale_l, Vbits, scale_h)
    _check_bias(bias, m, x)
    lead = x.shape[:-1]
    batch = 1
    for d in lead:
        batch *= d
    y = torch.empty((batch, m), dtype=x.dtype, device=x.device)
    if batch > 0 and m > 0:
        h = torch.empty((batch, max(r, 1)), dtype=torch.float32, device=x.device)
        with _on_device(x.device):
            _lib.check(_lib.lib().nq_gemv_forward_bias(_ptr(x), _ptr(scale_g), _ptr(Ubits), _ptr(scale_l), _ptr(Vbits),
                                                       _ptr(scale_h), _ptr(bias), _ptr(h), _ptr(y), batch, n, r, m,
                                                       _dtype_id(x), _stream(x.device)))
    return y.reshape(*lead, m)


def nanoquant_dyn_forward(x, scale_g, Ubits, scale_l, Vbits, scale_h,
                          num_thread_stage1=128, num_thread_stage2=128,
                          num_row_per_warp_stage1=2, num_row_per_warp_stage2=2,
                          num_acc_stage1=4, num_acc_stage2=4,
                          num_pipeline_stage1=2, num_pipeline_stage2=2):
    """y = scale_h * (Vbits (scale_l * (Ubits (scale_g * x)))): `Ubits` [r, n/32] is the FIRST stage,
    `Vbits` [m, r/32] the second (the reference's argument names, pybind.cpp:86-90)."""
    dims = _check_gemv_args(x, scale_g, Ubits, scale_l, Vbits, scale_h)
    _sweep("n_th1", num_thread_stage1)
    _sweep("n_rpw1", num_row_per_warp_stage1)
    _sweep("n_acc1", num_acc_stage1)
    _sweep("n_pipe1", num_pipeline_stage1)
    _sweep("n_th2", num_thread_stage2)
    _sweep("n_rpw2", num_row_per_warp_stage2)
    _sweep("n_acc2", num_acc_stage2)
    _sweep("n_pipe2", num_pipeline_stage2)
    return _gemv_forward(x, scale_g, Ubits, scale_l, Vbits, scale_h, dims=dims)


def _nanoquant_dyn_forward_meta(x, scale_g, Ubits, scale_l, Vbits, scale_h, *hints, **kw):
    shape = list(x.shape)
    shape[-1] = scale_h.size(0)
    return x.new_empty(shape)


# ---------------------------------------------------------------------------------------------
# prefill ops
# ---------------------------------------------------------------------------------------------
def _onebit_check(A, B, s_in, s_out, workspace):
    """marlin_onebit_check_and_alloc (gemm.cpp:36-56): returns (m, n, k)."""
    prob_m = A.size(0)
    prob_n = B.size(1) * 2
    prob_k = A.size(1)
    if prob_k != B.size(0) * 16:
        raise RuntimeError("k dimension mismatch")
    if s_in is not None and s_in.size(0) != prob_k:
        raise RuntimeError("s_in size mismatch")
    if s_out is not None and s_out.size(0) != prob_n:
        raise RuntimeError("s_out size mismatch")
    if workspace.numel() < prob_n // 128 * MARLIN_MIN_MAX_PAR:
        raise RuntimeError("workspace too small")
    return prob_m, prob_n, prob_k


def _gemm_dtype(A):
    if A.dtype == torch.float16:
        return _lib.NQ_F16
    if A.dtype == torch.bfloat16:
        return _lib.NQ_BF16
    raise RuntimeError("Unsupported dtype: Marlin only supports Half and BFloat16")


def _check_gemm_tensor(t, name, dtype=None):
    if t is None:
        return
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}")


# Split-k scratch (fp32 partial sums + tile counters).  The kernels require it to be zero on entry and
# leave it zero on exit, so one buffer per (device, stream) is allocated zeroed once, grown on demand and
# reused; no per-call memset.
_scratch_cache = {}


def _scratch(nbytes, device):
    if nbytes == 0:
        return None
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _scratch_cache.get(key)
    if buf is None or buf.numel() * 4 < nbytes:
        buf = torch.zeros((nbytes + 3) // 4, dtype=torch.float32, device=device)
        _scratch_cache[key] = buf
    return buf


# Workspace of the panel launches (partial tiles, hand-over flags, the count of finished workgroups): zero when
# first used, then owned by the launches; one per (device, stream) so that launches sharing it are stream-ordered.
_panel_ws_cache = {}
PANEL_MODES = {"auto": 0, "always": 1, "never": 2}


def _panel_workspace(device):
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _panel_ws_cache.get(key)
    if buf is None:
        with torch.cuda.device(device):
            nbytes = int(_lib.lib().nq_gemm_panel_workspace_bytes())
        if nbytes == 0:
            raise RuntimeError("nq_gemm_panel_workspace_bytes() returned 0: no usable device")
        buf = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        _panel_ws_cache[key] = buf
    return buf


def panel_status(device=None) -> int:
    """Status word of the current stream's panel workspace (synchronises; reads and clears): 0 ok, 1 = a bounded
    wait of a panel launch expired since the last call and that launch's outputs are invalid."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _panel_ws_cache.get(key)
    if buf is None:
        return 0
    out = ctypes.c_int(0)
    with torch.cuda.device(device):
        _lib.check(_lib.lib().nq_gemm_panel_status(_ptr(buf), ctypes.byref(out), _stream(device)))
    return int(out.value)


def marlin_onebit_forward(x, weight, scale_g, scale_h, workspace):
    """C[m, n] = s_out[n] * sum_k (x[m, k] * s_in[k]) * sgn(weight)[n, k]; weight from marlin_onebit_packer."""
    dt = _gemm_dtype(x)
    m, n, k = _onebit_check(x, weight, scale_g, scale_h, workspace)
    _check_gemm_tensor(x, "x")
    _check_gemm_tensor(weight, "weight", torch.int32)
    _check_gemm_tensor(scale_g, "scale_g", x.dtype)
    _check_gemm_tensor(scale_h, "scale_h", x.dtype)
    C = torch.empty((m, n), dtype=x.dtype, device=x.device)
    if m == 0 or n == 0:
        return C
    nbytes = int(_lib.lib().nq_gemm_scratch_bytes(m, k, n))
    scratch = _scratch(nbytes, x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().nq_gemm_onebit(_ptr(x), _ptr(weight), _ptr(scale_g), _ptr(scale_h), _ptr(C),
                                             _ptr(scratch), nbytes, m, k, n, dt, _stream(x.device)))
    return C


def _marlin_onebit_meta(x, weight, scale_g, scale_h, workspace):
    m, n, _ = _onebit_check(x, weight, scale_g, scale_h, workspace)
    return x.new_empty((m, n))


def _gemm_nanoquant_forward(x, weight_u, weight_v, scale_g, scale_l, scale_h, workspace, bias=None):
    dt = _gemm_dtype(x)
    t, r, n = _onebit_check(x, weight_u, scale_g, scale_l, workspace)
    _check_gemm_tensor(x, "x")
    _check_gemm_tensor(weight_u, "weight_u", torch.int32)
    _check_gemm_tensor(weight_v, "weight_v", torch.int32)
    for name, s in (("scale_g", scale_g), ("scale_l", scale_l), ("scale_h", scale_h)):
        _check_gemm_tensor(s, name, x.dtype)
    imm = torch.empty((t, r), dtype=x.dtype, device=x.device)
    _, m, _ = _onebit_check(imm, weight_v, None, scale_h, workspace)
    _check_bias(bias, m, x)
    out = torch.empty((t, m), dtype=x.dtype, device=x.device)
    if t == 0 or m == 0:
        return out
    nbytes = max(int(_lib.lib().nq_gemm_scratch_bytes(t, n, r)), int(_lib.lib().nq_gemm_scratch_bytes(t, r, m)))
    scratch = _scratch(nbytes, x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().nq_gemm_nanoquant_bias(_ptr(x), _ptr(weight_u), _ptr(weight_v), _ptr(scale_g), _ptr(scale_l),
                                                     _ptr(scale_h), _ptr(bias), _ptr(imm), _ptr(out), _ptr(scratch), nbytes,
                                                     t, n, r, m, dt, _stream(x.device)))
    return out


def marlin_nanoquant_forward(x, weight_u, weight_v, scale_g, scale_l, scale_h, workspace):
    """Two chained one-bit GEMMs (gemm.cpp:112-122): `weight_u` is the FIRST stage [n -> r],
    `weight_v` the second [r -> m] (the order marlin_nanoquant_packer returns them)."""
    return _gemm_nanoquant_forward(x, weight_u, weight_v, scale_g, scale_l, scale_h, workspace)


def _marlin_nanoquant_meta(x, weight_u, weight_v, scale_g, scale_l, scale_h, workspace):
    t, r, _ = _onebit_check(x, weight_u, scale_g, scale_l, workspace)
    imm = x.new_empty((t, r))
    _, m, _ = _onebit_check(imm, weight_v, None, scale_h, workspace)
    return x.new_empty((t, m))


# ---------------------------------------------------------------------------------------------
# extras above the reference's surface (plain functions, not dispatcher ops)
# ---------------------------------------------------------------------------------------------
def gemv_forward_with_bias(x, scale_g, Ubits, scale_l, Vbits, scale_h, bias):
    """nanoquant_dyn_forward + bias [m], added in the epilogue of the second stage.  The reference's kernel paths
    return before the module's bias is added (modules/linear.py:121-141); this keeps it."""
    return _gemv_forward(x, scale_g, Ubits, scale_l, Vbits, scale_h, bias)


def gemv_group_forward(xs, linears, biases=None, outs=None, one_launch=False):
    """`[nanoquant_dyn_forward(x_i, *linears[i]) (+ biases[i])]` for independent linears in two launches per
    `nq_gemv_group_max()` linears and piece of 1, 2 or 4 rows (`nq_gemv_forward_group`: all first stages, then all
    second stages): the q/k/v or gate/up projections of a decoder layer at decode time, which the reference launches
    one module and two kernels at a time (modules/linear.py:121-130).  `xs`: one tensor [rows, n] for all linears or
    one per linear (same row count); `linears`: (scale_g, Ubits, scale_l, Vbits, scale_h) per linear, the operands of
    the op in its order; `outs`: optional result tensors [rows, m_i] to write into; `one_launch`: a single launch per
    group whose second stages wait inside the kernel (slower on MI355X, see include/nq_gfx950.h)."""
    linears = list(linears)
    if not linears:
        return []
    xs = [xs] * len(linears) if isinstance(xs, torch.Tensor) else list(xs)
    if len(xs) != len(linears):
        raise ValueError("one input per linear")
    biases = [None] * len(linears) if biases is None else list(biases)
    from .runlist import NqLinear
    x0 = xs[0]
    batch = x0.numel() // max(x0.size(-1), 1) if x0.dim() >= 1 else 0
    dims, offsets, total = [], [], 0
    for x, lin, b in zip(xs, linears, biases):
        n, r, m = _check_gemv_args(x, *lin)
        _check_bias(b, m, x)
        if x.dtype != x0.dtype or x.device != x0.device:
            raise RuntimeError("all inputs of a group must share dtype and device")
        if x.numel() // max(n, 1) != batch:
            raise RuntimeError("all inputs of a group must have the same number of rows")
        dims.append((n, r, m))
        offsets.append(total)
        total += (batch * max(r, 1) + 63) // 64 * 64              # fp32: every h starts on a 256-byte boundary
    if outs is None:
        outs = [torch.empty((batch, m), dtype=x0.dtype, device=x0.device) for _, _, m in dims]
    else:
        outs = list(outs)
        for y, (_, _, m) in zip(outs, dims):
            _check_dev_cont(y, "out", x0.dtype, _FLOAT_WHAT[x0.dtype])
            if tuple(y.shape) != (batch, m):
                raise RuntimeError(f"out must be [{batch}, {m}], got {list(y.shape)}")
    if batch == 0:
        return outs
    h = torch.empty(total, dtype=torch.float32, device=x0.device)
    arr = (NqLinear * len(linears))()
    p = lambda t: None if t is None else t.data_ptr()
    for i, (x, (sg, ub, sl, vb, sh), b, y, (n, r, m)) in enumerate(zip(xs, linears, biases, outs, dims)):
        arr[i] = NqLinear(p(x), p(sg), p(ub), p(sl), p(vb), p(sh), h.data_ptr() + 4 * offsets[i], p(y), None, n, r, m, -1, -1, 0,
                          p(b), 0)
    with _on_device(x0.device):
        _lib.check(_lib.lib().nq_gemv_forward_group(arr, len(linears), batch, _dtype_id(x0), 1 if one_launch else 0,
                                                     _stream(x0.device)))
    return outs


class GemvGroup:
    """A group of independent decode linears checked once, for callers that launch it again and again from Python
    (`gemv_group_forward` checks every operand on every call, which costs more host time than the launches take on
    the GPU).  `linears` and `biases` as `gemv_group_forward` takes them; the tensors are kept alive and must not be
    resized.  `group(xs, outs=None, one_launch=False)` checks the inputs only."""

    def __init__(self, linears, biases=None):
        from .runlist import NqLinear
        self.linears = [tuple(lin) for lin in linears]
        if not self.linears:
            raise ValueError("at least one linear")
        self.biases = [None] * len(self.linears) if biases is None else list(biases)
        if len(self.biases) != len(self.linears):
            raise ValueError("one bias entry per linear")
        sg0 = self.linears[0][0]
        self.dtype, self.device = sg0.dtype, sg0.device
        self.dims = []
        for (sg, ub, sl, vb, sh), b in zip(self.linears, self.biases):
            n = sg.numel()
            probe = torch.empty((0, n), dtype=self.dtype, device=self.device)     # the operand checks of the op, without an input yet
            self.dims.append(_check_gemv_args(probe, sg, ub, sl, vb, sh))
            _check_bias(b, self.dims[-1][2], probe)
        self._arr = (NqLinear * len(self.linears))()
        p = lambda t: None if t is None else t.data_ptr()
        for i, ((sg, ub, sl, vb, sh), b, (n, r, m)) in enumerate(zip(self.linears, self.biases, self.dims)):
            self._arr[i] = NqLinear(None, p(sg), p(ub), p(sl), p(vb), p(sh), None, None, None, n, r, m, -1, -1, 0, p(b), 0)
        self._dtype_id = _dtype_id(sg0)

    def __call__(self, xs, outs=None, one_launch=False):
        count = len(self.linears)
        xs = [xs] * count if isinstance(xs, torch.Tensor) else list(xs)
        if len(xs) != count:
            raise ValueError("one input per linear")
        x0 = xs[0]
        batch = x0.numel() // self.dims[0][0] if x0.dim() >= 1 and self.dims[0][0] else 0
        total, offsets = 0, []
        for x, (n, r, m) in zip(xs, self.dims):
            if not x.is_cuda or x.dtype != self.dtype or x.device != self.device or not x.is_contiguous():
                raise RuntimeError("inputs of a group must be contiguous tensors of the group's dtype on its device")
            if x.dim() < 1 or x.size(-1) != n or x.numel() != batch * n:
                raise RuntimeError(f"input must be [{batch}, {n}], got {list(x.shape)}")
            offsets.append(total)
            total += (batch * max(r, 1) + 63) // 64 * 64
        if outs is None:
            outs = [torch.empty((batch, m), dtype=self.dtype, device=self.device) for _, _, m in self.dims]
        else:
            outs = list(outs)
            for y, (_, _, m) in zip(outs, self.dims):
                _check_dev_cont(y, "out", self.dtype, _FLOAT_WHAT[self.dtype])
                if tuple(y.shape) != (batch, m):
                    raise RuntimeError(f"out must be [{batch}, {m}], got {list(y.shape)}")
        if batch == 0:
            return outs
        h = torch.empty(total, dtype=torch.float32, device=self.device)
        hp, arr = h.data_ptr(), self._arr
        for i in range(count):
            arr[i].x, arr[i].h, arr[i].y = xs[i].data_ptr(), hp + 4 * offsets[i], outs[i].data_ptr()
        with _on_device(self.device):
            _lib.check(_lib.lib().nq_gemv_forward_group(arr, count, batch, self._dtype_id, 1 if one_launch else 0,
                                                         _stream(self.device)))
        return outs


def gemv_group_status(device=None) -> int:
    """Synchronises the current stream.  0, or 1 when a launch of `gemv_group_forward(one_launch=True)` on this device
    ran into its bounded wait since the last call: the outputs of that launch are invalid.  Clears the flag."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    out = ctypes.c_int(0)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().nq_gemv_group_status(ctypes.byref(out), _stream(dev)))
    return out.value


def gemm_forward_with_bias(x, weight_u, weight_v, scale_g, scale_l, scale_h, workspace, bias):
    """marlin_nanoquant_forward + bias [m], added in the epilogue of the second GEMM."""
    return _gemm_nanoquant_forward(x, weight_u, weight_v, scale_g, scale_l, scale_h, workspace, bias)


class NqGemmTerm(ctypes.Structure):
    """Mirror of `nq_gemm_term` in include/nq_gfx950.h."""
    _fields_ = [("x", ctypes.c_void_p), ("vt_tiles", ctypes.c_void_p), ("u_tiles", ctypes.c_void_p),
                ("s_in", ctypes.c_void_p), ("s_mid", ctypes.c_void_p), ("s_out", ctypes.c_void_p),
                ("bias", ctypes.c_void_p), ("h", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("n", ctypes.c_int), ("r", ctypes.c_int), ("m", ctypes.c_int)]


def gemm_group_forward(xs, terms, biases=None, outs=None, panel="auto"):
    """Several `marlin_nanoquant_forward` calls on the same number of tokens in two launches instead of two per
    call: `terms` is a list of argument tuples (weight_u, weight_v, scale_g, scale_l, scale_h, workspace) as that
    op takes them after x; `xs` is one tensor [tokens, n] read by every term or a list of one tensor per term;
    `biases` an optional list of [m] tensors / None; `outs` an optional list of contiguous [tokens, m] tensors of
    the activation type to write into (allocated here when absent); `panel` ("auto", "always", "never") says whether
    the stages may run as persistent panel launches (around 128 tokens, see include/nq_gfx950.h).  Returns the list of
    outputs.  The terms share
    launches (a single linear leaves most of the device idle up to some hundred tokens): few-token tiles up to 160
    tokens, 64-token block tiles without k-split above.  The
    reference launches every linear by itself (modules/linear.py:131-133)."""
    lib = _lib.lib()
    count = len(terms)
    if count == 0:
        return []
    if isinstance(xs, torch.Tensor):
        xs = [xs] * count
    if len(xs) != count or (biases is not None and len(biases) != count) or (outs is not None and len(outs) != count):
        raise RuntimeError("one x (and one bias / output entry) per term")
    dt = _gemm_dtype(xs[0])
    given, outs, keep, arr_items, nbytes = outs, [], [], [], 0
    for i, (x, term) in enumerate(zip(xs, terms)):
        weight_u, weight_v, scale_g, scale_l, scale_h, workspace = term
        bias = None if biases is None else biases[i]
        if x.dtype != xs[0].dtype or x.dim() != 2 or x.size(0) != xs[0].size(0) or x.device != xs[0].device:
            raise RuntimeError("all inputs of a group must be 2-D with the same token count, dtype and device")
        t, r, n = _onebit_check(x, weight_u, scale_g, scale_l, workspace)
        _check_gemm_tensor(x, "x")
        _check_gemm_tensor(weight_u, "weight_u", torch.int32)
        _check_gemm_tensor(weight_v, "weight_v", torch.int32)
        for name, s in (("scale_g", scale_g), ("scale_l", scale_l), ("scale_h", scale_h)):
            _check_gemm_tensor(s, name, x.dtype)
        imm = torch.empty((t, r), dtype=x.dtype, device=x.device)
        _, m, _ = _onebit_check(imm, weight_v, None, scale_h, workspace)
        _check_bias(bias, m, x)
        if given is None:
            out = torch.empty((t, m), dtype=x.dtype, device=x.device)
        else:
            out = given[i]
            if (tuple(out.shape) != (t, m) or out.dtype != x.dtype or out.device != x.device or not out.is_contiguous()
                    or out.data_ptr() % 16 != 0):
                raise RuntimeError(f"outs[{i}] must be a contiguous, 16-byte aligned [{t}, {m}] tensor of {x.dtype} on {x.device}")
        outs.append(out)
        keep.append(imm)
        nbytes = max(nbytes, int(lib.nq_gemm_scratch_bytes(t, n, r)), int(lib.nq_gemm_scratch_bytes(t, r, m)))
        pv = lambda ten: None if ten is None else ten.data_ptr()
        arr_items.append(NqGemmTerm(pv(x), pv(weight_u), pv(weight_v), pv(scale_g), pv(scale_l), pv(scale_h), pv(bias),
                                    pv(imm), pv(out), n, r, m))
    tokens = xs[0].size(0)
    if tokens == 0:
        return outs
    device = xs[0].device
    group_max = int(lib.nq_gemm_group_max())
    scratch = _scratch(nbytes, device)
    mode = PANEL_MODES[panel]
    ws = None if mode == 2 else _panel_workspace(device)
    with torch.cuda.device(device):
        for lo in range(0, count, group_max):
            part = arr_items[lo:lo + group_max]
            arr = (NqGemmTerm * len(part))(*part)
            _lib.check(lib.nq_gemm_nanoquant_group_ws(arr, len(part), tokens, dt, _ptr(scratch), nbytes, _ptr(ws),
                                                      0 if ws is None else ws.numel(), mode, _stream(device)))
    return outs


def gemm_group_sum_forward(xs, term_groups, bias_groups=None, panel="auto"):
    """`[sum_t marlin_nanoquant_forward(x_i, *term_groups[i][t]) for i]`: weights that are sums of several binary
    low-rank terms (mixture of ranks) on the grouped prefill launches.  All terms of all weights share the two
    launches of `gemm_group_forward`; the t-th terms of all weights write into one flat buffer per t, weights with
    more terms first, so that the sums over the terms are one in-place add per extra term index instead of one
    per weight.  `xs`: one tensor or one per weight; `bias_groups`: optional list (per weight) of lists (per term) of
    bias tensors / None; `panel` as in `gemm_group_forward`.  Returns one [tokens, m] tensor per weight (views of one
    buffer)."""
    nw = len(term_groups)
    if nw == 0:
        return []
    if isinstance(xs, torch.Tensor):
        xs = [xs] * nw
    if len(xs) != nw or any(len(g) == 0 for g in term_groups):
        raise RuntimeError("one x and at least one term per weight")
    tokens, dtype, device = xs[0].size(0), xs[0].dtype, xs[0].device
    ms = [g[0][1].size(1) * 2 for g in term_groups]                  # weight_v [r / 16, m / 2]
    order = sorted(range(nw), key=lambda i: -len(term_groups[i]))      # stable: more terms first
    depth = len(term_groups[order[0]])
    sizes = [sum(tokens * ms[i] for i in order if len(term_groups[i]) > t) for t in range(depth)]
    bufs = [torch.empty(n, dtype=dtype, device=device) for n in sizes]
    flat_x, flat_terms, flat_bias, flat_out = [], [], [], []
    results = [None] * nw
    for t in range(depth):
        off = 0
        for i in order:
            if len(term_groups[i]) <= t:
                break
            m = ms[i]
            if (off * bufs[t].element_size()) % 16 != 0:
                raise RuntimeError("tokens * out_features must keep the outputs 16-byte aligned")
            view = bufs[t][off:off + tokens * m].view(tokens, m)
            off += tokens * m
            if t == 0:
                results[i] = view
            flat_x.append(xs[i])
            flat_terms.append(term_groups[i][t])
            flat_bias.append(None if bias_groups is None or bias_groups[i] is None else bias_groups[i][t])
            flat_out.append(view)
    gemm_group_forward(flat_x, flat_terms, flat_bias if any(b is not None for b in flat_bias) else None, outs=flat_out,
                       panel=panel)
    for t in range(1, depth):
        bufs[0][:sizes[t]].add_(bufs[t])
    return results


def gemv_mixture_forward(x, terms):
    """Sum of several binary low-rank terms sharing x.  terms: sequence of
    (scale_g, Ubits, scale_l | None, Vbits, scale_h) with the operand meaning of nanoquant_dyn_forward."""
    if len(terms) == 0:
        raise ValueError("at least one term is required")
    ranks, m = [], None
    for (scale_g, Ubits, scale_l, Vbits, scale_h) in terms:
        n, r, mm = _check_gemv_args(x, scale_g, Ubits, scale_l, Vbits, scale_h)
        if m is not None and mm != m:
            raise RuntimeError("all terms must have the same output size")
        m = mm
        ranks.append(r)
    lead = x.shape[:-1]
    batch = 1
    for d in lead:
        batch *= d
    y = torch.empty((batch, m), dtype=x.dtype, device=x.device)
    if batch == 0 or m == 0:
        return y.reshape(*lead, m)
    nt = len(terms)
    h = torch.empty((batch, max(max(ranks), 1)), dtype=torch.float32, device=x.device)
    yacc = torch.empty((batch, m), dtype=torch.float32, device=x.device) if nt > 1 else None

    def ptr_array(idx):
        arr = (ctypes.c_void_p * nt)()
        for i, term in enumerate(terms):
            t = term[idx]
            arr[i] = None if t is None else t.data_ptr()
        return arr

    rank_arr = (ctypes.c_int * nt)(*ranks)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().nq_gemv_mixture(_ptr(x), ptr_array(0), ptr_array(1), ptr_array(2), ptr_array(3),
                                              ptr_array(4), rank_arr, nt, _ptr(h), _ptr(yacc), _ptr(y),
                                              batch, n, m, _dtype_id(x), _stream(x.device)))
    return y.reshape(*lead, m)


def repack_words_device(packed: torch.Tensor, src: str, dst: str) -> torch.Tensor:
    for name in (src, dst):
        if name not in _lib.ORDER_IDS:
            raise ValueError(f"Unsupported method: '{name}'. Supported methods are 'lsb_first', 'half2'.")
    packed = packed.contiguous()
    out = torch.empty_like(packed)
    with torch.cuda.device(packed.device):
        _lib.check(_lib.lib().nq_repack_words(_ptr(packed), _ptr(out), packed.numel(), _lib.ORDER_IDS[src],
                                              _lib.ORDER_IDS[dst], _stream(packed.device)))
    return out


def pack_gemm_tiles_device(words: torch.Tensor, rows_padded: int, k_padded: int, method: str) -> torch.Tensor:
    """Device pass of packing.pack_gemm_tiles_from_words."""
    rows, nwords = words.shape
    out = torch.empty(rows_padded * k_padded // 32, dtype=torch.int32, device=words.device)
    with torch.cuda.device(words.device):
        _lib.check(_lib.lib().nq_pack_gemm_tiles(_ptr(words), _ptr(out), rows, nwords, rows_padded, k_padded,
                                                 _lib.ORDER_IDS[method], _stream(words.device)))
    return out


def gemv_stage_forward(inp: torch.Tensor, s_col: Optional[torch.Tensor], bits: torch.Tensor,
                       s_row: Optional[torch.Tensor]) -> torch.Tensor:
    """One matmul-free stage on its own: out[b, row] = s_row[row] * sum_c sgn(bits[row, c]) * inp[b, c] * s_col[c]
    (what one of the reference's two launches computes, kernel/cuda/gemv_kernel.cu:283-301).  `bits` [rows,
    ceil(cols/32)] in the "half2" order; the result has inp's dtype."""
    if inp.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("Support only Half or BFloat16")
    what = _FLOAT_WHAT[inp.dtype]
    _check_dev_cont(inp, "in", inp.dtype, what)
    _check_dev_cont(bits, "bits", torch.int32, "tensor dtype must be int32")
    for name, t in (("s_col", s_col), ("s_row", s_row)):
        if t is not None:
            _check_dev_cont(t, name, inp.dtype, what)
    cols = inp.size(-1)
    if bits.dim() != 2 or bits.size(1) != (cols + 31) // 32:
        raise RuntimeError(f"bits must be [rows, {(cols + 31) // 32}] for {cols} input columns")
    rows = bits.size(0)
    if (s_col is not None and s_col.numel() != cols) or (s_row is not None and s_row.numel() != rows):
        raise RuntimeError("scale size mismatch")
    lead = inp.shape[:-1]
    batch = 1
    for d in lead:
        batch *= d
    out = torch.empty((batch, rows), dtype=inp.dtype, device=inp.device)
    if batch > 0 and rows > 0:
        with torch.cuda.device(inp.device):
            _lib.check(_lib.lib().nq_gemv_stage(_ptr(inp), _ptr(s_col), _ptr(bits), _ptr(s_row), _ptr(out), batch, cols,
                                                rows, _dtype_id(inp), _stream(inp.device)))
    return out.reshape(*lead, rows)


def tile_words_device(packed: torch.Tensor, inverse: bool, shape=None) -> torch.Tensor:
    """Device pass of packing.tile_words / untile_words.  The kernel trusts its sizes: what it is handed is checked
    here (a GPU tensor of contiguous int32 words, exactly as many as the shape needs, 16-byte aligned on the tiled
    side)."""
    lib = _lib.lib()
    if not packed.is_cuda:
        raise RuntimeError("packed words must be a CUDA tensor")
    if packed.dtype != torch.int32 or not packed.is_contiguous():
        raise RuntimeError("packed words must be a contiguous int32 tensor")
    if not inverse:
        if packed.dim() != 2:
            raise RuntimeError("row-major words must be a 2-D tensor [rows, words]")
        rows, words = packed.shape
        out = torch.empty(int(lib.nq_tiled_words(rows, words)), dtype=torch.int32, device=packed.device)
    else:
        rows, words = (int(v) for v in shape)
        if rows < 0 or words < 0 or packed.dim() != 1 or packed.numel() != int(lib.nq_tiled_words(rows, words)):
            raise RuntimeError(f"tiled words of a [{rows}, {words}] matrix must be a flat tensor of "
                               f"{int(lib.nq_tiled_words(rows, words))} words, got {list(packed.shape)}")
        if packed.data_ptr() % 16 != 0:
            raise RuntimeError("tiled words must be 16-byte aligned")
        out = torch.empty((rows, words), dtype=torch.int32, device=packed.device)
    if rows > 0 and words > 0:
        with torch.cuda.device(packed.device):
            _lib.check(lib.nq_tile_words(_ptr(packed), _ptr(out), rows, words, int(inverse), _stream(packed.device)))
    return out


def get_kernel_function(namespace: str, dtype: torch.dtype, kernel_type: str):
    """Operator lookup with the reference's naming rule (src/nanoquant/kernel/utils.py:33-48)."""
    mid = "_dyn" if kernel_type != "fixed" else ""
    op_name = f"{namespace}{mid}_forward"
    try:
        return getattr(torch.ops.binary_kernels, op_name)
    except AttributeError as exc:
        have = dir(torch.ops.binary_kernels) if hasattr(torch.ops, "binary_kernels") else []
        raise AttributeError(f"Dispatcher op `{namespace}::{op_name}` not found. "
                             f"Available in torch.ops.binary_kernels: {have}") from exc


# ---------------------------------------------------------------------------------------------
# registration
# ---------------------------------------------------------------------------------------------
_library = torch.library.Library(_NS, "DEF")
for _schema in _SCHEMAS:
    _library.define(_schema)
_library.impl("nanoquant_dyn_forward", nanoquant_dyn_forward, "CUDA")
_library.impl("marlin_onebit_forward", marlin_onebit_forward, "CUDA")
_library.impl("marlin_nanoquant_forward", marlin_nanoquant_forward, "CUDA")
_library.impl("nanoquant_dyn_forward", _nanoquant_dyn_forward_meta, "Meta")
_library.impl("marlin_onebit_forward", _marlin_onebit_meta, "Meta")
_library.impl("marlin_nanoquant_forward", _marlin_nanoquant_meta, "Meta")
