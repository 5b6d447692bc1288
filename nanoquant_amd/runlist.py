"""Host side of the run-list decode path: many linears, one kernel launch.

`DecodeRunList` owns the device workspace (stage table + completion counters) and the fp32
intermediates of a list of linears; `run()` enqueues the single launch on the current stream and can
be captured in a HIP graph.  The reference has no such object: its decode path is one Python op call,
two allocations and two launches per linear (src/nanoquant/modules/linear.py:121-130,
src/nanoquant/kernel/cuda/gemv_kernel.cu:340-425).
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence

import torch

from . import _lib


class NqLinear(ctypes.Structure):
    """Mirror of `nq_linear` in include/nq_gfx950.h."""
    _fields_ = [
        ("x", ctypes.c_void_p), ("s_in", ctypes.c_void_p), ("vt_bits", ctypes.c_void_p), ("s_mid", ctypes.c_void_p),
        ("u_bits", ctypes.c_void_p), ("s_out", ctypes.c_void_p), ("h", ctypes.c_void_p), ("y", ctypes.c_void_p),
        ("addend", ctypes.c_void_p),
        ("n", ctypes.c_int), ("r", ctypes.c_int), ("m", ctypes.c_int),
        ("x_from", ctypes.c_int), ("y_from", ctypes.c_int), ("out_f32", ctypes.c_int),
        ("bias", ctypes.c_void_p), ("tiled", ctypes.c_int),
    ]


class NqRunlistPlan(ctypes.Structure):
    """Mirror of `nq_runlist_plan`."""
    _fields_ = [("nlinears", ctypes.c_int), ("nstages", ctypes.c_int), ("nphases", ctypes.c_int),
                ("workgroups", ctypes.c_int), ("max_units", ctypes.c_int), ("batch", ctypes.c_int),
                ("dtype", ctypes.c_int), ("index_words", ctypes.c_int), ("bound", ctypes.c_int),
                ("spin_limit", ctypes.c_int)]


class DecodeRunList:
    BATCHES = (1, 2, 4, 8, 16)

    def __init__(self, batch: int, dtype: torch.dtype = torch.float16, device=None, interleave: int = 2,
                 deterministic: bool = False):
        """`deterministic=True`: every launch of the list gives bit-identical outputs.  Up to batch 4 partial sums are
        rounded to a grid on which additions are exact, at a small cost in precision; without it the order in which
        the wavefronts of a workgroup add up a row sum is left to the hardware and the last bit may differ from launch
        to launch.  At batch 8 and 16 one wavefront forms every row sum in a fixed order: launches repeat bit for bit
        either way and the switch changes nothing."""
        if batch not in self.BATCHES:
            raise ValueError(f"run-list batch must be one of {self.BATCHES}, got {batch}")
        if dtype not in (torch.float16, torch.bfloat16):
            raise RuntimeError("Support only Half or BFloat16")
        self.batch = batch
        self.dtype = dtype
        self.device = torch.device(device if device is not None else "cuda")
        self.interleave = interleave
        self.deterministic = bool(deterministic)
        # polls after which a dependency wait inside the kernel gives up (then status() == 1 and the outputs of that
        # launch are invalid); 0 = the library's default, about a second.  Takes effect with the next run().
        self.spin_limit = 0
        self._entries: List[dict] = []
        self._keep: list = []          # tensors referenced by raw pointers stay alive here
        self._workspace: Optional[torch.Tensor] = None
        # > 0: every so many launches `run` reads the status word (a synchronisation) and raises if a dependency wait
        # expired since the last check; never while the stream is being captured.  0: the caller polls `status()`.
        self.status_check_every = 0
        self._runs = 0

    # ---- building -----------------------------------------------------------------------------
    def add(self, x: Optional[torch.Tensor], scale_pre: torch.Tensor, V_int8: torch.Tensor, scale_mid: Optional[torch.Tensor],
            U_int8: torch.Tensor, scale_post: torch.Tensor, y: Optional[torch.Tensor] = None,
            x_from: int = -1, addend: Optional[torch.Tensor] = None, y_from: int = -1,
            out_f32: bool = False, bias: Optional[torch.Tensor] = None, tiled: bool = False,
            bind_y: bool = False) -> int:
        """Append one linear (operands as `NanoQuantLinear` holds them after `_prepare_kernel('gemv')`:
        V_int8 [r, n/32] first stage, U_int8 [m, r/32] second stage).  Returns its index; `y` is
        allocated when not given and is available as `outputs[index]`.  `bias` [m] is added after `scale_post`.

        `x=None` leaves the input unbound and `bind_y=True` the output: `run(x=..., y=...)` supplies them
        with each launch (one pointer each for the whole list), so one built list serves any tensors."""
        if x is None and x_from >= 0:
            raise RuntimeError("an entry fed by another entry cannot take a late-bound input")
        if bind_y and y is not None:
            raise RuntimeError("bind_y leaves the output to run(); do not pass y as well")
        n = scale_pre.numel() if x is None else x.shape[-1]
        if tiled:
            # tile order (packing.tile_words): flat buffers, the rank comes from scale_mid / the word count
            if scale_mid is None:
                raise RuntimeError("tiled factors need scale_mid (its length is the rank)")
            r, m = scale_mid.numel(), scale_post.numel()
        else:
            r, m = V_int8.shape[0], U_int8.shape[0]
        for name, t, dt in (("x", x, self.dtype), ("scale_pre", scale_pre, self.dtype), ("scale_post", scale_post, self.dtype),
                            ("V_int8", V_int8, torch.int32), ("U_int8", U_int8, torch.int32)):
            if t is None:
                continue
            if not t.is_cuda or not t.is_contiguous() or t.dtype != dt:
                raise RuntimeError(f"{name} must be a contiguous {dt} tensor on the GPU")
        if x is not None and x.numel() != self.batch * n:
            raise RuntimeError(f"x must hold {self.batch} rows of {n}")
        if tiled:
            lib = _lib.lib()
            if V_int8.numel() != lib.nq_tiled_words(r, (n + 31) // 32) or U_int8.numel() != lib.nq_tiled_words(m, (r + 31) // 32):
                raise RuntimeError("tiled factor sizes do not match the shapes")
        elif V_int8.shape[1] != (n + 31) // 32 or U_int8.shape[1] != (r + 31) // 32:
            raise RuntimeError("packed factor shapes do not match x / each other")
        if scale_pre.numel() != n or scale_post.numel() != m or (scale_mid is not None and scale_mid.numel() != r):
            raise RuntimeError("scale size mismatch")
        if bias is not None and (not bias.is_cuda or not bias.is_contiguous() or bias.dtype != self.dtype or bias.numel() != m):
            raise RuntimeError(f"bias must be a contiguous {self.dtype} tensor of {m} elements on the GPU")
        if y is None and not bind_y:
            y = torch.empty((self.batch, m), dtype=torch.float32 if out_f32 else self.dtype, device=self.device)
        h = torch.empty((self.batch, r), dtype=torch.float32, device=self.device)
        self._keep += [x, scale_pre, V_int8, scale_mid, U_int8, scale_post, y, h, addend, bias]
        self._entries.append(dict(x=x, s_in=scale_pre, vt=V_int8, s_mid=scale_mid, u=U_int8, s_out=scale_post, h=h, y=y,
                                  addend=addend, n=n, r=r, m=m, x_from=x_from, y_from=y_from, out_f32=int(out_f32),
                                  bias=bias, tiled=int(tiled)))
        self._workspace = None
        return len(self._entries) - 1

    @property
    def outputs(self) -> Sequence[torch.Tensor]:
        return [e["y"] for e in self._entries]

    def build(self) -> None:
        n = len(self._entries)
        if n == 0:
            raise ValueError("empty run list")
        arr = (NqLinear * n)()
        p = lambda t: None if t is None else t.data_ptr()
        for i, e in enumerate(self._entries):
            arr[i] = NqLinear(p(e["x"]), p(e["s_in"]), p(e["vt"]), p(e["s_mid"]), p(e["u"]), p(e["s_out"]), p(e["h"]),
                              p(e["y"]), p(e["addend"]), e["n"], e["r"], e["m"], e["x_from"], e["y_from"], e["out_f32"],
                              p(e["bias"]), e["tiled"])
        lib = _lib.lib()
        nbytes = int(lib.nq_runlist_workspace_bytes(arr, n))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        with torch.cuda.device(self.device):
            stream = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
            plan = NqRunlistPlan()
            _lib.check(lib.nq_runlist_build(arr, n, self.batch, self._dtype_id(), self.interleave,
                                            ctypes.c_void_p(ws.data_ptr()), nbytes, ctypes.byref(plan), stream))
        if self.deterministic:
            _lib.check(lib.nq_runlist_set_deterministic(ctypes.byref(plan), 1))
        self._plan = plan
        self._workspace = ws
        self._needs = (any(e["x"] is None for e in self._entries), any(e["y"] is None for e in self._entries))

    def _dtype_id(self) -> int:
        return _lib.NQ_F16 if self.dtype == torch.float16 else _lib.NQ_BF16

    # ---- running --------------------------------------------------------------------------------
    def run(self, x: Optional[torch.Tensor] = None, y: Optional[torch.Tensor] = None) -> Sequence[torch.Tensor]:
        """Enqueue the launch on the current stream (no allocation, no synchronisation).  `x` / `y` are
        the tensors of the entries added with `x=None` / `bind_y=True`."""
        if self._workspace is None:
            self.build()
        need_x, need_y = self._needs        # fixed at build(): a launch costs microseconds, a scan of a long list more
        if need_x != (x is not None) or need_y != (y is not None):
            raise RuntimeError("run(x=, y=) must be given exactly when the list has late-bound entries")
        for name, t, key in (("x", x, "n"), ("y", y, "m")):
            if t is None:
                continue
            ent = [e for e in self._entries if e[name] is None]
            width = ent[0][key]
            dt = torch.float32 if (name == "y" and ent[0]["out_f32"]) else self.dtype
            if any(e[key] != width for e in ent) or (name == "y" and any(e["out_f32"] != ent[0]["out_f32"] for e in ent)):
                raise RuntimeError(f"late-bound entries must agree on the shape of {name}")
            if not t.is_cuda or not t.is_contiguous() or t.dtype != dt or t.numel() != self.batch * width:
                raise RuntimeError(f"{name} must be a contiguous {dt} tensor of {self.batch} x {width} on the GPU")
        p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
        self._plan.spin_limit = int(self.spin_limit)
        with torch.cuda.device(self.device):
            stream = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
            _lib.check(_lib.lib().nq_runlist_run_bound(ctypes.c_void_p(self._workspace.data_ptr()),
                                                       ctypes.byref(self._plan), p(x), p(y), stream))
        self._runs += 1
        if self.status_check_every > 0 and self._runs % self.status_check_every == 0 \
                and not torch.cuda.is_current_stream_capturing():
            if self.status() != 0:
                raise RuntimeError("a dependency wait of a run-list launch expired since the last check (is the GPU shared "
                                   "with other kernels?): the outputs of that launch are invalid")
        return self.outputs

    def status(self) -> int:
        """Synchronises.  0 = ok; 1 = a dependency wait ran into its bound in some launch since the last call (the
        results of that launch are invalid: the kernel needs the GPU to itself).  Reading clears the flag."""
        out = ctypes.c_int(0)
        with torch.cuda.device(self.device):
            stream = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
            _lib.check(_lib.lib().nq_runlist_status(ctypes.c_void_p(self._workspace.data_ptr()), ctypes.byref(out), stream))
        return out.value
