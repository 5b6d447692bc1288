"""Quantized-linear module interface of the reference, inference side.

`NanoQuantLinear` keeps the attribute names and call protocol of
src/nanoquant/modules/linear.py (forward :106-150, _prepare_kernel :152-204, _compute_forward
:248-257, pack_weights/state_dict :288-321): dense +-1 factors `V` [rank, in] and `U` [out, rank]
with scales `scale_pre` [1, in], `scale_mid` [1, rank] (optional) and `scale_post` [1, out]; after
`_prepare_kernel(kernel_type, dtype)` the dense factors are replaced by packed words and `forward`
calls the `torch.ops.binary_kernels` operator.  The quantizer-side parts (latent weights, STE,
finalize) are not part of this package.

`MixtureOfRankLinear` sums several such terms (the sub-1-bit mixture-of-rank layout); the reference
describes it but ships no code for it, so its definition here is the sum of single-term layers.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .runlist import DecodeRunList
from .packing import (binary_packer, marlin_nanoquant_packer, pack_binary_marlin_fused_from_words, repack_words)


def _sign_pm1(x: torch.Tensor) -> torch.Tensor:
    y = x.sign()
    y[y == 0] = 1
    return y


class NanoQuantLinear(nn.Module):
    def __init__(self, in_features: int, out_features: int, rank: int, bias: bool = False,
                 has_scale_mid: bool = True, device=None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.rank = rank
        self.do_train = False
        self._binarized = True
        self.dtype = dtype
        # False mirrors the reference, whose kernel paths return before the bias is added; True adds it in the
        # epilogue of the last kernel (decode and prefill alike).
        self.kernel_path_bias = False
        # True: a decode call of 1, 2, 4, 8 or 16 rows is ONE launch of the run-list kernel (both stages, the
        # scales and the bias) on a list built once per row count, instead of the two launches of the
        # reference's op (linear.py:121-130).  It bypasses the torch op, so leave it off under torch.compile.
        self.fused_launch = False
        # With fused_launch: every so many launches of a list the status word is read back (one synchronisation) and an
        # expired wait raises; the first launch of a list is always checked.  0: only `fused_status()` tells.
        self.fused_status_every = 256
        # Opt-in (0: never): a module prepared for decode ("gemv") sends calls of at least this many rows to the
        # few-token MFMA tiles of the prefill path, whose cost does not grow with the row count while that of the
        # decode kernels does; 3 is the break-even on a Llama-2-7B layer.  The price is a second copy of the packed
        # factors (the prefill tiles, built once from the decode words on the device, on the first such call or by
        # `prepare_mfma_route()`, and kept beside them), and results that differ in the last bits from the decode
        # kernels' (other order of the fp32 additions, h rounded to 16 bits in between).  Needs
        # in_features % 256 == 0 and out_features % 32 == 0; other shapes stay on the decode kernels.
        self.mfma_from_rows = 0
        self._mfma_tiles = None
        self._fused_lists = {}
        self._fused_tiled = None
        self._fused_bias = None
        self.register_parameter("weight", None)
        if bias:
            self.bias = nn.Parameter(torch.zeros(out_features, device=device, dtype=dtype), requires_grad=False)
        else:
            self.register_parameter("bias", None)
        self._alloc(has_scale_mid, device)

    # ---- construction ------------------------------------------------------------------------
    def _alloc(self, has_scale_mid: bool, device) -> None:
        def p(*shape):
            return nn.Parameter(torch.empty(*shape, device=device, dtype=self.dtype), requires_grad=False)

        self.scale_pre = p(1, self.in_features)
        self.scale_post = p(1, self.out_features)
        self.V = p(self.rank, self.in_features)
        self.U = p(self.out_features, self.rank)
        if has_scale_mid:
            self.scale_mid = p(1, self.rank)

    def init_for_inference(self, rank: int, has_scale_mid: bool = False) -> None:
        """Re-shape the module for a given rank (reference: linear.py:86-99)."""
        self.rank = rank
        self.do_train = False
        self._binarized = True
        self.dtype = torch.bfloat16
        device = self.bias.device if self.bias is not None else None
        if hasattr(self, "scale_mid"):
            delattr(self, "scale_mid")
        self._alloc(has_scale_mid, device)

    @classmethod
    def from_factors(cls, V: torch.Tensor, U: torch.Tensor, scale_pre: torch.Tensor,
                     scale_mid: Optional[torch.Tensor], scale_post: torch.Tensor,
                     bias: Optional[torch.Tensor] = None, dtype: torch.dtype = torch.bfloat16) -> "NanoQuantLinear":
        """V [rank, in] and U [out, rank] hold +-1 (any dtype); scales are 1-D or [1, D]."""
        rank, in_f = V.shape
        out_f = U.shape[0]
        mod = cls(in_f, out_f, rank, bias=bias is not None, has_scale_mid=scale_mid is not None,
                  device=V.device, dtype=dtype)
        with torch.no_grad():
            mod.V.copy_(_sign_pm1(V.float()))
            mod.U.copy_(_sign_pm1(U.float()))
            mod.scale_pre.copy_(scale_pre.reshape(1, -1))
            mod.scale_post.copy_(scale_post.reshape(1, -1))
            if scale_mid is not None:
                mod.scale_mid.copy_(scale_mid.reshape(1, -1))
            if bias is not None:
                mod.bias.copy_(bias)
        return mod

    # ---- forward -----------------------------------------------------------------------------
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if getattr(self, "do_kernel_inference", False):
            orig_dtype = x.dtype
            if x.dtype != self.dtype:
                x = x.to(self.dtype)
            original_shape = None
            if x.ndim == 3:
                original_shape = x.shape
                x = x.contiguous().view(-1, x.size(-1))
            elif x.ndim == 2:
                x = x.contiguous()
            else:
                raise ValueError(f"Expected 2D or 3D input tensor, got {x.ndim}D")

            # As in the reference (linear.py:121-141) the kernel paths do not add the bias, unless
            # `kernel_path_bias` is set: then it is added in the epilogue of the last kernel.
            bias = None
            if self.kernel_path_bias and self.bias is not None:
                bias = self.bias if self.bias.dtype == self.dtype else self.bias.to(self.dtype)
            if self.kernel_type == "gemv" and self.fused_launch and x.shape[0] in DecodeRunList.BATCHES:
                y = self._fused_forward(x, bias)
            elif self.kernel_type == "gemv" and self._routes_to_mfma(x):
                tiles = self._mfma_tiles
                if bias is not None:
                    y = ops.gemm_forward_with_bias(x, *tiles, bias)
                else:
                    y = torch.ops.binary_kernels.marlin_nanoquant_forward(x, *tiles)
            elif self.kernel_type == "gemv":
                if bias is not None:
                    y = ops.gemv_forward_with_bias(x, self.scale_pre, self.V_int8, self.scale_mid, self.U_int8,
                                                   self.scale_post, bias)
                else:
                    y = self.kernel_forward(x, self.scale_pre, self.V_int8, self.scale_mid, self.U_int8,
                                            self.scale_post, **self.kernel_kwargs)
            elif self.kernel_type == "gemm":
                if bias is not None:
                    y = ops.gemm_forward_with_bias(x, self.V_int8, self.U_int8, self.s1, self.s2, self.s3, self.workspace,
                                                   bias)
                else:
                    y = self.kernel_forward(x, self.V_int8, self.U_int8, self.s1, self.s2, self.s3, self.workspace)
            else:
                raise ValueError(f"Unknown kernel_type: {self.kernel_type}")
            if original_shape is not None:
                y = y.view(original_shape[0], original_shape[1], -1)
            return y.to(orig_dtype) if y.dtype != orig_dtype else y

        s_mid = getattr(self, "scale_mid", None)
        y = self._compute_forward(x, self.V, self.U, self.scale_pre, s_mid, self.scale_post)
        if self.bias is not None:
            y += self.bias
        return y

    def _routes_to_mfma(self, x: torch.Tensor) -> bool:
        """Whether this decode call runs on the prefill path's few-token tiles; builds them on first use (eagerly:
        under torch.compile and during a stream capture only tiles made beforehand are used)."""
        if not self.mfma_from_rows or x.shape[0] < self.mfma_from_rows or not x.is_cuda:
            return False
        if self.in_features % 256 != 0 or self.out_features % 32 != 0:
            return False
        if self._mfma_tiles is None or self._mfma_tiles[0].device != x.device:
            # never build inside a trace or a stream capture (the packing pass and its allocations would become part
            # of the graph): such a call stays on the decode kernels unless the tiles were prepared beforehand
            if torch.compiler.is_compiling() or torch.cuda.is_current_stream_capturing():
                return False
            self.prepare_mfma_route()
        return True

    def prepare_mfma_route(self) -> None:
        """Prefill tiles (the 6-tuple of `marlin_nanoquant_packer`) from the decode words of a module prepared with
        kernel_type "gemv": one pass over the words on their device, no dense matrix."""
        if not getattr(self, "do_kernel_inference", False) or self.kernel_type != "gemv":
            raise RuntimeError("prepare_mfma_route() needs a module prepared with kernel_type='gemv'")
        if self.in_features % 256 != 0 or self.out_features % 32 != 0:
            raise ValueError("the prefill path needs in_features % 256 == 0 and out_features % 32 == 0")
        self._mfma_tiles = pack_binary_marlin_fused_from_words(
            self.V_int8, self.U_int8, self.rank, self.scale_pre.data,
            None if self.scale_mid is None else self.scale_mid.data, self.scale_post.data, "half2")

    def _fused_forward(self, x: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
        """One launch for the whole layer: a one-entry run list per row count whose input and output are
        bound at launch.  Up to 4 rows the list reads a tile-order copy of the packed factors (made once,
        one more bit per weight of device memory); above, the row-major words the op reads."""
        rows = x.shape[0]
        if not x.is_cuda:
            raise RuntimeError("the fused decode launch needs GPU tensors")
        if x.data_ptr() % 16 != 0:
            x = x.clone()
        if bias is not None and bias is not self.bias:     # a converted copy: keep one, so that the list can point at it
            tag = (self.bias.data_ptr(), self.bias._version)
            if self._fused_bias is None or self._fused_bias[0] != tag:
                self._fused_bias = (tag, bias.contiguous())
            bias = self._fused_bias[1]
        key = (rows, None if bias is None else bias.data_ptr(), x.device)
        rl = self._fused_lists.get(key)
        if rl is None:
            tiled = rows <= 4
            if tiled:
                if self._fused_tiled is None:
                    self._fused_tiled = (ops.tile_words_device(self.V_int8, False), ops.tile_words_device(self.U_int8, False))
                V, U = self._fused_tiled
            else:
                V, U = self.V_int8, self.U_int8
            scale_mid = self.scale_mid
            if tiled and scale_mid is None:      # the tile order carries no rank: a unit scale_mid supplies it
                scale_mid = torch.ones(self.V_int8.shape[0], dtype=self.dtype, device=x.device)
            rl = DecodeRunList(rows, dtype=self.dtype, device=x.device)
            rl.add(None, self.scale_pre, V, scale_mid, U, self.scale_post, bias=bias, tiled=tiled, bind_y=True)
            rl.build()
            rl.status_check_every = self.fused_status_every
            self._fused_lists[key] = rl
            # The first launch of a new list is checked (one synchronisation per list): the kernel needs its whole
            # grid resident at once, and a device shared with other work makes its bounded waits expire.
            y = torch.empty((rows, self.scale_post.numel()), dtype=self.dtype, device=x.device)
            rl.run(x=x, y=y)
            if rl.status() != 0:
                del self._fused_lists[key]
                raise RuntimeError("the fused decode launch could not keep its grid resident (is the GPU shared with "
                                   "other kernels?); set fused_launch = False to use the two-launch operator")
            return y
        y = torch.empty((rows, self.scale_post.numel()), dtype=self.dtype, device=x.device)
        rl.run(x=x, y=y)
        return y

    def fused_status(self) -> int:
        """Synchronises.  0 when no fused launch of this module has run into its bounded dependency wait since the
        last call; 1 otherwise (the outputs of such a launch are invalid).  Reading clears the flag."""
        worst = 0
        for rl in self._fused_lists.values():
            worst = max(worst, rl.status())
        return worst

    def _compute_forward(self, x, V, U, scale_pre, scale_mid, scale_post):
        """Dense definition of the layer (reference: linear.py:248-257)."""
        y = F.linear(x * scale_pre, V)
        if scale_mid is not None:
            y = y * scale_mid
        y = F.linear(y, U)
        return y * scale_post

    # ---- kernel preparation --------------------------------------------------------------------
    def _prepare_kernel(self, kernel_type: str = "gemv", dtype: torch.dtype = torch.float16) -> None:
        if kernel_type == "gemlite":
            raise NotImplementedError("the GemLite/Triton backend is not part of the gfx950 implementation")
        if kernel_type not in ("gemv", "gemm"):
            raise ValueError("kernel_type must be one of ['gemv', 'gemm', 'gemlite'].")
        self.do_kernel_inference = True
        self.kernel_type = kernel_type
        self.dtype = dtype
        self._fused_lists, self._fused_tiled, self._fused_bias = {}, None, None
        self._mfma_tiles = None

        self.scale_pre = nn.Parameter(self.scale_pre.to(dtype).squeeze(0), requires_grad=False)
        self.scale_post = nn.Parameter(self.scale_post.to(dtype).squeeze(0), requires_grad=False)
        self.scale_mid = getattr(self, "scale_mid", None)
        if self.scale_mid is not None:
            self.scale_mid = nn.Parameter(self.scale_mid.to(dtype).squeeze(0), requires_grad=False)

        if kernel_type == "gemv":
            self.U_int8 = binary_packer(self.U.to(torch.int8), method="half2")
            self.V_int8 = binary_packer(self.V.to(torch.int8), method="half2")
            delattr(self, "U")
            delattr(self, "V")
            self.kernel_forward = ops.get_kernel_function("nanoquant", dtype, kernel_type="dynamic")
            # Tuning hints of the CUDA kernels, passed through unchanged (linear.py:176-185); the
            # gfx950 op validates and ignores them.
            self.kernel_kwargs = {
                "num_thread_stage1": 128, "num_thread_stage2": 128,
                "num_row_per_warp_stage1": 2, "num_row_per_warp_stage2": 2,
                "num_acc_stage1": 1, "num_acc_stage2": 1,
                "num_pipeline_stage1": 8, "num_pipeline_stage2": 8,
            }
        else:
            if self.scale_mid is None:
                self.scale_mid = nn.Parameter(torch.ones(self.rank, device=self.scale_pre.device, dtype=dtype),
                                              requires_grad=False)
            (self.V_int8, self.U_int8, self.s1, self.s2, self.s3, self.workspace) = marlin_nanoquant_packer(
                self.V.to(torch.int8).T, self.U.to(torch.int8).T, self.scale_pre.data, self.scale_mid.data,
                self.scale_post.data)
            for key in ["U", "V", "scale_pre", "scale_mid", "scale_post"]:
                delattr(self, key)
            self.kernel_forward = torch.ops.binary_kernels.marlin_nanoquant_forward

    # ---- packed checkpoint format ----------------------------------------------------------------
    def pack_weights(self) -> dict:
        """{V,U}_packed int32 `lsb_first` words + {V,U}_shape (reference: linear.py:288-305)."""
        packed = {}
        for name in ("V", "U"):
            param = getattr(self, name, None)
            if param is None:
                continue
            packed[f"{name}_packed"] = binary_packer(_sign_pm1(param.data.float()).to(torch.int8))
            packed[f"{name}_shape"] = torch.tensor(param.shape, dtype=torch.long)
        return packed

    def state_dict(self, *args, **kwargs):
        state = super().state_dict(*args, **kwargs)
        prefix = kwargs.get("prefix", "")
        for k in [k for k in state.keys() if k in (prefix + "V", prefix + "U")]:
            del state[k]
        for k, v in self.pack_weights().items():
            state[prefix + k] = v
        return state

    def load_packed(self, state: dict, prefix: str = "", kernel_type: str = "gemv",
                    dtype: torch.dtype = torch.float16) -> None:
        """Load a packed checkpoint entry.  The dense +-1 matrices of the reference's loader
        (src/nanoquant/utils/load_utils.py:269-293) are never materialised: for the decode path the `lsb_first`
        words are permuted to the kernel's `half2` order word by word, for the prefill path they go to the 32 x 256
        tiles in one pass over the words (with the rank padding of the reference's packer, kernel/utils.py:262-271)."""
        dev = self.scale_pre.device
        v_shape = tuple(int(v) for v in state[prefix + "V_shape"])
        u_shape = tuple(int(v) for v in state[prefix + "U_shape"])
        self.rank = v_shape[0]
        for name in ("scale_pre", "scale_post", "scale_mid"):
            key = prefix + name
            if key in state:
                setattr(self, name, nn.Parameter(state[key].to(dev, self.dtype).reshape(1, -1), requires_grad=False))
            elif name == "scale_mid" and hasattr(self, "scale_mid"):
                delattr(self, "scale_mid")
        v_words = state[prefix + "V_packed"].to(dev)
        u_words = state[prefix + "U_packed"].to(dev)
        if kernel_type not in ("gemv", "gemm"):
            raise ValueError("kernel_type must be one of ['gemv', 'gemm'].")
        if u_shape[1] != v_shape[0] or tuple(v_words.shape) != (v_shape[0], (v_shape[1] + 31) // 32) or \
                tuple(u_words.shape) != (u_shape[0], (u_shape[1] + 31) // 32):
            raise ValueError("packed factor shapes do not match V_shape / U_shape")
        for name in ("V", "U"):
            if hasattr(self, name):
                delattr(self, name)
        self.in_features, self.out_features = v_shape[1], u_shape[0]
        self._fused_lists, self._fused_tiled, self._fused_bias = {}, None, None   # built on the previous words
        self._mfma_tiles = None
        self._prepare_scales_only(dtype)
        if kernel_type == "gemv":
            self.V_int8 = repack_words(v_words, "lsb_first", "half2")
            self.U_int8 = repack_words(u_words, "lsb_first", "half2")
        else:
            if v_shape[1] % 256 != 0 or u_shape[0] % 32 != 0:
                raise ValueError("the prefill path needs in_features % 256 == 0 and out_features % 32 == 0")
            self.kernel_type = "gemm"
            (self.V_int8, self.U_int8, self.s1, self.s2, self.s3, self.workspace) = pack_binary_marlin_fused_from_words(
                v_words, u_words, self.rank, self.scale_pre.data, None if self.scale_mid is None else self.scale_mid.data,
                self.scale_post.data, "lsb_first")
            for key in ["scale_pre", "scale_mid", "scale_post", "kernel_kwargs"]:
                delattr(self, key)
            self.kernel_forward = torch.ops.binary_kernels.marlin_nanoquant_forward

    def _prepare_scales_only(self, dtype: torch.dtype) -> None:
        self.do_kernel_inference = True
        self.kernel_type = "gemv"
        self.dtype = dtype
        self.scale_pre = nn.Parameter(self.scale_pre.to(dtype).squeeze(0), requires_grad=False)
        self.scale_post = nn.Parameter(self.scale_post.to(dtype).squeeze(0), requires_grad=False)
        self.scale_mid = getattr(self, "scale_mid", None)
        if self.scale_mid is not None:
            self.scale_mid = nn.Parameter(self.scale_mid.to(dtype).squeeze(0), requires_grad=False)
        self.kernel_forward = ops.get_kernel_function("nanoquant", dtype, kernel_type="dynamic")
        self.kernel_kwargs = {
            "num_thread_stage1": 128, "num_thread_stage2": 128,
            "num_row_per_warp_stage1": 2, "num_row_per_warp_stage2": 2,
            "num_acc_stage1": 1, "num_acc_stage2": 1,
            "num_pipeline_stage1": 8, "num_pipeline_stage2": 8,
        }


def prefill_group(modules: Sequence, x) -> list:
    """`[mod(x) for mod in modules]` for modules prepared with `_prepare_kernel("gemm")`, with the GEMMs of all
    modules sharing launches (`ops.gemm_group_forward`): the projections of a decoder block that read the same
    tokens (q/k/v, gate/up).  `x` is one tensor for all modules or a list of one tensor per module, 2-D or 3-D as
    `forward` takes it (linear.py:106-141 of the reference launches each module by itself).  A
    `MixtureOfRankLinear` among the modules contributes all its terms to the shared launches; its output is the
    sum of their outputs."""
    entries = list(modules)
    if not entries:
        return []
    xs_in = [x] * len(entries) if isinstance(x, torch.Tensor) else list(x)
    if len(xs_in) != len(entries):
        raise ValueError("one input per module")
    mods, xs, owner = [], [], []               # one entry per term; owner = index of the module it belongs to
    for i, (entry, t) in enumerate(zip(entries, xs_in)):
        for mod in (entry.terms if isinstance(entry, MixtureOfRankLinear) else (entry,)):
            mods.append(mod)
            xs.append(t)
            owner.append(i)
    for mod in mods:
        if not getattr(mod, "do_kernel_inference", False) or mod.kernel_type != "gemm":
            raise ValueError("prefill_group needs modules prepared with _prepare_kernel('gemm', dtype)")
        if mod.dtype != mods[0].dtype:
            raise ValueError("all modules of a group must be prepared for the same dtype")
    flat, cache = [], {}
    for t in xs:
        if t.ndim not in (2, 3):
            raise ValueError(f"Expected 2D or 3D input tensor, got {t.ndim}D")
        if id(t) not in cache:                 # a shared input is converted once
            v = t if t.dtype == mods[0].dtype else t.to(mods[0].dtype)
            cache[id(t)] = v.contiguous().view(-1, v.size(-1))
        flat.append(cache[id(t)])
    biases = []
    for mod in mods:
        b = mod.bias if (mod.kernel_path_bias and mod.bias is not None) else None
        biases.append(None if b is None else (b if b.dtype == mod.dtype else b.to(mod.dtype)))
    pack = lambda m: (m.V_int8, m.U_int8, m.s1, m.s2, m.s3, m.workspace)
    if len(mods) == len(entries):              # no mixtures: one output per module
        outs = ops.gemm_group_forward(flat, [pack(m) for m in mods], biases if any(b is not None for b in biases) else None)
    else:                                      # the terms of a mixture are summed (one add per extra term index)
        groups, bias_groups, group_x = [[] for _ in entries], [[] for _ in entries], [None] * len(entries)
        for mod, xf, b, i in zip(mods, flat, biases, owner):
            groups[i].append(pack(mod))
            bias_groups[i].append(b)
            group_x[i] = xf
        outs = ops.gemm_group_sum_forward(group_x, groups, bias_groups if any(b is not None for b in biases) else None)
    for i, t in enumerate(xs_in):
        y = outs[i]
        if t.ndim == 3:
            y = y.view(t.shape[0], t.shape[1], -1)
        outs[i] = y.to(t.dtype) if y.dtype != t.dtype else y
    return outs


def decode_group(modules: Sequence, x) -> list:
    """`[mod(x) for mod in modules]` for modules prepared with `_prepare_kernel("gemv")`, with the stages of all
    modules sharing launches (`ops.gemv_group_forward`; pieces of 1, 2 and 4 rows, two launches per 8 modules): what a
    decoder issues per layer at decode time is then eight launches, two each for {q,k,v}, {o}, {gate,up}, {down}, with
    its attention, norms and activations between them, instead of the reference's two launches per module
    (linear.py:121-130).  No run list is built: any activations on every call, no requirement on what else the GPU
    runs; only the checked operand table of the group (`ops.GemvGroup`) is kept with the first module, and rebuilt
    when a module's tensors are replaced.  `x` is one tensor for all modules or a list of one tensor per module, 2-D or 3-D as `forward` takes it."""
    mods = list(modules)
    if not mods:
        return []
    xs_in = [x] * len(mods) if isinstance(x, torch.Tensor) else list(x)
    if len(xs_in) != len(mods):
        raise ValueError("one input per module")
    for mod in mods:
        if not getattr(mod, "do_kernel_inference", False) or getattr(mod, "kernel_type", None) != "gemv":
            raise ValueError("decode_group needs modules prepared with _prepare_kernel('gemv', dtype)")
        if mod.dtype != mods[0].dtype:
            raise ValueError("all modules of a group must be prepared for the same dtype")
    flat, cache = [], {}
    for t in xs_in:
        if t.ndim not in (2, 3):
            raise ValueError(f"Expected 2D or 3D input tensor, got {t.ndim}D")
        if id(t) not in cache:                 # a shared input is converted once
            v = t if t.dtype == mods[0].dtype else t.to(mods[0].dtype)
            cache[id(t)] = v.contiguous().view(-1, v.size(-1))
        flat.append(cache[id(t)])
    biases = []
    for mod in mods:
        b = mod.bias if (mod.kernel_path_bias and mod.bias is not None) else None
        biases.append(None if b is None else (b if b.dtype == mod.dtype else b.to(mod.dtype)))
    # the operands are checked once per set of modules and tensors: a prepared group is kept while every operand is
    # still the tensor it was built on
    operands = [(m.scale_pre, m.V_int8, m.scale_mid, m.U_int8, m.scale_post) for m in mods]
    cache = mods[0].__dict__.setdefault("_decode_groups", {})      # lives and dies with the first module of the group
    key = tuple(id(m) for m in mods)
    hit = cache.get(key)
    if hit is None or len(hit[1]) != len(operands) or any(a is not b for old, new in zip(hit[1], operands) for a, b in zip(old, new)) \
            or any(a is not b for a, b in zip(hit[2], biases)):
        if len(cache) >= 16:
            cache.clear()
        hit = (ops.GemvGroup(operands, biases if any(b is not None for b in biases) else None), operands, list(biases))
        cache[key] = hit
    outs = hit[0](flat)
    for i, t in enumerate(xs_in):
        y = outs[i]
        if t.ndim == 3:
            y = y.view(t.shape[0], t.shape[1], -1)
        outs[i] = y.to(t.dtype) if y.dtype != t.dtype else y
    return outs


class MixtureOfRankLinear(nn.Module):
    """y = sum_t term_t(x): several binary low-rank terms with their own scale vectors."""

    def __init__(self, terms: Sequence[NanoQuantLinear]):
        super().__init__()
        if len(terms) == 0:
            raise ValueError("at least one term is required")
        self.terms = nn.ModuleList(terms)
        self.in_features = terms[0].in_features
        self.out_features = terms[0].out_features
        for t in terms:
            if t.in_features != self.in_features or t.out_features != self.out_features:
                raise ValueError("all terms must share in_features and out_features")
        self.kernel_type = None

    def _prepare_kernel(self, kernel_type: str = "gemv", dtype: torch.dtype = torch.float16) -> None:
        for t in self.terms:
            t._prepare_kernel(kernel_type, dtype)
        self.kernel_type = kernel_type
        self.dtype = dtype

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.kernel_type == "gemv":
            orig_dtype = x.dtype
            xk = x.to(self.dtype).contiguous()
            y = ops.gemv_mixture_forward(
                xk, [(t.scale_pre, t.V_int8, t.scale_mid, t.U_int8, t.scale_post) for t in self.terms])
            return y.to(orig_dtype) if y.dtype != orig_dtype else y
        if self.kernel_type == "gemm":            # all terms in shared launches, summed afterwards
            return prefill_group([self], x)[0]
        y = self.terms[0](x)
        for t in self.terms[1:]:
            y = y + t(x)
        return y
