"""The decode step under torch.compile, as the reference's harness runs it
(src/nanoquant/kernel/test_decode.py:385-402: `torch.compile(mode="reduce-overhead", fullgraph=True, dynamic=False)`,
i.e. Inductor plus graph capture and replay of the whole step).  A small stack of prepared modules is compiled, run
three times (warm-up, capture, replay) with fresh inputs and checked against the oracle every time.  If Inductor cannot
build on this machine the same stack runs under `backend="cudagraphs"` (capture and replay without code generation);
which one ran is printed."""
import numpy as np
import pytest
import torch
import torch._dynamo
import torch._inductor.config as inductor_config

import nanoquant_amd  # noqa: F401
from nanoquant_amd.linear import NanoQuantLinear
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu


class _Stack(torch.nn.Module):
    def __init__(self, mods):
        super().__init__()
        self.mods = torch.nn.ModuleList(mods)

    def forward(self, x):
        for mod in self.mods:
            x = mod(x)
        return x


def _stack(dev, kernel_type, dtype):
    dims = [(512, 256, 96), (768, 512, 128), (256, 768, 160)]          # (out, in, rank), chained
    mods, terms = [], []
    for i, (m, n, r) in enumerate(dims):
        vt, u, s_in, s_mid, s_out = oracle.synth_term(m, n, r, 2000 + i)
        s_out = (s_out.astype(np.float32) * 40.0).astype(np.float16)  # keeps the activations of the chain of order one
        f = lambda a: torch.from_numpy(a.astype(np.float32))
        mod = NanoQuantLinear.from_factors(f(vt), f(u), f(s_in), f(s_mid), f(s_out), dtype=dtype).to(dev)
        mod._prepare_kernel(kernel_type, dtype)
        assert mod.mfma_from_rows == 0                                 # as built: "gemv" is the decode op at 4 rows too
        mods.append(mod)
        terms.append((vt, u, s_in, s_mid, s_out))
    return _Stack(mods).to(dev), terms


def _reference(x, terms, dtype):
    """The chain with every layer's output rounded to the activation type, as the modules hand it on."""
    y = x.astype(np.float64)
    for term in terms:
        y = oracle.layer_forward(y, *term, dtype=np.float64)
        y = torch.from_numpy(y).to(dtype).double().numpy()
    return y


@pytest.mark.parametrize("kernel_type,rows", [("gemv", 1), ("gemv", 4), ("gemm", 128)])
def test_compiled_stack_matches_the_oracle(dev, kernel_type, rows):
    dtype = torch.float16
    stack, terms = _stack(dev, kernel_type, dtype)
    xs = [oracle.synth_x(rows, 256, 2100 + i) for i in range(3)]
    eager = stack(torch.from_numpy(xs[0]).to(dev))
    torch.cuda.synchronize()
    assert oracle.max_rel_err(eager.float().cpu().numpy(), _reference(xs[0], terms, dtype)) < 1e-2

    def run(compiled):
        outs = []
        with torch.no_grad():
            for x in xs:                                               # warm-up, capture, replay
                y = compiled(torch.from_numpy(x).to(dev))
                outs.append(y.clone())                                 # replays reuse the output buffer
                torch.cuda.synchronize()
        return outs

    inductor_config.compile_threads = 1                                # no pool of compile workers beside the GPU process
    torch._dynamo.reset()
    how = "inductor, mode=reduce-overhead"
    print(f"compile {kernel_type} rows={rows}: trying {how}", flush=True)
    try:
        outs = run(torch.compile(stack, mode="reduce-overhead", fullgraph=True, dynamic=False))
    except Exception as exc:                                           # no working code generator on this machine
        print(f"inductor unavailable ({type(exc).__name__}: {str(exc)[:200]}); running backend=cudagraphs", flush=True)
        torch._dynamo.reset()
        how = "backend=cudagraphs"
        outs = run(torch.compile(stack, backend="cudagraphs", fullgraph=True, dynamic=False))
    print(f"compile {kernel_type} rows={rows}: ran under {how}", flush=True)
    for x, y in zip(xs, outs):
        assert y.shape == (rows, 256) and y.dtype == dtype
        err = oracle.max_rel_err(y.float().cpu().numpy(), _reference(x, terms, dtype))
        assert err < 1e-2, (how, err)
    torch._dynamo.reset()
