"""The launches that bench.py times, checked against the oracle: the 32-layer Llama-2-7B-shaped stack (224 linears in
tile order, ranks 2048 and 2985 padded to 3008 with a zero mid scale, random words generated on the device) as ONE
run-list launch at batch 1, 4 and 16, every linear with an output buffer of its own.  For the first, a middle and the
last layer a seeded sample of 256 output rows of every linear is compared with the dense definition
(src/nanoquant/modules/linear.py:248-257 of the reference) evaluated by the oracle on the same packed words.  The
kernel instance that serves such a list (wavefronts owning row pairs, bit 5 of the plan) is selected by list length,
so only a list of this length exercises it."""
import numpy as np
import pytest
import torch

import nanoquant_amd  # noqa: F401
from nanoquant_amd import DecodeRunList, packing
from oracle import nq_oracle as oracle

pytestmark = pytest.mark.gpu

LLAMA2_7B_LAYER = (("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
                   ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008))
LAYERS = 32


def _stack(dev, batch, dtype=torch.float16):
    gen = torch.Generator(device=dev)
    gen.manual_seed(321)
    i32 = torch.iinfo(torch.int32)
    sc = lambda k: (torch.randn(k, device=dev, generator=gen).abs() * 0.02 + 1e-3).to(dtype)
    xs = {n: torch.randn(batch, n, device=dev, generator=gen).to(dtype) for n in (4096, 11008)}
    rl = DecodeRunList(batch, dtype, dev)
    sampled = {}
    for layer in range(LAYERS):
        for name, m, n in LLAMA2_7B_LAYER:
            r = oracle.nominal_rank(m, n)
            rp = (r + 31) // 32 * 32
            vt = torch.randint(i32.min, i32.max, (rp, n // 32), dtype=torch.int32, device=dev, generator=gen)
            u = torch.randint(i32.min, i32.max, (m, rp // 32), dtype=torch.int32, device=dev, generator=gen)
            s_in, s_mid, s_out = sc(n), sc(rp), sc(m)
            s_mid[r:] = 0
            idx = rl.add(xs[n], s_in, packing.tile_words(vt), s_mid, packing.tile_words(u), s_out, tiled=True)
            if layer in (0, LAYERS // 2, LAYERS - 1):
                sampled[idx] = (name, layer, xs[n], s_in, vt, s_mid, u, s_out)
    rl.build()
    return rl, sampled


def _reference(x, s_in, vt, s_mid, u, s_out, rows):
    c = lambda t: t.cpu().numpy()
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    return oracle.layer_forward_packed(f64(x), f64(s_in), c(vt), f64(s_mid), c(u)[rows], f64(s_out)[rows], dtype=np.float64)


@pytest.mark.parametrize("batch", [1, 4, 16])
def test_benchmarked_stack_against_the_oracle(dev, batch):
    rl, sampled = _stack(dev, batch)
    bound = int(rl._plan.bound)
    assert bound & 4                                   # tile order
    if batch in (1, 4):
        assert bound & 32, bound                       # wavefronts own row pairs: the instance behind the headline
    outs = rl.outputs
    assert len({o.data_ptr() for o in outs}) == len(outs) == 7 * LAYERS      # no two linears share an output
    print(f"benchmarked stack, batch {batch}, plan.bound {bound}", flush=True)
    for rep in range(2):                               # the second launch reuses the counters of the first
        for o in outs:
            o.zero_()
        ys = rl.run()
        torch.cuda.synchronize()
        assert rl.status() == 0
        worst = (0.0, 0.0)
        for idx, (name, layer, x, s_in, vt, s_mid, u, s_out) in sampled.items():
            rows = np.random.default_rng(1000 * layer + idx).choice(u.shape[0], size=256, replace=False)
            ref = _reference(x, s_in, vt, s_mid, u, s_out, rows)
            got = ys[idx].float().cpu().numpy()[:, rows]
            e, ee = oracle.max_rel_err(got, ref), oracle.elementwise_err(got, ref)
            worst = (max(worst[0], e), max(worst[1], ee))
            assert e < 1e-3, (name, layer, batch, rep, e)
            # fp16 outputs cost 2^-11 of the element; the 16-bit arithmetic of batch 16 also rounds x * s_in and the
            # intermediate vector to fp16, as the reference's kernels do
            assert ee < (5e-3 if batch <= 4 else 5e-2), (name, layer, batch, rep, ee)
        if rep == 0:
            print(f"  worst of 21 linears: max_rel_err {worst[0]:.2e}, element-wise (floor 0.1 rms) {worst[1]:.2e}", flush=True)
