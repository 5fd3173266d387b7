"""Seeded sweep over operator shapes and argument combinations against the oracle: window sizes from 1 to 330
tokens, head dimensions 8 .. 128, several heads / batches / mask window counts, every optional argument on
and off, fp32 or same-dtype masks, a clamped logit scale now and then.  Tolerances as everywhere: bf16 max
abs 2e-2 on o and 5e-2 relative on every gradient, fp16 5e-3 / 2e-2; 5e-2 / 0.15 where a head runs at the
clamp s = 100 (reason at the place)."""
import random

import pytest
import torch

from oracle.classic_torch import classic_fwd_bwd
from tests.test_gpu_parity import TOL, _rel

pytestmark = pytest.mark.gpu


def _case(seed):
    r = random.Random(seed)
    n = r.choice([1, 2, 3, 5, 8, 15, 16, 17, 24, 31, 32, 33, 48, 49, 63, 64, 65, 80, 96, 100, 127, 128, 129, 144,
                  160, 161, 192, 200, 224, 255, 256, 257, 288, 330])
    d = 32 if r.random() < 0.6 else r.choice([8, 16, 24, 40, 64, 96, 128])
    heads = r.choice([1, 2, 3, 5])
    nw = r.choice([1, 1, 2, 3, 4])
    batch = r.choice([1, 2, 3])
    dtype = r.choice([torch.bfloat16, torch.float16])
    return dict(n=n, d=d, heads=heads, nw=nw, batch=batch, dtype=dtype, with_scale=r.random() < 0.7,
                with_bias=r.random() < 0.75, with_mask=r.random() < 0.6, mask_f32=r.random() < 0.4,
                clamp=r.random() < 0.15, seed=seed)


@pytest.mark.parametrize("seed", range(48))
def test_random_shape(seed):
    from flash_window_attention_v2_amd import flash_win_attn_v2_func
    c = _case(seed)
    n, d, heads, nw, dtype = c["n"], c["d"], c["heads"], c["nw"], c["dtype"]
    bw = c["batch"] * nw
    g = torch.Generator().manual_seed(1000 + seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    q, k, v, do = (rnd(bw, heads, n, d).to(dtype) for _ in range(4))
    bias = (16 * torch.sigmoid(rnd(heads, n, n))).to(dtype) if c["with_bias"] else None
    scale = None
    if c["with_scale"]:
        scale = torch.full((heads, 1, 1), 2.3)
        if c["clamp"]:
            scale[0] = 5.0                          # above ln 100: clamped, its gradient is exactly zero
        scale = scale.to(dtype)
    mask = None
    if c["with_mask"]:
        mask = torch.where(torch.rand(nw, n, n, generator=g) < 0.3, -100.0, 0.0)
        mask[0] = 0                                 # one window with nothing masked
        mask[:, torch.arange(n), torch.arange(n)] = 0
        if not c["mask_f32"]:
            mask = mask.to(dtype)
    ref = classic_fwd_bwd(q, k, v, scale, bias, mask, do)

    dev = lambda t: None if t is None else t.cuda().requires_grad_()
    gq, gk, gv, gs, gb = dev(q), dev(k), dev(v), dev(scale), dev(bias)
    o = flash_win_attn_v2_func(gq, gk, gv, gs, gb, None if mask is None else mask.cuda())
    tol_o, tol_g = TOL[dtype]
    if c["clamp"]:
        # s = 100: rounding q^ and k^ to 11 mantissa bits alone moves a logit by up to 100 * 2^-11 = 0.05, the
        # probabilities by 5 %; no low-precision matrix path (the reference's included) does better there
        tol_o, tol_g = 5e-2, 0.15
    assert float((o.detach().float().cpu() - ref["o"]).abs().max()) <= tol_o, c
    if n == 1:
        return          # one key: p = 1, every gradient but dv is pure rounding noise around zero
    o.backward(do.cuda())
    for t, name in ((gq, "dq"), (gk, "dk"), (gv, "dv"), (gb, "dbias")):
        if t is not None:
            assert _rel(t.grad, ref[name]) <= tol_g, (name, c)
    if gs is not None:
        got, want = gs.grad.float().cpu().flatten(), ref["dscale"].float().cpu().flatten()
        if c["clamp"]:
            assert float(got[0]) == 0.0
        bound = torch.maximum(want.abs().max().expand_as(want), 0.1 * ref["dscale_l1"].float().cpu().flatten())
        assert bool(((got - want).abs() <= tol_g * bound).all()), ("dscale", c)
