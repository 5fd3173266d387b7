"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU: the numpy oracle reproduces them, and an independent route -- float64 autograd through the
classic torch restatement, which shares no backward code with the numpy oracle -- lands on the same
numbers.  GPU: the kernels, through the C ABI, meet the stated tolerances against them.
"""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import window_attention_np as wnp
from oracle.classic_torch import classic_fwd_bwd

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(GOLDEN, "*.npz")))
OUTPUTS = ("o", "dq", "dk", "dv", "dbias", "dscale")


def _load(case):
    with np.load(os.path.join(GOLDEN, case + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def test_fixtures_present():
    assert CASES == ["bf16_n16_shift_mask", "f16_n49_no_mask"]


@pytest.mark.parametrize("case", CASES)
def test_numpy_oracle_reproduces_fixture(case):
    fx = _load(case)
    side = [fx.get("in_" + k) for k in ("logit_scale", "bias", "mask")]
    o, lse = wnp.forward(fx["in_q"], fx["in_k"], fx["in_v"], *side)
    got = wnp.backward(fx["in_q"], fx["in_k"], fx["in_v"], fx["in_do"], *side)
    got["o"], got["lse"] = o, lse
    for name in OUTPUTS + ("lse",):
        if name in fx:
            np.testing.assert_allclose(got[name], fx[name], rtol=2e-6, atol=2e-6, err_msg=name)
        else:
            assert got[name] is None


@pytest.mark.parametrize("case", CASES)
def test_autograd_route_agrees_with_fixture(case):
    fx = _load(case)
    t = {k[3:]: torch.from_numpy(v) for k, v in fx.items() if k.startswith("in_")}
    got = classic_fwd_bwd(t["q"], t["k"], t["v"], t.get("logit_scale"), t.get("bias"), t.get("mask"), t["do"],
                          dtype=torch.float64)
    for name in OUTPUTS:
        if name in fx:
            np.testing.assert_allclose(got[name].numpy(), fx[name], rtol=1e-5, atol=1e-5, err_msg=name)
    if case.startswith("bf16"):
        assert fx["dscale"][1, 0, 0] == 0.0 and fx["dscale"][0, 0, 0] != 0.0     # head 1 sits past the clamp


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_kernels_against_fixture(case):
    from flash_window_attention_v2_amd import flash_win_attn_v2_func

    fx = _load(case)
    dtype, tol_o, tol_g = (torch.bfloat16, 2e-2, 5e-2) if case.startswith("bf16") else (torch.float16, 5e-3, 2e-2)
    t = {k[3:]: torch.from_numpy(v).to(dtype).cuda() for k, v in fx.items() if k.startswith("in_")}
    for k in t:
        assert torch.equal(t[k].float().cpu(), torch.from_numpy(fx["in_" + k])), "fixture inputs must be exact"
    for name in ("q", "k", "v", "bias", "logit_scale"):
        if name in t:
            t[name].requires_grad_(True)
    o = flash_win_attn_v2_func(t["q"], t["k"], t["v"], t.get("logit_scale"), t.get("bias"), t.get("mask"))
    o.backward(t["do"])
    # A head past the clamp runs at s = 100, where rounding q_hat.k_hat moves the logits by up to
    # 100 * 2^-9 in bf16: such a head is held to what the eager classic path reaches in the same dtype on the
    # same inputs, the others to the stated tolerances.  The clamped head's logit-scale gradient must be exactly zero.
    heads = t["q"].shape[1]
    clamped = [bool(t["logit_scale"][h] > 4.6051) for h in range(heads)] if "logit_scale" in t else [False] * heads
    cpu = {k: v.detach().cpu() for k, v in t.items()}
    eager = classic_fwd_bwd(cpu["q"], cpu["k"], cpu["v"], cpu.get("logit_scale"), cpu.get("bias"), cpu.get("mask"), cpu["do"],
                            dtype=dtype)
    o_ref = torch.from_numpy(fx["o"])
    o_err = (o.detach().float().cpu() - o_ref).abs()
    eager_err = (eager["o"].float() - o_ref).abs()
    for h in range(heads):
        assert float(o_err[:, h].max()) <= (float(eager_err[:, h].max()) if clamped[h] else tol_o), f"o head {h}"
    for gname, tname in (("dq", "q"), ("dk", "k"), ("dv", "v"), ("dbias", "bias"), ("dscale", "logit_scale")):
        if gname not in fx:
            continue
        ref = torch.from_numpy(fx[gname])
        got = t[tname].grad.float().cpu()
        axis = 0 if gname in ("dbias", "dscale") else 1
        for h in range(heads):
            r, g = ref.select(axis, h), got.select(axis, h)
            if gname == "dscale" and clamped[h]:
                assert float(g.abs().max()) == 0.0 and float(r.abs().max()) == 0.0
                continue
            rel = float((g - r).abs().max() / r.abs().max())
            bound = tol_g
            if clamped[h]:
                bound = float((eager[gname].float().select(axis, h) - r).abs().max() / r.abs().max())
            assert rel <= bound, f"{gname} head {h}: {rel} (bound {bound})"
