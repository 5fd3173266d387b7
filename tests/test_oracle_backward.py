"""Pins the oracle's hand-derived backward: autograd of the classic path in
float64, finite differences, and structural invariants of the gradients."""
import math

import numpy as np
import pytest
import torch

from oracle import window_attention_np as wa
from oracle.classic_torch import classic_fwd_bwd, win_attention_classic


def _rand(seed, bw=4, nw=2, h=2, n=6, d=4, scale_mean=1.0):
    r = np.random.default_rng(seed)
    q, k, v, do = (r.standard_normal((bw, h, n, d)) for _ in range(4))
    bias = r.standard_normal((h, n, n)) * 2
    mask = np.where(r.random((nw, n, n)) < 0.3, -100.0, 0.0)
    ls = r.standard_normal((h, 1, 1)) * 0.3 + scale_mean
    return q, k, v, do, ls, bias, mask


@pytest.mark.parametrize("use_scale,use_bias,use_mask", [(1, 1, 1), (0, 1, 1), (1, 0, 0), (0, 0, 1)])
def test_backward_matches_autograd(use_scale, use_bias, use_mask):
    q, k, v, do, ls, bias, mask = _rand(11)
    ls_, bias_, mask_ = (ls if use_scale else None, bias if use_bias else None, mask if use_mask else None)
    g = wa.backward(q, k, v, do, ls_, bias_, mask_)
    T = lambda x: None if x is None else torch.from_numpy(x)
    ref = classic_fwd_bwd(T(q), T(k), T(v), T(ls_), T(bias_), T(mask_), T(do), dtype=torch.float64)
    for name in ("dq", "dk", "dv", "dbias", "dscale"):
        if ref[name] is None:
            assert g[name] is None
        else:
            np.testing.assert_allclose(g[name], ref[name].numpy(), rtol=1e-9, atol=1e-11, err_msg=name)


def test_backward_finite_differences():
    q, k, v, do, ls, bias, mask = _rand(12, bw=2, nw=2, h=1, n=4, d=3)
    g = wa.backward(q, k, v, do, ls, bias, mask)
    loss = lambda **kw: float(np.sum(wa.forward(kw.get("q", q), kw.get("k", k), kw.get("v", v), kw.get("ls", ls),
                                                kw.get("bias", bias), mask)[0] * do))
    eps = 1e-6
    for name, arr, grad in (("q", q, g["dq"]), ("k", k, g["dk"]), ("v", v, g["dv"]), ("bias", bias, g["dbias"]),
                            ("ls", ls, g["dscale"])):
        idx = tuple(np.random.default_rng(3).integers(0, s) for s in arr.shape)
        hi, lo = arr.copy(), arr.copy()
        hi[idx] += eps
        lo[idx] -= eps
        fd = (loss(**{name: hi}) - loss(**{name: lo})) / (2 * eps)
        assert abs(fd - grad[idx]) < 1e-6 * max(1.0, abs(fd)), name


def test_gradient_invariants():
    q, k, v, do, ls, bias, mask = _rand(13)
    g = wa.backward(q, k, v, do, ls, bias, mask)
    # cosine attention: gradient is orthogonal to the vector it normalises
    assert np.max(np.abs(np.sum(g["dq"] * q, axis=-1))) < 1e-12
    assert np.max(np.abs(np.sum(g["dk"] * k, axis=-1))) < 1e-12
    # softmax: every row of dbias sums to zero
    assert np.max(np.abs(g["dbias"].sum(axis=-1))) < 1e-12
    # dV with dO = 1 sums attention columns: total equals number of rows
    g1 = wa.backward(q, k, v, np.ones_like(do), ls, bias, mask)
    np.testing.assert_allclose(g1["dv"].sum(axis=2), np.full(q.shape[:2] + (q.shape[-1],), q.shape[2]), rtol=1e-10)


def test_scale_gate():
    q, k, v, do, ls, bias, mask = _rand(14)
    ls = ls.copy()
    ls[0] = 5.0                      # above ln 100: clamp blocks the gradient
    ls[1] = math.log(100.0)          # at the boundary the gradient passes (<=)
    g = wa.backward(q, k, v, do, ls, bias, mask)
    assert g["dscale"][0, 0, 0] == 0.0 and g["dscale"][1, 0, 0] != 0.0
    ref = classic_fwd_bwd(*(torch.from_numpy(x) for x in (q, k, v, ls, bias, mask, do)), dtype=torch.float64)
    np.testing.assert_allclose(g["dscale"][0], ref["dscale"].numpy()[0], atol=1e-12)
    # without a tensor scale there is no scale gradient and no bias gradient without bias
    g2 = wa.backward(q, k, v, do, None, None, mask)
    assert g2["dscale"] is None and g2["dbias"] is None


def test_dscale_l1_is_the_sum_of_absolute_terms():
    """`dscale_l1`, the yardstick the GPU tests hold the logit-scale gradient against, recomputed from first
    principles with numpy: P from the logits, dZ = P (dP - delta), then sum |dZ c| per head.  The signed sum
    of the same terms times s must give back dscale itself (for heads below the clamp), which ties the
    yardstick to the gradient it measures."""
    q, k, v, do, ls, bias, mask = _rand(15, bw=4, nw=2, h=3, n=7, d=4)
    ls = ls.copy()
    ls[2] = 5.0                                                   # one clamped head: s = 100, dscale = 0
    ref = classic_fwd_bwd(*(torch.from_numpy(x) for x in (q, k, v, ls, bias, mask, do)), dtype=torch.float64)
    z, c, s = wa.logits(q, k, ls, bias, mask)
    p = np.exp(z - z.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    dp = np.einsum("bhid,bhjd->bhij", do, v)
    delta = np.einsum("bhij,bhij->bhi", p, dp)[..., None]
    dz = p * (dp - delta)
    s = np.asarray(s).reshape(-1)
    np.testing.assert_allclose(s, [math.exp(ls[0, 0, 0]), math.exp(ls[1, 0, 0]), 100.0], rtol=1e-12)
    # the helper differentiates with respect to the cosine scores, so each term carries the factor s once
    l1 = np.abs(dz * c).sum(axis=(0, 2, 3)) * s
    np.testing.assert_allclose(ref["dscale_l1"].numpy(), l1, rtol=1e-9)
    signed = (dz * c).sum(axis=(0, 2, 3)) * s
    np.testing.assert_allclose(ref["dscale"].numpy().reshape(-1)[:2], signed[:2], rtol=1e-9)
    assert float(ref["dscale"].reshape(-1)[2]) == 0.0 and np.all(l1 >= np.abs(signed) - 1e-12)
