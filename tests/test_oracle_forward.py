"""Pins the float64 oracle's forward against independent computations.

The reference holds no golden vectors for this path, so the oracle is pinned
by: scalar brute force, torch's scaled_dot_product_attention as a library
special case, and invariants that a dropped term / wrong index would break.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import window_attention_np as wa
from oracle.classic_torch import win_attention_classic


def _rand(seed, bw=4, nw=2, h=2, n=5, d=3):
    r = np.random.default_rng(seed)
    q, k, v = (r.standard_normal((bw, h, n, d)) for _ in range(3))
    bias = r.standard_normal((h, n, n)) * 2
    mask = np.where(r.random((nw, n, n)) < 0.3, -100.0, 0.0)
    ls = r.standard_normal((h, 1, 1)) + 1.0
    return q, k, v, ls, bias, mask


@pytest.mark.parametrize("use_scale,use_bias,use_mask", [(1, 1, 1), (0, 1, 1), (1, 0, 1), (1, 1, 0), (0, 0, 0)])
def test_forward_matches_bruteforce(use_scale, use_bias, use_mask):
    q, k, v, ls, bias, mask = _rand(1)
    args = (ls if use_scale else None, bias if use_bias else None, mask if use_mask else None)
    o, _ = wa.forward(q, k, v, *args)
    ob = wa.forward_bruteforce(q, k, v, *args)
    np.testing.assert_allclose(o, ob, rtol=1e-12, atol=1e-12)


def test_forward_matches_sdpa_special_case():
    q, k, v, ls, bias, mask = _rand(2, bw=6, nw=3, h=2, n=7, d=4)
    o, _ = wa.forward(q, k, v, ls, bias, mask)
    tq, tk, tv = (torch.from_numpy(x) for x in (q, k, v))
    s = torch.exp(torch.clamp(torch.from_numpy(ls), max=math.log(100.0)))
    add = torch.from_numpy(bias)[None] + torch.from_numpy(mask)[torch.arange(6) % 3][:, None]
    ref = F.scaled_dot_product_attention(F.normalize(tq, dim=-1) * s, F.normalize(tk, dim=-1), tv,
                                         attn_mask=add, scale=1.0)
    np.testing.assert_allclose(o, ref.numpy(), rtol=1e-10, atol=1e-12)


def test_no_scale_is_sdpa_with_inv_sqrt_d():
    q, k, v, *_ = _rand(3, n=6, d=8)
    o, _ = wa.forward(q, k, v)
    tq, tk, tv = (torch.from_numpy(x) for x in (q, k, v))
    ref = F.scaled_dot_product_attention(F.normalize(tq, dim=-1), F.normalize(tk, dim=-1), tv)
    np.testing.assert_allclose(o, ref.numpy(), rtol=1e-10, atol=1e-12)


def test_classic_torch_agrees_with_numpy():
    q, k, v, ls, bias, mask = _rand(4, bw=6, nw=3, n=9, d=5)
    o, _ = wa.forward(q, k, v, ls, bias, mask)
    t = win_attention_classic(*(torch.from_numpy(x) for x in (q, k, v, ls, bias, mask)))
    np.testing.assert_allclose(o, t.numpy(), rtol=1e-10, atol=1e-12)


def test_invariants():
    q, k, v, ls, bias, mask = _rand(5)
    o, lse = wa.forward(q, k, v, ls, bias, mask)
    r = np.random.default_rng(0)
    # positive per-row rescaling of q or k changes nothing (cosine attention)
    o2, _ = wa.forward(q * r.uniform(0.5, 3, q.shape[:-1] + (1,)), k * r.uniform(0.5, 3, k.shape[:-1] + (1,)),
                       v, ls, bias, mask)
    np.testing.assert_allclose(o, o2, rtol=1e-10, atol=1e-12)
    # a per-row constant added to the bias cancels in the softmax, shifts lse
    shift = r.standard_normal((bias.shape[0], bias.shape[1], 1))
    o3, lse3 = wa.forward(q, k, v, ls, bias + shift, mask)
    np.testing.assert_allclose(o, o3, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(lse3, lse + shift[None, :, :, 0], rtol=1e-10, atol=1e-12)
    # an all-zero mask is no mask
    o4, _ = wa.forward(q, k, v, ls, bias, np.zeros_like(mask))
    o5, _ = wa.forward(q, k, v, ls, bias, None)
    np.testing.assert_array_equal(o4, o5)
    # the logit scale saturates at ln 100
    big = np.full_like(ls, 7.0)
    o6, _ = wa.forward(q, k, v, big, bias, mask)
    o7, _ = wa.forward(q, k, v, np.full_like(ls, math.log(100.0)), bias, mask)
    np.testing.assert_allclose(o6, o7, rtol=1e-12, atol=1e-12)
    # uniform scores (k rows identical, no bias/mask) average v; lse = s + log N
    kk = np.broadcast_to(k[:, :, :1], k.shape)
    o8, lse8 = wa.forward(q, kk, v, ls)
    np.testing.assert_allclose(o8, np.broadcast_to(v.mean(axis=2, keepdims=True), v.shape), rtol=1e-10, atol=1e-12)
    z, c, s = wa.logits(q, kk, ls)
    np.testing.assert_allclose(lse8, z[..., 0] + math.log(q.shape[2]), rtol=1e-10)


def test_mask_window_index_is_bw_mod_nw():
    # a mask that kills every key but one, different per window, reads back v rows
    bw, nw, h, n, d = 6, 3, 1, 4, 2
    r = np.random.default_rng(7)
    q, k, v = (r.standard_normal((bw, h, n, d)) for _ in range(3))
    mask = np.full((nw, n, n), -np.inf)
    for w in range(nw):
        mask[w, :, w] = 0.0
    o, lse = wa.forward(q, k, v, None, None, mask)
    for b in range(bw):
        np.testing.assert_allclose(o[b, 0], np.broadcast_to(v[b, 0, b % nw], (n, d)), rtol=1e-12)


def test_fully_masked_row_gives_zero():
    q, k, v, ls, bias, _ = _rand(8)
    mask = np.zeros((2, 5, 5))
    mask[1, 2, :] = -np.inf
    o, lse = wa.forward(q, k, v, ls, bias, mask)
    assert np.all(o[1::2, :, 2] == 0) and np.all(np.isneginf(lse[1::2, :, 2]))
    assert np.all(np.isfinite(o))
