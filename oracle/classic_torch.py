"""Classic (materialised N x N) window attention in PyTorch.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

A restatement of the reference's classic definition
(flash_win_attn_v2/win_attention_func.py:11-39): L2-normalise q and k,
q_hat k_hat^T, times exp(clamp(logit_scale, max=ln 100)) (or 1/sqrt(d) when no
scale is given), plus the per-head bias, plus the per-window mask (window
index = bw % nW), softmax over keys, times v.  It runs in the dtype of its
inputs; given fp32 inputs on the CPU it is the parity bar for the HIP kernels
and the reported CPU baseline, with gradients from torch.autograd.
"""
import math

import torch
import torch.nn.functional as F


def win_attention_classic(q, k, v, logit_scale=None, bias=None, mask=None):
    bw, heads, n_q, d = q.shape
    n_k = k.shape[2]
    cos = F.normalize(q, dim=-1) @ F.normalize(k, dim=-1).transpose(-1, -2)
    if logit_scale is None:
        scores = cos * (1.0 / math.sqrt(d))
    else:
        scores = cos * torch.exp(torch.clamp(logit_scale, max=math.log(100.0)))
    if bias is not None:
        scores = scores + bias[None]
    if mask is not None:
        n_w = mask.shape[0]
        scores = (scores.reshape(bw // n_w, n_w, heads, n_q, n_k) + mask[None, :, None]).reshape(
            bw, heads, n_q, n_k
        )
    return torch.softmax(scores, dim=-1) @ v


def classic_fwd_bwd(q, k, v, logit_scale, bias, mask, do, dtype=torch.float32):
    """Run the classic path forward + backward in `dtype`, from (possibly low
    precision) inputs that are first upcast/cast to `dtype`.  Returns a dict of
    o, dq, dk, dv, dbias, dscale (the last two None when not applicable)."""
    def leaf(t):
        return None if t is None else t.detach().to(dtype).clone().requires_grad_(True)

    ql, kl, vl, sl, bl = leaf(q), leaf(k), leaf(v), leaf(logit_scale), leaf(bias)
    ml = None if mask is None else mask.detach().to(dtype)
    o = win_attention_classic(ql, kl, vl, sl, bl, ml)
    o.backward(do.detach().to(dtype))
    # Conditioning of dlogit_scale: it is the signed sum over all (bw, i, j) of s dZ_ij c_ij, which
    # can cancel almost completely; dscale_l1[h] is the sum of the absolute terms.  The cosine scores
    # are recovered from the gradient identity d(o.dO)/dC = dZ, i.e. from autograd of the same graph.
    dscale_l1 = None
    if sl is not None:
        with torch.enable_grad():
            qh = F.normalize(ql.detach(), dim=-1)
            kh = F.normalize(kl.detach(), dim=-1)
            cos = (qh @ kh.transpose(-1, -2)).requires_grad_(True)
            s = torch.exp(torch.clamp(sl.detach(), max=math.log(100.0)))
            scores = cos * s
            if bl is not None:
                scores = scores + bl.detach()[None]
            if ml is not None:
                n_w = ml.shape[0]
                bw_, h_, n_q, n_k = scores.shape
                scores = (scores.reshape(bw_ // n_w, n_w, h_, n_q, n_k) + ml[None, :, None]).reshape(bw_, h_, n_q, n_k)
            (torch.softmax(scores, dim=-1) @ vl.detach() * do.detach().to(dtype)).sum().backward()
        dscale_l1 = (cos.grad * cos.detach()).abs().sum(dim=(0, 2, 3))
    return {
        "dscale_l1": dscale_l1,
        "o": o.detach(),
        "dq": ql.grad,
        "dk": kl.grad,
        "dv": vl.grad,
        "dbias": None if bl is None else bl.grad,
        "dscale": None if sl is None else sl.grad,
    }
