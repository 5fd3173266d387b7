"""Float64 numpy oracle for scaled-cosine window attention (forward + backward).

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Semantics follow the reference's classic definition
(flash_win_attn_v2/win_attention_func.py:11-39) for the forward, and the
gradient formulas spelled out by its backward kernel
(flash_win_attn_v2/kernels/attn_kernel_backward.py:246-269, 336, 703-711)
for the backward.  Everything is computed in float64 whatever the input
dtype, so rounding inside the oracle is negligible against bf16/fp16 kernels.

Shapes: q, k, v [BW, H, N, d]; logit_scale [H, 1, 1] or None; bias [H, N, N]
or None; mask [nW, N, N] or None, with window index bw % nW
(win_attention_func.py:33-36 views the scores as [B, nW, H, N, N]).
"""
import math

import numpy as np

LN_100 = math.log(100.0)
NORM_EPS = 1e-12  # torch.nn.functional.normalize default, win_attention_func.py:22-23


def _f64(x):
    return None if x is None else np.asarray(x, dtype=np.float64)


def head_scale(logit_scale, n_heads, head_dim):
    """Per-head multiplier of the cosine scores.

    exp(min(l_h, ln 100)) when a logit scale is given
    (win_attention_func.py:25-26), 1/sqrt(d) otherwise (:27-28).
    """
    if logit_scale is None:
        return np.full((n_heads,), 1.0 / math.sqrt(head_dim))
    ls = _f64(logit_scale).reshape(n_heads)
    return np.exp(np.minimum(ls, LN_100))


def l2_normalise(x):
    """x / max(||x||_2, eps) along the last axis; returns (x_hat, denom)."""
    nrm = np.sqrt(np.sum(x * x, axis=-1, keepdims=True))
    den = np.maximum(nrm, NORM_EPS)
    return x / den, den, nrm


def logits(q, k, logit_scale=None, bias=None, mask=None):
    """Pre-softmax scores z [BW,H,N,N] and the unscaled cosine c."""
    q, k = _f64(q), _f64(k)
    bw, h, n, d = q.shape
    qh, _, _ = l2_normalise(q)
    kh, _, _ = l2_normalise(k)
    c = np.einsum("bhid,bhjd->bhij", qh, kh)
    s = head_scale(logit_scale, h, d)
    z = c * s[None, :, None, None]
    if bias is not None:
        z = z + _f64(bias)[None]
    if mask is not None:
        m = _f64(mask)
        nw = m.shape[0]
        assert bw % nw == 0, "BW must be a multiple of the number of windows"
        z = z + m[np.arange(bw) % nw][:, None]
    return z, c, s


def forward(q, k, v, logit_scale=None, bias=None, mask=None):
    """Returns (o [BW,H,N,d], lse [BW,H,N]) in float64.

    A row whose scores are all -inf yields o = 0 and lse = -inf (the flash
    kernel's convention, attn_kernel_forward.py:233); the classic softmax
    would give NaN there.
    """
    z, _, _ = logits(q, k, logit_scale, bias, mask)
    v = _f64(v)
    zmax = np.max(z, axis=-1, keepdims=True)
    zmax_safe = np.where(np.isfinite(zmax), zmax, 0.0)
    e = np.exp(z - zmax_safe)
    l = np.sum(e, axis=-1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        p = np.where(l > 0, e / np.where(l > 0, l, 1.0), 0.0)
        lse = np.where(l > 0, zmax_safe + np.log(np.where(l > 0, l, 1.0)), -np.inf)
    o = np.einsum("bhij,bhjd->bhid", p, v)
    return o, lse[..., 0]


def backward(q, k, v, do, logit_scale=None, bias=None, mask=None):
    """Hand-derived gradients; returns dict(dq, dk, dv, dbias, dscale).

    dbias is None without a bias, dscale is None without a tensor scale.
    Formulas (attn_kernel_backward.py line numbers):
      delta_i = sum_d O_id dO_id                               (:45)
      P       = exp(z - lse)                                   (:246-247)
      dV      = P^T dO                                         (:250)
      dP      = dO V^T                                         (:253)
      dZ      = P * (dP - delta)   (= per-unit bias gradient)  (:256-257)
      dC      = s_h dZ                                         (:258)
      dscale  = [l_h <= ln100] * sum dC * c                    (:261-262, :706-711)
      dq_hat  = dC k_hat ; dk_hat = dC^T q_hat                 (:265, :268)
      dx      = dx_hat/n - x (dx_hat . x_hat)/n^2              (:269, :336)
    The last line is written for the classic eps convention
    (x / max(||x||, eps)): rows with ||x|| <= eps get dx = dx_hat / eps.
    """
    q, k, v, do = _f64(q), _f64(k), _f64(v), _f64(do)
    bw, h, n, d = q.shape
    z, c, s = logits(q, k, logit_scale, bias, mask)
    o, lse = forward(q, k, v, logit_scale, bias, mask)
    lse_safe = np.where(np.isfinite(lse), lse, np.inf)
    with np.errstate(invalid="ignore"):
        p = np.exp(z - lse_safe[..., None])
    p = np.where(np.isnan(p), 0.0, p)
    delta = np.sum(o * do, axis=-1, keepdims=True)
    dv = np.einsum("bhij,bhid->bhjd", p, do)
    dp = np.einsum("bhid,bhjd->bhij", do, v)
    dz = p * (dp - delta)
    dc = dz * s[None, :, None, None]

    qh, qden, qn = l2_normalise(q)
    kh, kden, kn = l2_normalise(k)
    dqh = np.einsum("bhij,bhjd->bhid", dc, kh)
    dkh = np.einsum("bhij,bhid->bhjd", dc, qh)

    def through_norm(dxh, xh, den, nrm):
        live = nrm > NORM_EPS
        proj = np.sum(dxh * xh, axis=-1, keepdims=True)
        return np.where(live, (dxh - xh * proj) / den, dxh / den)

    out = {
        "dq": through_norm(dqh, qh, qden, qn),
        "dk": through_norm(dkh, kh, kden, kn),
        "dv": dv,
        "dbias": None,
        "dscale": None,
    }
    if bias is not None:
        out["dbias"] = dz.sum(axis=0)
    if logit_scale is not None:
        ls = _f64(logit_scale).reshape(h)
        gate = (ls <= LN_100).astype(np.float64)
        out["dscale"] = (gate * np.einsum("bhij,bhij->h", dc, c)).reshape(h, 1, 1)
    return out


def forward_bruteforce(q, k, v, logit_scale=None, bias=None, mask=None):
    """Scalar-loop forward for tiny shapes: an independent check of forward()."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    bw, h, n, d = q.shape
    nk = k.shape[2]
    o = np.zeros((bw, h, n, d))
    for b in range(bw):
        for hh in range(h):
            if logit_scale is None:
                s = 1.0 / math.sqrt(d)
            else:
                s = math.exp(min(float(np.asarray(logit_scale, dtype=np.float64).reshape(-1)[hh]), LN_100))
            for i in range(n):
                qi = q[b, hh, i]
                qn = max(math.sqrt(sum(x * x for x in qi)), NORM_EPS)
                row = []
                for j in range(nk):
                    kj = k[b, hh, j]
                    kn = max(math.sqrt(sum(x * x for x in kj)), NORM_EPS)
                    zij = s * sum((a / qn) * (c_ / kn) for a, c_ in zip(qi, kj))
                    if bias is not None:
                        zij += float(bias[hh][i][j])
                    if mask is not None:
                        zij += float(mask[b % len(mask)][i][j])
                    row.append(zij)
                top = max(row)
                w = [math.exp(x - top) for x in row]
                tot = sum(w)
                for dd in range(d):
                    o[b, hh, i, dd] = sum(w[j] * v[b, hh, j, dd] for j in range(nk)) / tot
    return o
