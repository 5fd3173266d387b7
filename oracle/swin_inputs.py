"""Closed-form Swin V2 side inputs and seeded tensors for the benchmark configs.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

shifted_window_mask   closed form of the buffer SwinTransformerBlock builds by
                      painting nine slices of a label image and partitioning it
                      (flash_win_attn_v2/swin_transformer_v2.py:386-405).
relative_position_index / relative_coords_table
                      closed forms of the WindowAttention buffers
                      (swin_transformer_v2.py:223-254).
make_inputs           seeded q, k, v, bias, logit_scale, mask, dO of one
                      operator call, generated in fp32 on the CPU and rounded to
                      the requested dtype so that every consumer sees identical
                      values.
"""
import math

import numpy as np
import torch


def shifted_window_mask(resolution, window, shift, dtype=torch.float32):
    """[nW, N, N] mask of 0 / -100 for a square token grid.

    Region label of token (r, c) of the rolled grid is 3*band(r) + band(c),
    band(x) = 0 for x < R - window, 1 for x < R - shift, else 2; an entry is
    -100 where the two tokens of a window carry different labels.  Windows
    are numbered row-major, tokens inside a window row-major
    (swin_transformer_v2.py:156-168).
    """
    R, ws = resolution, window
    assert R % ws == 0 and 0 < shift < ws
    x = np.arange(R)
    band = (x >= R - ws).astype(np.int64) + (x >= R - shift).astype(np.int64)
    label = 3 * band[:, None] + band[None, :]                       # [R, R]
    g = R // ws
    lab = label.reshape(g, ws, g, ws).transpose(0, 2, 1, 3).reshape(g * g, ws * ws)
    differ = lab[:, :, None] != lab[:, None, :]
    return torch.from_numpy(np.where(differ, -100.0, 0.0)).to(dtype)


def relative_position_index(wh, ww):
    """[N, N] integer index into the (2Wh-1)(2Ww-1) bias table:
    (r_i - r_j + Wh - 1)(2Ww - 1) + (c_i - c_j + Ww - 1)."""
    r = np.repeat(np.arange(wh), ww)
    c = np.tile(np.arange(ww), wh)
    idx = (r[:, None] - r[None, :] + wh - 1) * (2 * ww - 1) + (c[:, None] - c[None, :] + ww - 1)
    return torch.from_numpy(idx.astype(np.int64))


def relative_coords_table(wh, ww, pretrained=(0, 0)):
    """[1, 2Wh-1, 2Ww-1, 2] table sign(x) log2(|8x/(W-1)| + 1) / 3."""
    dh = np.arange(-(wh - 1), wh, dtype=np.float64)
    dw = np.arange(-(ww - 1), ww, dtype=np.float64)
    nh = (pretrained[0] if pretrained[0] > 0 else wh) - 1
    nw = (pretrained[1] if pretrained[1] > 0 else ww) - 1
    t = np.stack(np.meshgrid(dh / nh * 8.0, dw / nw * 8.0, indexing="ij"), axis=-1)
    t = np.sign(t) * np.log2(np.abs(t) + 1.0) / 3.0
    return torch.from_numpy(t[None]).to(torch.float32)


# (batch, windows per image, heads, tokens per window, head dim, token grid side, window, shift)
CONFIGS = {
    "C1": dict(batch=2, n_windows=16, heads=4, n=64, d=32, resolution=32, window=8, shift=4),
    "C2": dict(batch=64, n_windows=64, heads=3, n=64, d=32, resolution=64, window=8, shift=4),
    "C3": dict(batch=64, n_windows=64, heads=3, n=256, d=32, resolution=128, window=16, shift=8),
}


def make_inputs(batch, n_windows, heads, n, d=32, dtype=torch.float32, seed=0,
                resolution=None, window=None, shift=None, with_mask=True,
                with_bias=True, with_scale=True, **_):
    """Seeded operator inputs (CPU tensors already rounded to `dtype`).

    q, k, v, dO ~ N(0,1); bias = 16 sigmoid(N(0,1)); logit_scale = ln 10;
    mask = shifted-window 0/-100 when a grid is given, else None.
    """
    g = torch.Generator().manual_seed(seed)
    bw = batch * n_windows
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    out = {
        "q": rnd(bw, heads, n, d).to(dtype),
        "k": rnd(bw, heads, n, d).to(dtype),
        "v": rnd(bw, heads, n, d).to(dtype),
        "do": rnd(bw, heads, n, d).to(dtype),
        "bias": (16.0 * torch.sigmoid(rnd(heads, n, n))).to(dtype) if with_bias else None,
        "logit_scale": torch.full((heads, 1, 1), math.log(10.0)).to(dtype) if with_scale else None,
        "mask": None,
    }
    if with_mask and resolution is not None:
        m = shifted_window_mask(resolution, window, shift)
        assert m.shape == (n_windows, n, n)
        out["mask"] = m.to(dtype)
    return out
