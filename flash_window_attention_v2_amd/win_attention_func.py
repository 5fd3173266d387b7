"""Operator entry points, named as in the reference
(flash_win_attn_v2/win_attention_func.py): the fused gfx950 path and the
classic materialised path that `WindowAttention(is_flash=False)` uses."""
import math

import torch
import torch.nn.functional as F

from .flash_window_attention_v2 import (FlashWindowAttentionV2, FlashWindowAttentionV2Grid,
                                         FlashWindowAttentionV2QKVPacked)

#: fused forward/backward: (q, k, v, logit_scale=None, bias=None, mask=None) -> o
flash_win_attn_v2_func = FlashWindowAttentionV2.apply
#: the same fed from the packed projection: (qkv [BW, N, 3, H, d], logit_scale=None, bias=None, mask=None)
#: -> o [BW, N, H, d]; the gradient comes back as one packed tensor
flash_win_attn_v2_qkvpacked_func = FlashWindowAttentionV2QKVPacked.apply
#: the packed operator on the un-partitioned token grid, with the cyclic shift and the window partition /
#: reverse done by the kernels: (qkv [B, gh*gw, 3, H, d], (gh, gw), (wh, ww), (shift_h, shift_w),
#: logit_scale=None, bias=None, mask=None) -> o [B, gh*gw, H, d]
flash_win_attn_v2_grid_func = FlashWindowAttentionV2Grid.apply


def win_attention_torch(q, k, v, logit_scale=None, bias=None, mask=None):
    """Classic window attention with explicit [BW, H, N, N] scores, in the dtype of
    its inputs (the operator selected by `is_flash=False`; it is a different,
    slower operator chosen by the caller, never a substitute for the fused one).

    q, k, v: [BW, H, N, d]; logit_scale: [H, 1, 1] or None; bias: [H, N, N] or
    None; mask: [nW, N, N] or None with window index bw % nW.
    """
    bw, heads, n_q, d = q.shape
    n_k = k.shape[2]
    scores = F.normalize(q, p=2, dim=-1) @ F.normalize(k, p=2, dim=-1).transpose(-2, -1)
    if logit_scale is None:
        scores = scores * (1.0 / math.sqrt(d))
    else:
        limit = torch.log(torch.tensor(100.0, dtype=logit_scale.dtype, device=logit_scale.device))
        scores = scores * logit_scale.clamp(max=limit).exp()
    if bias is not None:
        scores = scores + bias.unsqueeze(0)
    if mask is not None:
        n_w = mask.shape[0]
        scores = scores.view(bw // n_w, n_w, heads, n_q, n_k) + mask.unsqueeze(1).unsqueeze(0)
        scores = scores.view(bw, heads, n_q, n_k)
    return torch.softmax(scores, dim=-1) @ v


_compiled_classic = None


def win_attention_torch_compile(q, k, v, logit_scale=None, bias=None, mask=None):
    """`win_attention_torch` under `torch.compile`, the third operator the reference
    exports (flash_win_attn_v2/win_attention_func.py:42) as a comparison line for its
    benchmarks.  Compiled on first use; nothing in the fused path depends on it."""
    global _compiled_classic
    if _compiled_classic is None:
        _compiled_classic = torch.compile(win_attention_torch)
    return _compiled_classic(q, k, v, logit_scale, bias, mask)
