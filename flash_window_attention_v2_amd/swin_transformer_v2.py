"""Swin Transformer V2 around the fused window-attention operator.

The caller side of the hot path: `WindowAttention` keeps the reference's
constructor and forward signature (flash_win_attn_v2/swin_transformer_v2.py:203-204,
268) and hands the operator the same things the reference does -- strided
q/k/v views of one qkv GEMM output, a [H, N, N] bias from the
continuous-position MLP, the [H, 1, 1] logit-scale parameter and the block's
shifted-window mask (:274-293).  The rest of the model (blocks, patch merging,
embedding, head) is plain PyTorch with the reference's module and parameter
names, so a state_dict moves between the two implementations unchanged; it is
the harness for whole-model runs, not an optimisation target.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.utils.checkpoint import checkpoint

from .win_attention_func import (flash_win_attn_v2_func, flash_win_attn_v2_grid_func, flash_win_attn_v2_qkvpacked_func,
                                 win_attention_torch)
from .flash_window_attention_v2 import CpbBias, MAPPED_MAX_N, tensor_version
from .kernels import mask_window_flags


def _pair(x):
    return tuple(x) if isinstance(x, (tuple, list)) else (x, x)


def window_partition(x, window_size):
    """[B, H, W, C] -> [B * nW, ws, ws, C], batch outermost (swin_transformer_v2.py:156-168)."""
    b, h, w, c = x.shape
    x = x.reshape(b, h // window_size, window_size, w // window_size, window_size, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(-1, window_size, window_size, c)


def window_reverse(windows, window_size, h, w):
    """Inverse of window_partition (swin_transformer_v2.py:171-185)."""
    gh, gw = h // window_size, w // window_size
    b = windows.shape[0] // (gh * gw)
    x = windows.reshape(b, gh, gw, window_size, window_size, -1)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(b, h, w, -1)


def shifted_window_attn_mask(resolution, window_size, shift_size):
    """[nW, N, N] float32 mask of 0 / -100: two tokens of a window may attend to each other only
    if they come from the same region of the cyclically shifted image
    (swin_transformer_v2.py:386-405)."""
    h, w = resolution

    def bands(extent):
        idx = torch.arange(extent)
        return (idx >= extent - window_size).long() + (idx >= extent - shift_size).long()

    region = (3 * bands(h)[:, None] + bands(w)[None, :]).float()
    tiles = window_partition(region[None, :, :, None], window_size).reshape(-1, window_size * window_size)
    return torch.where(tiles[:, None, :] != tiles[:, :, None], -100.0, 0.0)


class Mlp(nn.Module):
    def __init__(self, in_features, hidden_features=None, out_features=None, act_layer=nn.GELU, drop=0.):
        super().__init__()
        self.fc1 = nn.Linear(in_features, hidden_features or in_features)
        self.act = act_layer()
        self.fc2 = nn.Linear(hidden_features or in_features, out_features or in_features)
        self.drop = nn.Dropout(drop)

    def forward(self, x):
        return self.drop(self.fc2(self.drop(self.act(self.fc1(x)))))


def trunc_normal_(tensor, mean=0., std=1., a=-2., b=2.):
    """Truncated-normal initialiser under the reference's name (swin_transformer_v2.py:88-113)."""
    return nn.init.trunc_normal_(tensor, mean=mean, std=std, a=a, b=b)


def drop_path(input, drop_prob=0.0, training=False):
    """Stochastic depth as a function (swin_transformer_v2.py:116-139): whole samples of a residual branch
    are dropped with probability `drop_prob` while training, the survivors scaled by 1 / (1 - drop_prob)."""
    if drop_prob == 0. or not training:
        return input
    keep = 1.0 - drop_prob
    gate = input.new_empty((input.shape[0],) + (1,) * (input.dim() - 1)).bernoulli_(keep)
    return input * gate / keep


class DropPath(nn.Module):
    """Stochastic depth: drops whole samples of a residual branch while training."""

    def __init__(self, drop_prob=0.):
        super().__init__()
        self.drop_prob = drop_prob

    def forward(self, x):
        return drop_path(x, self.drop_prob, self.training)

    def extra_repr(self):
        return f"p={self.drop_prob}"


class WindowAttention(nn.Module):
    """Window multi-head self attention with scaled-cosine scores and a continuous relative
    position bias.  Same arguments as the reference (swin_transformer_v2.py:188-266)."""

    #: feed the fused operator from the packed projection (flash path only); False selects the
    #: reference's call with three strided views
    packed_qkv = True
    #: build the bias (and take its gradient back to table space) with the library's two small kernels
    #: instead of gather / permute / sigmoid and autograd's sort-based scatter (flash path only)
    fused_bias = True
    #: let the kernels do the cyclic shift and the window partition / reverse of the enclosing block by
    #: address arithmetic (flash path only; used by SwinTransformerBlock when `grid_ready` says so)
    fused_grid = True
    #: keep the position bias between calls that record no gradient (see relative_position_bias)
    cache_bias = True
    _bias_cache = None

    def __init__(self, dim, window_size, num_heads, is_flash=True, qkv_bias=True, attn_drop=0., proj_drop=0.,
                 pretrained_window_size=[0, 0]):
        super().__init__()
        self.dim = dim
        self.window_size = _pair(window_size)
        self.pretrained_window_size = _pair(pretrained_window_size)
        self.num_heads = num_heads
        self.is_flash = is_flash
        if is_flash:
            assert attn_drop == 0.0, "flash window attention doesn't support dropout yet"

        self.logit_scale = nn.Parameter(torch.full((num_heads, 1, 1), math.log(10.0)))
        self.cpb_mlp = nn.Sequential(nn.Linear(2, 512, bias=True), nn.ReLU(inplace=True),
                                     nn.Linear(512, num_heads, bias=False))

        wh, ww = self.window_size
        # log-spaced relative coordinates in [-1, 1] * log2(9)/3
        dh = torch.arange(-(wh - 1), wh, dtype=torch.float32)
        dw = torch.arange(-(ww - 1), ww, dtype=torch.float32)
        ph, pw = self.pretrained_window_size
        dh = dh / ((ph if ph > 0 else wh) - 1) * 8
        dw = dw / ((pw if pw > 0 else ww) - 1) * 8
        table = torch.stack(torch.meshgrid(dh, dw, indexing="ij"), dim=-1)[None]
        table = torch.sign(table) * torch.log2(table.abs() + 1.0) / 3.0
        self.register_buffer("relative_coords_table", table)

        rows = torch.arange(wh).repeat_interleave(ww)
        cols = torch.arange(ww).repeat(wh)
        index = (rows[:, None] - rows[None, :] + wh - 1) * (2 * ww - 1) + (cols[:, None] - cols[None, :] + ww - 1)
        self.register_buffer("relative_position_index", index)

        self.qkv = nn.Linear(dim, dim * 3, bias=False)
        if qkv_bias:
            self.q_bias = nn.Parameter(torch.zeros(dim))
            self.v_bias = nn.Parameter(torch.zeros(dim))
        else:
            self.q_bias = None
            self.v_bias = None
        self.attn_drop = nn.Dropout(attn_drop)
        self.proj = nn.Linear(dim, dim)
        self.proj_drop = nn.Dropout(proj_drop)

    def _index_is_closed_form(self):
        """Whether the relative_position_index buffer (it travels in state_dicts) still holds the closed
        form the fused bias kernels compute on the fly; checked once per buffer version."""
        buf = self.relative_position_index
        seen = getattr(self, "_index_checked", None)
        version = tensor_version(buf)
        if seen is None or seen[0] != version or seen[1] != buf.data_ptr():
            wh, ww = self.window_size
            rows = torch.arange(wh, device=buf.device).repeat_interleave(ww)
            cols = torch.arange(ww, device=buf.device).repeat(wh)
            want = (rows[:, None] - rows[None, :] + wh - 1) * (2 * ww - 1) + (cols[:, None] - cols[None, :] + ww - 1)
            seen = (version, buf.data_ptr(), bool(torch.equal(buf, want)))
            self._index_checked = seen
        return seen[2]

    def relative_position_bias(self):
        """[H, N, N] bias = 16 sigmoid(cpb_mlp(table)[index]) (swin_transformer_v2.py:283-287).

        The bias depends on parameters and buffers only.  When no gradient is recorded (inference) it is kept
        until one of them changes (their version counters, dtype or device), which saves the two small GEMMs
        and the gather of every call; with gradients on it is rebuilt every call, as the reference does."""
        srcs = (*self.cpb_mlp.parameters(), self.relative_coords_table, self.relative_position_index)
        # parameters created under torch.inference_mode track no modifications: nothing is kept for them
        if torch.is_grad_enabled() or not self.cache_bias or any(t.is_inference() for t in srcs):
            self._bias_cache = None
            return self._build_relative_position_bias()
        key = tuple((t._version, t.data_ptr(), t.dtype) for t in srcs) + (torch.is_autocast_enabled(),)
        cached = self._bias_cache
        if cached is None or cached[0] != key:
            cached = (key, self._build_relative_position_bias())
            self._bias_cache = cached
        return cached[1]

    def _build_relative_position_bias(self):
        n = self.window_size[0] * self.window_size[1]
        per_offset = self.cpb_mlp(self.relative_coords_table).view(-1, self.num_heads)
        if (self.is_flash and self.fused_bias and per_offset.is_cuda
                and per_offset.dtype in (torch.float16, torch.bfloat16) and self._index_is_closed_form()):
            return CpbBias.apply(per_offset, self.window_size[0], self.window_size[1])
        bias = per_offset[self.relative_position_index.view(-1)].view(n, n, self.num_heads)
        return 16 * torch.sigmoid(bias.permute(2, 0, 1).contiguous())

    def forward(self, x, mask=None, mask_flags=None):
        """x: [B * nW, N, C]; mask: [nW, N, N] of 0 / -100 or None.  `mask_flags`: the per-window flags of `mask`
        when the caller holds them already (`kernels.mask_window_flags`); used by the packed path only."""
        b_, n, c = x.shape
        bias = None
        if self.q_bias is not None:
            bias = torch.cat((self.q_bias, torch.zeros_like(self.v_bias, requires_grad=False), self.v_bias))
        qkv = F.linear(x, self.qkv.weight, bias).reshape(b_, n, 3, self.num_heads, -1)
        rel_bias = self.relative_position_bias()
        scale = self.logit_scale
        if self.is_flash:
            scale, rel_bias = self._operator_dtype(qkv, scale, rel_bias)
        if self.is_flash and self.packed_qkv:
            # the kernels read q, k, v out of the GEMM output and write [B_, N, H, d]: no copies either
            # side, and one packed gradient instead of three that autograd would have to re-pack
            out = flash_win_attn_v2_qkvpacked_func(qkv, scale, rel_bias, mask, mask_flags).reshape(b_, n, c)
        else:
            q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)      # strided views, unit inner stride
            if self.is_flash:
                out = flash_win_attn_v2_func(q, k, v, scale, rel_bias, mask)
            else:
                out = win_attention_torch(q, k, v, scale, rel_bias, mask)
            out = out.transpose(1, 2).reshape(b_, n, c)
        return self.proj_drop(self.proj(out))

    @staticmethod
    def _operator_dtype(qkv, scale, rel_bias):
        """Under autocast the projection comes out in half precision while the parameters stay fp32; the
        fused operator wants its scale and bias in the dtype of q (attn_kernel_forward.py:274, 282), so they
        are cast on the way in (autograd casts the gradients back).  A module cast as a whole, as the
        reference's benchmarks do, passes through untouched."""
        if scale.dtype != qkv.dtype:
            scale = scale.to(qkv.dtype)
        if rel_bias.dtype != qkv.dtype:
            rel_bias = rel_bias.to(qkv.dtype)
        return scale, rel_bias

    def flops(self, N):
        """Multiply-accumulates of one window of N tokens, by the reference's count
        (swin_transformer_v2.py:304-315): qkv projection, q k^T, attn v, output projection."""
        head_dim = self.dim // self.num_heads
        return (N * self.dim * 3 * self.dim + 2 * self.num_heads * N * N * head_dim + N * self.dim * self.dim)

    def grid_ready(self, x):
        """True when `forward_grid` can take `x`: the fused path on the GPU in half precision, and a window the
        library addresses through a window map."""
        if not (self.is_flash and self.packed_qkv and self.fused_grid and x.is_cuda):
            return False
        if x.dtype not in (torch.float16, torch.bfloat16) and not torch.is_autocast_enabled():
            return False
        return self.window_size[0] * self.window_size[1] <= MAPPED_MAX_N and self.window_size[1] <= 64

    def forward_grid(self, x, grid, shift, mask=None, mask_flags=None):
        """The attention of every (shifted) window of the token grid x [B, gh * gw, C], result in the same
        layout: what the reference's block computes with roll + window_partition around `forward` and
        window_reverse + roll after it (swin_transformer_v2.py:419-441), with the permutation done by the
        kernels' addressing.  `shift` = (shift_size, shift_size) of the block."""
        b, length, c = x.shape
        bias = None
        if self.q_bias is not None:
            bias = torch.cat((self.q_bias, torch.zeros_like(self.v_bias, requires_grad=False), self.v_bias))
        qkv = F.linear(x, self.qkv.weight, bias).reshape(b, length, 3, self.num_heads, -1)
        rel_bias = self.relative_position_bias()
        scale, rel_bias = self._operator_dtype(qkv, self.logit_scale, rel_bias)
        out = flash_win_attn_v2_grid_func(qkv, grid, self.window_size, shift, scale, rel_bias, mask, mask_flags)
        return self.proj_drop(self.proj(out.reshape(b, length, c)))

    def extra_repr(self):
        return (f"dim={self.dim}, window_size={self.window_size}, "
                f"pretrained_window_size={self.pretrained_window_size}, num_heads={self.num_heads}")


class SwinTransformerBlock(nn.Module):
    """(Shifted-)window attention + MLP with residual post-normalisation
    (swin_transformer_v2.py:318-447)."""

    def __init__(self, dim, input_resolution, num_heads, window_size=7, shift_size=0, is_flash=True, mlp_ratio=4.,
                 qkv_bias=True, drop=0., attn_drop=0., drop_path=0., act_layer=nn.GELU, norm_layer=nn.LayerNorm,
                 pretrained_window_size=0):
        super().__init__()
        self.dim = dim
        self.input_resolution = input_resolution
        self.num_heads = num_heads
        self.window_size = window_size
        self.shift_size = shift_size
        self.is_flash = is_flash
        self.mlp_ratio = mlp_ratio
        if min(input_resolution) <= window_size:     # one window covers the map: no shift
            self.shift_size = 0
            self.window_size = min(input_resolution)
        assert 0 <= self.shift_size < self.window_size, "shift_size must in 0-window_size"

        self.norm1 = norm_layer(dim)
        self.attn = WindowAttention(dim, window_size=_pair(self.window_size), num_heads=num_heads, is_flash=is_flash,
                                    qkv_bias=qkv_bias, attn_drop=attn_drop, proj_drop=drop,
                                    pretrained_window_size=_pair(pretrained_window_size))
        self.drop_path = DropPath(drop_path) if drop_path > 0. else nn.Identity()
        self.norm2 = norm_layer(dim)
        self.mlp = Mlp(in_features=dim, hidden_features=int(dim * mlp_ratio), act_layer=act_layer, drop=drop)
        mask = None
        if self.shift_size > 0:
            mask = shifted_window_attn_mask(input_resolution, self.window_size, self.shift_size)
        self.register_buffer("attn_mask", mask)
        self._attn_mask_flags = None

    def _apply(self, fn, *args, **kwargs):
        # .to() / .cuda() / .half() replace the buffer: its flags are scanned again on the next call
        self._attn_mask_flags = None
        return super()._apply(fn, *args, **kwargs)

    def mask_flags(self):
        """Per-window flags of `attn_mask` for the fused operator, scanned once per buffer and kept on the block.
        The block owns the buffer and never edits it, so the flags stay valid whatever mode the buffer was
        created in: a model built under torch.inference_mode (benchmark/bench_model.py:14-19 of the reference)
        has a mask without a modification counter, which `mask_window_flags` alone would rescan on every call."""
        mask = self.attn_mask
        if mask is None or not (self.is_flash and mask.is_cuda):
            return None
        key = (mask.data_ptr(), mask.device, mask.dtype, tuple(mask.shape), tensor_version(mask))
        held = self._attn_mask_flags
        if held is not None and held[0] == key:
            return held[1]
        flags = mask_window_flags(mask)
        if not torch.cuda.is_current_stream_capturing():
            self._attn_mask_flags = (key, flags)
        return flags

    def forward(self, x):
        h, w = self.input_resolution
        b, length, c = x.shape
        assert length == h * w, "input feature has wrong size"
        shortcut = x
        if self.attn.grid_ready(x):
            # roll, window_partition, window_reverse and the roll back happen inside the kernels
            x = self.attn.forward_grid(x, (h, w), (self.shift_size, self.shift_size), mask=self.attn_mask,
                                       mask_flags=self.mask_flags())
            x = shortcut + self.drop_path(self.norm1(x))
            return x + self.drop_path(self.norm2(self.mlp(x)))
        x = x.view(b, h, w, c)
        if self.shift_size > 0:
            x = torch.roll(x, shifts=(-self.shift_size, -self.shift_size), dims=(1, 2))
        windows = window_partition(x, self.window_size).view(-1, self.window_size * self.window_size, c)
        windows = self.attn(windows, mask=self.attn_mask, mask_flags=self.mask_flags())
        x = window_reverse(windows.view(-1, self.window_size, self.window_size, c), self.window_size, h, w)
        if self.shift_size > 0:
            x = torch.roll(x, shifts=(self.shift_size, self.shift_size), dims=(1, 2))
        x = shortcut + self.drop_path(self.norm1(x.reshape(b, h * w, c)))
        return x + self.drop_path(self.norm2(self.mlp(x)))

    def flops(self):
        """The reference's count (swin_transformer_v2.py:453-465): two norms, the windows' attention, the MLP."""
        h, w = self.input_resolution
        n_windows = h * w / self.window_size / self.window_size
        return (2 * self.dim * h * w + n_windows * self.attn.flops(self.window_size * self.window_size)
                + 2 * h * w * self.dim * self.dim * self.mlp_ratio)

    def extra_repr(self):
        return (f"dim={self.dim}, input_resolution={self.input_resolution}, num_heads={self.num_heads}, "
                f"window_size={self.window_size}, shift_size={self.shift_size}, mlp_ratio={self.mlp_ratio}")


class PatchMerging(nn.Module):
    """2x2 neighbourhood concat -> linear 4C -> 2C -> norm (swin_transformer_v2.py:468-514)."""

    def __init__(self, input_resolution, dim, norm_layer=nn.LayerNorm):
        super().__init__()
        self.input_resolution = input_resolution
        self.dim = dim
        self.reduction = nn.Linear(4 * dim, 2 * dim, bias=False)
        self.norm = norm_layer(2 * dim)

    def forward(self, x):
        h, w = self.input_resolution
        b, length, c = x.shape
        assert length == h * w, "input feature has wrong size"
        assert h % 2 == 0 and w % 2 == 0, f"x size ({h}*{w}) are not even."
        x = x.view(b, h // 2, 2, w // 2, 2, c)
        # channel order (row parity, column parity) = (0,0), (1,0), (0,1), (1,1)
        x = x.permute(0, 1, 3, 4, 2, 5).reshape(b, (h // 2) * (w // 2), 4 * c)
        return self.norm(self.reduction(x))

    def flops(self):
        """The reference's count (swin_transformer_v2.py:510-514): the 4C -> 2C reduction and the norm."""
        h, w = self.input_resolution
        return (h // 2) * (w // 2) * 4 * self.dim * 2 * self.dim + h * w * self.dim // 2


class BasicLayer(nn.Module):
    """One stage: `depth` blocks alternating unshifted / shifted windows, then optional merging
    (swin_transformer_v2.py:517-617)."""

    def __init__(self, dim, input_resolution, depth, num_heads, window_size, is_flash=True, mlp_ratio=4.,
                 qkv_bias=True, drop=0., attn_drop=0., drop_path=0., norm_layer=nn.LayerNorm, downsample=None,
                 use_checkpoint=False, pretrained_window_size=0):
        super().__init__()
        self.dim = dim
        self.input_resolution = input_resolution
        self.depth = depth
        self.use_checkpoint = use_checkpoint
        self.blocks = nn.ModuleList([
            SwinTransformerBlock(dim=dim, input_resolution=input_resolution, num_heads=num_heads,
                                 window_size=window_size, shift_size=0 if i % 2 == 0 else window_size // 2,
                                 is_flash=is_flash, mlp_ratio=mlp_ratio, qkv_bias=qkv_bias, drop=drop,
                                 attn_drop=attn_drop,
                                 drop_path=drop_path[i] if isinstance(drop_path, (list, tuple)) else drop_path,
                                 norm_layer=norm_layer, pretrained_window_size=pretrained_window_size)
            for i in range(depth)])
        self.downsample = downsample(input_resolution, dim=dim, norm_layer=norm_layer) if downsample else None

    def forward(self, x):
        for blk in self.blocks:
            x = checkpoint(blk, x, use_reentrant=False) if self.use_checkpoint else blk(x)
        return self.downsample(x) if self.downsample is not None else x

    def flops(self):
        total = sum(blk.flops() for blk in self.blocks)
        return total + (self.downsample.flops() if self.downsample is not None else 0)

    def _init_respostnorm(self):
        """Residual post-norm starts as the identity: both LayerNorms of every block at zero."""
        for blk in self.blocks:
            for norm in (blk.norm1, blk.norm2):
                nn.init.zeros_(norm.weight)
                nn.init.zeros_(norm.bias)


class PatchEmbed(nn.Module):
    """Non-overlapping patch projection (swin_transformer_v2.py:620-665)."""

    def __init__(self, img_size=224, patch_size=4, in_chans=3, embed_dim=96, norm_layer=None):
        super().__init__()
        self.img_size = _pair(img_size)
        self.patch_size = _pair(patch_size)
        self.patches_resolution = [self.img_size[0] // self.patch_size[0], self.img_size[1] // self.patch_size[1]]
        self.num_patches = self.patches_resolution[0] * self.patches_resolution[1]
        self.in_chans = in_chans
        self.embed_dim = embed_dim
        self.proj = nn.Conv2d(in_chans, embed_dim, kernel_size=self.patch_size, stride=self.patch_size)
        self.norm = norm_layer(embed_dim) if norm_layer is not None else None

    def forward(self, x):
        assert tuple(x.shape[2:]) == self.img_size, \
            f"Input image size ({x.shape[2]}*{x.shape[3]}) doesn't match model ({self.img_size[0]}*{self.img_size[1]})."
        x = self.proj(x).flatten(2).transpose(1, 2)
        return self.norm(x) if self.norm is not None else x

    def flops(self):
        """The reference's count (swin_transformer_v2.py:660-665): the patch projection and its norm."""
        ho, wo = self.patches_resolution
        total = ho * wo * self.embed_dim * self.in_chans * (self.patch_size[0] * self.patch_size[1])
        return total + (ho * wo * self.embed_dim if self.norm is not None else 0)


class SwinTransformerV2(nn.Module):
    """Hierarchical Swin V2 classifier with the reference's constructor arguments and parameter
    names (swin_transformer_v2.py:668-822)."""

    def __init__(self, img_size=256, patch_size=4, in_chans=3, num_classes=1000, embed_dim=96, depths=[2, 2, 6, 2],
                 num_heads=[3, 6, 12, 24], window_size=8, is_flash=True, mlp_ratio=4., qkv_bias=True, drop_rate=0.,
                 attn_drop_rate=0., drop_path_rate=0.1, norm_layer=nn.LayerNorm, ape=False, patch_norm=True,
                 use_checkpoint=False, pretrained_window_sizes=[0, 0, 0, 0], **kwargs):
        super().__init__()
        self.num_classes = num_classes
        self.num_layers = len(depths)
        self.embed_dim = embed_dim
        self.ape = ape
        self.patch_norm = patch_norm
        self.num_features = int(embed_dim * 2 ** (self.num_layers - 1))
        self.is_flash = is_flash
        self.mlp_ratio = mlp_ratio

        self.patch_embed = PatchEmbed(img_size=img_size, patch_size=patch_size, in_chans=in_chans, embed_dim=embed_dim,
                                      norm_layer=norm_layer if patch_norm else None)
        res = self.patch_embed.patches_resolution
        self.patches_resolution = res
        if ape:
            self.absolute_pos_embed = nn.Parameter(torch.zeros(1, self.patch_embed.num_patches, embed_dim))
            nn.init.trunc_normal_(self.absolute_pos_embed, std=.02)
        self.pos_drop = nn.Dropout(p=drop_rate)

        rates = torch.linspace(0, drop_path_rate, sum(depths)).tolist()
        self.layers = nn.ModuleList()
        for i, depth in enumerate(depths):
            first = sum(depths[:i])
            self.layers.append(BasicLayer(
                dim=int(embed_dim * 2 ** i), input_resolution=(res[0] // 2 ** i, res[1] // 2 ** i), depth=depth,
                num_heads=num_heads[i], window_size=window_size, is_flash=is_flash, mlp_ratio=mlp_ratio,
                qkv_bias=qkv_bias, drop=drop_rate, attn_drop=attn_drop_rate, drop_path=rates[first:first + depth],
                norm_layer=norm_layer, downsample=PatchMerging if i < self.num_layers - 1 else None,
                use_checkpoint=use_checkpoint, pretrained_window_size=pretrained_window_sizes[i]))

        self.norm = norm_layer(self.num_features)
        self.avgpool = nn.AdaptiveAvgPool1d(1)
        self.head = nn.Linear(self.num_features, num_classes) if num_classes > 0 else nn.Identity()

        self.apply(self._init_weights)
        for layer in self.layers:
            layer._init_respostnorm()

    @staticmethod
    def _init_weights(m):
        if isinstance(m, nn.Linear):
            nn.init.trunc_normal_(m.weight, std=.02)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, nn.LayerNorm):
            nn.init.zeros_(m.bias)
            nn.init.ones_(m.weight)

    @torch.jit.ignore
    def no_weight_decay(self):
        return {"absolute_pos_embed"}

    @torch.jit.ignore
    def no_weight_decay_keywords(self):
        return {"cpb_mlp", "logit_scale", "relative_position_bias_table"}

    def forward_features(self, x):
        x = self.patch_embed(x)
        if self.ape:
            x = x + self.absolute_pos_embed
        x = self.pos_drop(x)
        for layer in self.layers:
            x = layer(x)
        x = self.norm(x)
        return torch.flatten(self.avgpool(x.transpose(1, 2)), 1)

    def forward(self, x):
        return self.head(self.forward_features(x))

    def flops(self):
        """The reference's count (swin_transformer_v2.py:816-823): embedding, stages, final norm, head."""
        total = self.patch_embed.flops() + sum(layer.flops() for layer in self.layers)
        total += self.num_features * self.patches_resolution[0] * self.patches_resolution[1] // (2 ** self.num_layers)
        return total + self.num_features * self.num_classes
