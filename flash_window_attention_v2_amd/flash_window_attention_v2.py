"""`FlashWindowAttentionV2`: the autograd Function of the reference
(flash_win_attn_v2/flash_window_attention_v2.py:5-57) with the same signature, saved tensors and six-value
backward, on top of the launchers of `kernels.py` as the reference's sits on its `kernels` package; and two
Functions without a counterpart there, fed from the packed qkv projection and from the un-partitioned
token grid.
"""
import torch

from . import _abi
from .kernels import (_DTYPES, _check_inputs, _describe, _flags_for, _flash_attn_backward, _flash_attn_forward,
                      _kernel_ready, _on_device, _rows_16b_aligned, _set_t4, mask_window_flags, tensor_version)


def _scale_argument(logit_scale, device):
    """(tensor for the saved-tensor slot, scale_type) as the reference derives them
    (flash_window_attention_v2.py:9-17)."""
    if logit_scale is not None:
        assert isinstance(logit_scale, torch.Tensor), \
            "Make sure logit_scale is a tensor if defined in the paramaters."
        return (logit_scale if logit_scale.is_contiguous() else logit_scale.contiguous()), "tensor"
    # placeholder for the saved-tensor slot (the reference keeps 1/sqrt(d) there); the kernels derive the
    # default scale from head_dim, and filling a device scalar from the host would synchronise and break
    # stream capture
    return torch.empty((), device=device), "scalar"


def _packed_forward(q, k, v, units, logit_scale, bias, mask, scale_type, window_map=None, mask_flags=None):
    """Forward of the two packed Functions: q, k, v are [B, H, L, d] views of one qkv buffer, `units` the
    (number of windows, tokens per window) the library sees.  Returns out [B, L, H, d], lse and the mask's
    per-window flags (kept for backward).  `mask_flags`: flags the caller already holds for this mask (the
    result of `mask_window_flags`), for masks that cannot carry their own cache."""
    b, heads, length, d = q.shape
    bw, n = units
    lse = torch.empty((bw, heads, (n + 63) // 64 * 64), device=q.device, dtype=torch.float32)
    out = torch.empty((b, length, heads, d), device=q.device, dtype=q.dtype)
    if mask is None:
        mask_live = None
    elif mask_flags is not None:
        assert (mask_flags.dtype == torch.uint8 and mask_flags.device == mask.device
                and mask_flags.shape == (mask.shape[0],)), "mask_flags must be what mask_window_flags(mask) returns"
        mask_live = mask_flags
    else:
        mask_live = mask_window_flags(mask)
    p = _describe(q, k, v, out.transpose(1, 2), lse, logit_scale, bias, mask, mask_live, scale_type, window_map)
    with _on_device(q.device) as stream:
        p.stream = stream
        _abi.check(_abi.load().fwa2_forward(p), "fwa2_forward")
    return out, lse, mask_live


def _packed_backward(qkv, q, k, v, out, lse, logit_scale, bias, mask, mask_live, scale_type, do, window_map=None):
    """Backward of the two packed Functions: dq, dk, dv land in one buffer shaped like qkv."""
    dqkv = torch.empty_like(qkv)
    dq, dk, dv = (dqkv[:, :, i].transpose(1, 2) for i in range(3))
    dscale = torch.empty_like(logit_scale, memory_format=torch.contiguous_format) if scale_type == "tensor" else None
    db = torch.empty_like(bias, memory_format=torch.contiguous_format) if bias is not None else None
    lib = _abi.load()
    p = _describe(q, k, v, out.transpose(1, 2), lse, logit_scale, bias, mask, mask_live, scale_type, window_map)
    _set_t4(p.d_o, do); _set_t4(p.dq, dq); _set_t4(p.dk, dk); _set_t4(p.dv, dv)
    if db is not None:
        p.dbias = db.data_ptr()
    if dscale is not None:
        p.dscale = dscale.data_ptr()
    with _on_device(qkv.device) as stream:
        need = lib.fwa2_backward_workspace_bytes(p)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=qkv.device)
        p.workspace, p.workspace_bytes = ws.data_ptr(), need
        p.stream = stream
        _abi.check(lib.fwa2_backward(p), "fwa2_backward")
    return dqkv, dscale, db


class FlashWindowAttentionV2(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, logit_scale=None, bias=None, mask=None):
        logit_scale, scale_type = _scale_argument(logit_scale, q.device)

        # unit inner stride is the reference's requirement (flash_window_attention_v2.py:20), 16-byte-aligned
        # rows this library's: copy only when either fails
        q, k, v = (_kernel_ready(x) for x in (q, k, v))
        o, lse, logit_scale = _flash_attn_forward(q, k, v, logit_scale, bias=bias, mask=mask, scale_type=scale_type)

        ctx.save_for_backward(q, k, v, o, lse, logit_scale, bias, mask)
        ctx.scale_type = scale_type
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, logit_scale, bias, mask = ctx.saved_tensors
        scale_type = ctx.scale_type
        dq, dk, dv = (torch.empty_like(x) for x in (q, k, v))
        if not all(_rows_16b_aligned(x) for x in (dq, dk, dv)):      # rows the kernels can write directly
            dq, dk, dv = (torch.empty(x.shape, device=x.device, dtype=x.dtype) for x in (q, k, v))
        dscale = torch.empty_like(logit_scale, memory_format=torch.contiguous_format) if scale_type == "tensor" else None
        db = torch.empty_like(bias, memory_format=torch.contiguous_format) if bias is not None else None
        _flash_attn_backward(do, q, k, v, logit_scale, o, lse, dq, dk, dv, dscale, db, bias=bias, mask=mask,
                             scale_type=scale_type)
        return dq, dk, dv, dscale, db, None


class FlashWindowAttentionV2QKVPacked(torch.autograd.Function):
    """The same operator fed straight from the qkv projection, for the caller at
    swin_transformer_v2.py:279-295 of the reference: `qkv` is the GEMM output viewed as
    [BW, N, 3, H, d]; the result is [BW, N, H, d], so the caller's transpose + reshape to
    [BW, N, C] is a view.  Backward writes dq, dk and dv into one [BW, N, 3, H, d] buffer,
    which removes the three zero-fill + strided-copy passes autograd otherwise spends on
    re-packing separate gradients.  Has no counterpart in the reference, whose kernels
    take the same strided views but return separate tensors."""

    @staticmethod
    def forward(ctx, qkv, logit_scale=None, bias=None, mask=None, mask_flags=None):
        assert qkv.dim() == 5 and qkv.shape[2] == 3, "qkv must be [BW, N, 3, H, d]"
        if not (_rows_16b_aligned(qkv) and qkv.is_contiguous()):
            qkv = qkv.contiguous()
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))       # [BW, H, N, d] views
        logit_scale, scale_type = _scale_argument(logit_scale, q.device)
        _check_inputs(q, k, v, logit_scale, bias, mask, scale_type)
        if bias is not None and bias.stride(-1) != 1:
            bias = bias.contiguous()
        if mask is not None and mask.stride(-1) != 1:
            mask = mask.contiguous()

        bw, heads, n, d = q.shape
        out, lse, mask_live = _packed_forward(q, k, v, (bw, n), logit_scale, bias, mask, scale_type, mask_flags=mask_flags)

        ctx.save_for_backward(qkv, out, lse, logit_scale, bias, mask)
        ctx.scale_type = scale_type
        ctx.mask_live = mask_live
        return out

    @staticmethod
    def backward(ctx, dout):
        qkv, out, lse, logit_scale, bias, mask = ctx.saved_tensors
        scale_type = ctx.scale_type
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
        do = dout.transpose(1, 2)                                          # [BW, H, N, d] view
        if not _rows_16b_aligned(do):
            do = do.contiguous()
        dqkv, dscale, db = _packed_backward(qkv, q, k, v, out, lse, logit_scale, bias, mask, ctx.mask_live, scale_type, do)
        return dqkv, dscale, db, None, None


MAPPED_MAX_N = 1024     # largest window the library addresses through a window map


class FlashWindowAttentionV2Grid(torch.autograd.Function):
    """The packed operator applied to the un-partitioned token grid: the cyclic shift, window_partition,
    window_reverse and the shift back that surround the attention call in the reference's block
    (swin_transformer_v2.py:419-441) become address arithmetic inside the kernels, so none of the four
    copies (nor their four backward copies) is made.  `qkv` is the projection output [B, gh * gw, 3, H, d]
    of the image tokens in row-major order; the result is [B, gh * gw, H, d] in the same order.  The qkv and
    output projections act on single tokens, so they commute with the permutation and the caller applies
    them to the grid.  `shift` is the block's shift_size (the reference rolls by -shift before partitioning).
    Has no counterpart in the reference."""

    @staticmethod
    def forward(ctx, qkv, grid, window, shift, logit_scale=None, bias=None, mask=None, mask_flags=None):
        (gh, gw), (wh, ww), (sh, sw) = grid, window, shift
        assert qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.shape[1] == gh * gw, "qkv must be [B, gh * gw, 3, H, d]"
        assert gh % wh == 0 and gw % ww == 0, "the grid must be a whole number of windows"
        if not (_rows_16b_aligned(qkv) and qkv.is_contiguous()):
            qkv = qkv.contiguous()
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))       # [B, H, L, d] views
        logit_scale, scale_type = _scale_argument(logit_scale, q.device)
        b, heads, length, d = q.shape
        n, nw = wh * ww, (gh // wh) * (gw // ww)
        assert d <= 128, "FlashAttention only support head dimensions up to 128"
        assert q.dtype in (torch.float16, torch.bfloat16), "Only support fp16 and bf16"
        assert q.is_cuda, "qkv must be on the GPU"
        if scale_type == "tensor":
            assert logit_scale.is_cuda and logit_scale.shape == (heads, 1, 1) and logit_scale.dtype == q.dtype
        if bias is not None:
            assert bias.is_cuda and bias.dtype == q.dtype and bias.shape == (heads, n, n)
            if bias.stride(-1) != 1:
                bias = bias.contiguous()
        if mask is not None:
            assert mask.is_cuda and mask.dtype in (q.dtype, torch.float32)
            assert mask.shape == (nw, n, n), "mask must be [nW, N, N] with nW the windows of one image"
            if mask.stride(-1) != 1:
                mask = mask.contiguous()

        window_map = ((gh, gw), (wh, ww), (sh % gh, sw % gw))
        out, lse, mask_live = _packed_forward(q, k, v, (b * nw, n), logit_scale, bias, mask, scale_type, window_map,
                                              mask_flags=mask_flags)

        ctx.save_for_backward(qkv, out, lse, logit_scale, bias, mask)
        ctx.scale_type = scale_type
        ctx.mask_live = mask_live
        ctx.window_map = window_map
        return out

    @staticmethod
    def backward(ctx, dout):
        qkv, out, lse, logit_scale, bias, mask = ctx.saved_tensors
        scale_type = ctx.scale_type
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
        do = dout.transpose(1, 2)                                          # [B, H, L, d] view
        if not _rows_16b_aligned(do):
            do = do.contiguous()
        dqkv, dscale, db = _packed_backward(qkv, q, k, v, out, lse, logit_scale, bias, mask, ctx.mask_live, scale_type, do,
                                            ctx.window_map)
        return dqkv, None, None, None, dscale, db, None, None


class CpbBias(torch.autograd.Function):
    """bias[H, N, N] = 16 sigmoid(table[index]) for a window of wh x ww tokens, where `table` is the
    [(2wh-1)(2ww-1), H] output of the continuous-position-bias MLP and `index` the closed form of the
    reference's relative_position_index buffer (swin_transformer_v2.py:240-254, 283-287).  One small kernel
    each way instead of gather + permute + sigmoid + scale, and in backward a fixed-order fp32 sum per
    table entry instead of autograd's sort-based index_put(accumulate)."""

    @staticmethod
    def forward(ctx, table, wh, ww):
        assert table.is_cuda and table.dtype in (torch.float16, torch.bfloat16), "fused bias path: fp16 / bf16 on the GPU"
        assert table.dim() == 2 and table.shape[0] == (2 * wh - 1) * (2 * ww - 1), "table must be [(2wh-1)(2ww-1), H]"
        table = table.contiguous()
        heads = table.shape[1]
        n = wh * ww
        bias = torch.empty((heads, n, n), device=table.device, dtype=table.dtype)
        lib = _abi.load()
        with _on_device(table.device) as stream:
            _abi.check(lib.fwa2_cpb_bias_forward(table.data_ptr(), _DTYPES[table.dtype], heads, wh, ww, bias.data_ptr(),
                                                 stream), "fwa2_cpb_bias_forward")
        ctx.save_for_backward(table)
        ctx.window = (wh, ww)
        return bias

    @staticmethod
    def backward(ctx, dbias):
        (table,) = ctx.saved_tensors
        wh, ww = ctx.window
        dbias = dbias.contiguous()
        dtable = torch.empty_like(table)
        lib = _abi.load()
        with _on_device(table.device) as stream:
            _abi.check(lib.fwa2_cpb_bias_backward(table.data_ptr(), dbias.data_ptr(), _DTYPES[table.dtype], table.shape[1],
                                                  wh, ww, dtable.data_ptr(), stream),
                       "fwa2_cpb_bias_backward")
        return dtable, None, None
