"""`FlashWindowAttentionV2`: the autograd Function of the reference
(flash_win_attn_v2/flash_window_attention_v2.py:5-57) with the same
signature, saved tensors and six-value backward, whose body marshals raw
device pointers and strides to the gfx950 kernels in libfwa2.so.

Every buffer -- outputs, log-sum-exp, gradients and the backward workspace --
is a torch tensor allocated here, so torch's allocator statistics stay honest
and the C side allocates nothing.
"""

import torch

from . import _abi

_DTYPES = {torch.float16: _abi.F16, torch.bfloat16: _abi.BF16, torch.float32: _abi.F32}


def _t4(t):
    return _abi.Tensor4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def _set_t4(dst, t):
    st = t.stride()
    dst.ptr, dst.stride_bw, dst.stride_h, dst.stride_n = t.data_ptr(), st[0], st[1], st[2]


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", None)


class _on_device:
    """Make `device` current for the duration of a library call and hand back the raw handle of its
    current stream.  The common case (the device is current already) costs two C calls; only a
    different device goes through torch's device guard."""

    __slots__ = ("index", "guard")

    def __init__(self, device):
        self.index = device.index if device.index is not None else torch.cuda.current_device()
        self.guard = None

    def __enter__(self):
        if _get_device is None or _get_device() != self.index:
            self.guard = torch.cuda.device(self.index)
            self.guard.__enter__()
        if _raw_stream is not None:
            return _raw_stream(self.index)
        return torch.cuda.current_stream(self.index).cuda_stream

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def _rows_16b_aligned(t):
    return t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])


def _kernel_ready(t):
    """Unit inner stride is the reference's requirement (flash_window_attention_v2.py:20);
    16-byte-aligned rows are this library's: copy only when either fails."""
    return t if _rows_16b_aligned(t) else t.contiguous()


def tensor_version(t):
    """The in-place modification counter of `t`, or None for a tensor created under torch.inference_mode,
    which keeps none (asking for it raises)."""
    return None if t.is_inference() else t._version


def mask_window_flags(mask):
    """uint8[nW]: 1 where a window's mask has a non-zero entry (device tensor).
    Cached on the mask tensor object and refreshed if the tensor is modified in place (a mask created under
    torch.inference_mode tracks no modifications: edit such a mask by making a new tensor)."""
    cached = getattr(mask, "_fwa2_live", None)
    version = tensor_version(mask)
    if cached is not None and cached[0] == version and cached[1].device == mask.device:
        return cached[1]
    lib = _abi.load()
    live = torch.empty(mask.shape[0], dtype=torch.uint8, device=mask.device)
    with _on_device(mask.device) as stream:
        st = lib.fwa2_mask_scan(mask.data_ptr(), _DTYPES[mask.dtype], mask.shape[0], mask.shape[1], mask.stride(0),
                                mask.stride(1), live.data_ptr(), stream)
    _abi.check(st, "fwa2_mask_scan")
    try:
        mask._fwa2_live = (version, live)
    except Exception:
        pass
    return live


def _describe(q, k, v, o, lse, logit_scale, bias, mask, mask_live, scale_type, window_map=None):
    bw, heads, n, d = q.shape
    p = _abi.new_problem()
    if window_map is not None:
        # q, k, v, o are token grids [B, H, gh * gw, d]; the library partitions them into windows
        (gh, gw), (wh, ww), (sh, sw) = window_map
        p.grid_h, p.grid_w, p.win_h, p.win_w, p.shift_h, p.shift_w = gh, gw, wh, ww, sh, sw
        bw, n = bw * (gh // wh) * (gw // ww), wh * ww
    p.dtype = _DTYPES[q.dtype]
    p.scale_kind = _abi.SCALE_TENSOR if scale_type == "tensor" else _abi.SCALE_DEFAULT
    p.bw, p.heads, p.n, p.head_dim = bw, heads, n, d
    if window_map is None and k.shape[2] != n:
        p.n_keys = k.shape[2]
    p.n_windows = mask.shape[0] if mask is not None else 1
    _set_t4(p.q, q); _set_t4(p.k, k); _set_t4(p.v, v); _set_t4(p.o, o)
    if scale_type == "tensor":
        p.logit_scale = logit_scale.data_ptr()
    if bias is not None:
        p.bias.ptr, p.bias.stride_a, p.bias.stride_n = bias.data_ptr(), bias.stride(0), bias.stride(1)
    if mask is not None:
        p.mask.ptr, p.mask.stride_a, p.mask.stride_n = mask.data_ptr(), mask.stride(0), mask.stride(1)
        p.mask_dtype = _DTYPES[mask.dtype]
        if mask_live is not None:
            p.mask_live = mask_live.data_ptr()
    else:
        p.mask_dtype = p.dtype
    p.lse = lse.data_ptr()
    p.lse_stride_bw, p.lse_stride_h = lse.stride(0), lse.stride(1)
    return p


def _check_inputs(q, k, v, logit_scale, bias, mask, scale_type):
    """The reference launcher's assertions (attn_kernel_forward.py:263-292)."""
    bw, heads, n, d = q.shape
    n_k = k.shape[2]      # may differ from n (attn_kernel_forward.py:263-264); no caller of the reference does
    assert k.shape == (bw, heads, n_k, d) and v.shape == k.shape, "q, k, v shapes do not match"
    assert d <= 128, "FlashAttention only support head dimensions up to 128"
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in (torch.float16, torch.bfloat16), "Only support fp16 and bf16"
    assert q.is_cuda and k.is_cuda and v.is_cuda, "q, k, v must be on the GPU"
    if scale_type == "tensor":
        assert logit_scale.is_cuda
        assert logit_scale.shape == (heads, 1, 1)
        assert logit_scale.dtype == q.dtype
    if bias is not None:
        assert bias.dtype == q.dtype
        assert bias.is_cuda
        assert bias.shape == (heads, n, n_k)
    if mask is not None:
        assert mask.dtype in (q.dtype, torch.float32)
        assert mask.is_cuda
        assert mask.dim() == 3 and mask.shape[1:] == (n, n_k) and bw % mask.shape[0] == 0, \
            "mask must be [nW, N, N_k] with BW % nW == 0"


class FlashWindowAttentionV2(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, logit_scale=None, bias=None, mask=None):
        if logit_scale is not None:
            assert isinstance(logit_scale, torch.Tensor), \
                "Make sure logit_scale is a tensor if defined in the paramaters."
            scale_type = "tensor"
            logit_scale = logit_scale if logit_scale.stride(-1) == 1 else logit_scale.contiguous()
        else:
            scale_type = "scalar"
            # placeholder for the saved-tensor slot (the reference keeps 1/sqrt(d) there, fn.py:15-17); the
            # kernels derive the default scale from head_dim, and filling a device scalar from the host
            # would synchronise and break stream capture
            logit_scale = torch.empty((), device=q.device)

        _check_inputs(q, k, v, logit_scale, bias, mask, scale_type)
        q, k, v = (_kernel_ready(x) for x in (q, k, v))
        if scale_type == "tensor" and not logit_scale.is_contiguous():
            logit_scale = logit_scale.contiguous()
        if bias is not None and bias.stride(-1) != 1:
            bias = bias.contiguous()
        if mask is not None and mask.stride(-1) != 1:
            mask = mask.contiguous()

        bw, heads, n, _ = q.shape
        lib = _abi.load()
        lse = torch.empty((bw, heads, (n + 63) // 64 * 64), device=q.device, dtype=torch.float32)
        o = torch.empty_like(q)
        if not _rows_16b_aligned(o):
            o = torch.empty(q.shape, device=q.device, dtype=q.dtype)
        # the flag scan covers square masks; with other key counts the kernels go without the flags
        mask_live = mask_window_flags(mask) if mask is not None and mask.shape[1] == mask.shape[2] else None
        p = _describe(q, k, v, o, lse, logit_scale, bias, mask, mask_live, scale_type)
        with _on_device(q.device) as stream:
            p.stream = stream
            _abi.check(lib.fwa2_forward(p), "fwa2_forward")

        ctx.save_for_backward(q, k, v, o, lse, logit_scale, bias, mask)
        ctx.scale_type = scale_type
        ctx.mask_live = mask_live
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, logit_scale, bias, mask = ctx.saved_tensors
        scale_type = ctx.scale_type
        do = _kernel_ready(do)
        dq, dk, dv = (torch.empty_like(x) for x in (q, k, v))
        if not all(_rows_16b_aligned(x) for x in (dq, dk, dv)):
            dq, dk, dv = (torch.empty(x.shape, device=x.device, dtype=x.dtype) for x in (q, k, v))
        dscale = torch.empty_like(logit_scale, memory_format=torch.contiguous_format) if scale_type == "tensor" else None
        db = torch.empty_like(bias, memory_format=torch.contiguous_format) if bias is not None else None

        lib = _abi.load()
        p = _describe(q, k, v, o, lse, logit_scale, bias, mask, ctx.mask_live, scale_type)
        _set_t4(p.d_o, do); _set_t4(p.dq, dq); _set_t4(p.dk, dk); _set_t4(p.dv, dv)
        if db is not None:
            p.dbias = db.data_ptr()
        if dscale is not None:
            p.dscale = dscale.data_ptr()
        with _on_device(q.device) as stream:
            need = lib.fwa2_backward_workspace_bytes(p)
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device=q.device)
            p.workspace, p.workspace_bytes = ws.data_ptr(), need
            p.stream = stream
            _abi.check(lib.fwa2_backward(p), "fwa2_backward")
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
    def forward(ctx, qkv, logit_scale=None, bias=None, mask=None):
        assert qkv.dim() == 5 and qkv.shape[2] == 3, "qkv must be [BW, N, 3, H, d]"
        if not (_rows_16b_aligned(qkv) and qkv.is_contiguous()):
            qkv = qkv.contiguous()
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))       # [BW, H, N, d] views
        if logit_scale is not None:
            assert isinstance(logit_scale, torch.Tensor), \
                "Make sure logit_scale is a tensor if defined in the paramaters."
            scale_type = "tensor"
            logit_scale = logit_scale.contiguous()
        else:
            scale_type = "scalar"
            # placeholder for the saved-tensor slot (the reference keeps 1/sqrt(d) there, fn.py:15-17); the
            # kernels derive the default scale from head_dim, and filling a device scalar from the host
            # would synchronise and break stream capture
            logit_scale = torch.empty((), device=q.device)
        _check_inputs(q, k, v, logit_scale, bias, mask, scale_type)
        if bias is not None and bias.stride(-1) != 1:
            bias = bias.contiguous()
        if mask is not None and mask.stride(-1) != 1:
            mask = mask.contiguous()

        bw, heads, n, d = q.shape
        lib = _abi.load()
        lse = torch.empty((bw, heads, (n + 63) // 64 * 64), device=q.device, dtype=torch.float32)
        out = torch.empty((bw, n, heads, d), device=q.device, dtype=q.dtype)
        mask_live = mask_window_flags(mask) if mask is not None else None
        p = _describe(q, k, v, out.transpose(1, 2), lse, logit_scale, bias, mask, mask_live, scale_type)
        with _on_device(q.device) as stream:
            p.stream = stream
            _abi.check(lib.fwa2_forward(p), "fwa2_forward")

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
        dqkv = torch.empty_like(qkv)
        dq, dk, dv = (dqkv[:, :, i].transpose(1, 2) for i in range(3))
        dscale = torch.empty_like(logit_scale, memory_format=torch.contiguous_format) if scale_type == "tensor" else None
        db = torch.empty_like(bias, memory_format=torch.contiguous_format) if bias is not None else None

        lib = _abi.load()
        p = _describe(q, k, v, out.transpose(1, 2), lse, logit_scale, bias, mask, ctx.mask_live, scale_type)
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
        return dqkv, dscale, db, None


MAPPED_MAX_N = 256      # largest window the library addresses through a window map


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
    def forward(ctx, qkv, grid, window, shift, logit_scale=None, bias=None, mask=None):
        (gh, gw), (wh, ww), (sh, sw) = grid, window, shift
        assert qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.shape[1] == gh * gw, "qkv must be [B, gh * gw, 3, H, d]"
        assert gh % wh == 0 and gw % ww == 0, "the grid must be a whole number of windows"
        if not (_rows_16b_aligned(qkv) and qkv.is_contiguous()):
            qkv = qkv.contiguous()
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))       # [B, H, L, d] views
        if logit_scale is not None:
            assert isinstance(logit_scale, torch.Tensor), \
                "Make sure logit_scale is a tensor if defined in the paramaters."
            scale_type = "tensor"
            logit_scale = logit_scale.contiguous()
        else:
            scale_type = "scalar"
            # placeholder for the saved-tensor slot (the reference keeps 1/sqrt(d) there, fn.py:15-17); the
            # kernels derive the default scale from head_dim, and filling a device scalar from the host
            # would synchronise and break stream capture
            logit_scale = torch.empty((), device=q.device)
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

        lib = _abi.load()
        lse = torch.empty((b * nw, heads, (n + 63) // 64 * 64), device=q.device, dtype=torch.float32)
        out = torch.empty((b, length, heads, d), device=q.device, dtype=q.dtype)
        mask_live = mask_window_flags(mask) if mask is not None else None
        window_map = ((gh, gw), (wh, ww), (sh % gh, sw % gw))
        p = _describe(q, k, v, out.transpose(1, 2), lse, logit_scale, bias, mask, mask_live, scale_type, window_map)
        with _on_device(q.device) as stream:
            p.stream = stream
            _abi.check(lib.fwa2_forward(p), "fwa2_forward")

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
        dqkv = torch.empty_like(qkv)
        dq, dk, dv = (dqkv[:, :, i].transpose(1, 2) for i in range(3))
        dscale = torch.empty_like(logit_scale, memory_format=torch.contiguous_format) if scale_type == "tensor" else None
        db = torch.empty_like(bias, memory_format=torch.contiguous_format) if bias is not None else None

        lib = _abi.load()
        p = _describe(q, k, v, out.transpose(1, 2), lse, logit_scale, bias, mask, ctx.mask_live, scale_type,
                      ctx.window_map)
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
        return dqkv, None, None, None, dscale, db, None


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
