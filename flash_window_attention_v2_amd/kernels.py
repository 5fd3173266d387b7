"""Host launchers under the reference's names: `_flash_attn_forward` and `_flash_attn_backward`
(flash_win_attn_v2/kernels/attn_kernel_forward.py:261-345, attn_kernel_backward.py:567-711), with the same
arguments, returns and in-place gradient outputs, whose bodies describe the problem to libfwa2.so (raw device
pointers and strides) instead of launching Triton kernels.  The helpers the three autograd Functions share
live here as well.

Every buffer -- outputs, log-sum-exp, gradients and the backward workspace -- is a torch tensor allocated on
this side, so torch's allocator statistics stay honest and the C side allocates nothing.
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
    """What the kernels address directly: unit inner stride, rows on 16-byte boundaries, and a row stride small
    enough for the 32-bit offsets they use inside one unit (below 2^24 elements, rows x stride below 2^30)."""
    st = t.stride()
    if len(st) == 4:            # q, k, v, o and their gradients: no generator in the way
        s0, s1, s2, s3 = st
        return (s3 == 1 and (s0 | s1 | s2) % 8 == 0 and t.data_ptr() % 16 == 0 and s2 < (1 << 24)
                and t.shape[2] * s2 < (1 << 30))
    return (st[-1] == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in st[:-1])
            and st[-2] < (1 << 24) and t.shape[-2] * st[-2] < (1 << 30))


def _kernel_ready(t):
    """Unit inner stride is the reference's requirement (flash_window_attention_v2.py:20);
    16-byte-aligned rows are this library's: copy only when either fails."""
    return t if _rows_16b_aligned(t) else t.contiguous()


def tensor_version(t):
    """The in-place modification counter of `t`, or None for a tensor created under torch.inference_mode,
    which keeps none (asking for it raises)."""
    return None if t.is_inference() else t._version


def mask_window_flags(mask):
    """uint8[nW] device tensor of per-window flags: 0 where a window's mask is all zero, bit 0 where it has a
    non-zero entry, bit 1 where it only removes keys and never a whole row, bit 2 where it is exactly
    c * [id_i != id_j] (what the reference's builder produces, swin_transformer_v2.py:386-405).  For the last
    kind the scan also fills one record per window (c and the N ids), kept on the returned tensor as
    `_fwa2_regions` and handed to the library with the flags.
    Cached on the mask tensor object, keyed by its storage address and in-place modification counter, so a
    mask edited in place or re-pointed at other memory (`mask.data = ...`) is scanned again.  Two cases are
    never cached and scan on every call: a mask created under torch.inference_mode, which tracks no
    modifications, and a first scan made while a graph is being captured, whose flags live in the graph's
    own memory pool and must not be handed to eager calls (scan once eagerly before capturing to avoid the
    extra node).  A caller that owns such a mask and never edits it (the Swin block and its `attn_mask` buffer)
    scans it once itself and hands the flags to the packed operators (`mask_flags=`).
    The region records only serve windows of up to 256 tokens; longer windows get the plain scan."""
    version = tensor_version(mask)
    key = (version, mask.data_ptr(), mask.device)
    cached = getattr(mask, "_fwa2_live", None)
    if version is not None and cached is not None and cached[0] == key:
        return cached[1]
    lib = _abi.load()
    live = torch.empty(mask.shape[0], dtype=torch.uint8, device=mask.device)
    if mask.shape[1] <= 256:
        regions = torch.empty(mask.shape[0] * _abi.MASK_REGION_BYTES, dtype=torch.uint8, device=mask.device)
        with _on_device(mask.device) as stream:
            st = lib.fwa2_mask_scan_regions(mask.data_ptr(), _DTYPES[mask.dtype], mask.shape[0], mask.shape[1],
                                            mask.stride(0), mask.stride(1), live.data_ptr(), regions.data_ptr(), stream)
        _abi.check(st, "fwa2_mask_scan_regions")
        live._fwa2_regions = regions
    else:
        with _on_device(mask.device) as stream:
            st = lib.fwa2_mask_scan(mask.data_ptr(), _DTYPES[mask.dtype], mask.shape[0], mask.shape[1],
                                    mask.stride(0), mask.stride(1), live.data_ptr(), stream)
        _abi.check(st, "fwa2_mask_scan")
    if version is not None and not torch.cuda.is_current_stream_capturing():
        try:
            mask._fwa2_live = (key, live)
        except Exception:
            pass
    return live


def _rows_of_8(t, cache):
    """`t` ([A, N, N], N not a multiple of 8) with rows padded to the next multiple of 8 entries.  With `cache`
    the copy is kept on the tensor object under the same rules as the mask flags (a mask is the same tensor call
    after call; a bias is rebuilt every step)."""
    if t is None or t.shape[-1] % 8 == 0:
        return t
    version = tensor_version(t) if cache else None
    key = (version, t.data_ptr(), t.device)
    if version is not None:
        cached = getattr(t, "_fwa2_rows8", None)
        if cached is not None and cached[0] == key:
            return cached[1]
    padded = torch.nn.functional.pad(t, (0, -t.shape[-1] % 8))
    if version is not None and not torch.cuda.is_current_stream_capturing():
        try:
            t._fwa2_rows8 = (key, padded)
        except Exception:
            pass
    return padded


def _describe(q, k, v, o, lse, logit_scale, bias, mask, mask_live, scale_type, window_map=None, scale_dim=0):
    bw, heads, n, d = q.shape
    p = _abi.new_problem()
    p.scale_head_dim = scale_dim
    # whatever the description points at stays alive with it: the flags and region records may be temporaries
    # (an uncached scan), and a later allocation must not land on their memory before the launch has been queued
    p._keep = (mask_live, getattr(mask_live, "_fwa2_regions", None))
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
    if 64 < n <= 256 and n % 8 and p.n_keys == 0:
        # Windows such as 14 x 14 tokens: rows of bias and mask start off 16-byte boundaries, which would put the
        # resident-tile kernels on element-wise loads.  Copies with rows padded to a multiple of 8 entries keep
        # them on 16-byte loads; the kernels never use the entries beyond n.  The copies live as long as the
        # problem description (the launch that follows is ordered behind them on the same stream).
        bias, mask = _rows_of_8(bias, cache=False), _rows_of_8(mask, cache=True)
        p._keep = p._keep + (bias, mask)
    if bias is not None:
        p.bias.ptr, p.bias.stride_a, p.bias.stride_n = bias.data_ptr(), bias.stride(0), bias.stride(1)
    if mask is not None:
        p.mask.ptr, p.mask.stride_a, p.mask.stride_n = mask.data_ptr(), mask.stride(0), mask.stride(1)
        p.mask_dtype = _DTYPES[mask.dtype]
        if mask_live is not None:
            p.mask_live = mask_live.data_ptr()
            regions = getattr(mask_live, "_fwa2_regions", None)
            if regions is not None:
                p.mask_regions = regions.data_ptr()
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


def _pad8(x):
    """Rows padded with zeros to the next multiple of 8 elements (a new contiguous tensor)."""
    return torch.nn.functional.pad(x, (0, -x.shape[-1] % 8))


def _flash_attn_forward(q, k, v, logit_scale, bias=None, mask=None, scale_type="scalar", _scale_dim=0, _events=None):
    """(o, lse, logit_scale) as the reference's launcher returns them (attn_kernel_forward.py:261-345):
    o like q, lse fp32 [BW, H, ceil(N / 64) * 64] holding the natural-log normaliser of every query row.
    A head dimension that is not a multiple of 8 runs on zero-padded copies (the reference pads inside its
    kernels, attn_kernel_forward.py:267,298): zero columns change neither the norms nor the products, and the
    default scale keeps referring to the true dimension.
    `_events`: an optional pair of raw hipEvent_t handles that the library records on the stream around the
    kernels of this call (a measurement hook without a counterpart in the reference)."""
    _check_inputs(q, k, v, logit_scale, bias, mask, scale_type)
    d = q.shape[-1]
    if d % 8:
        o, lse, logit_scale = _flash_attn_forward(_pad8(q), _pad8(k), _pad8(v), logit_scale, bias, mask, scale_type, d,
                                                  _events)
        return o[..., :d].contiguous(), lse, logit_scale
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
    if bw == 0:         # nothing to launch: the classic path returns an empty output here too
        return o, lse, logit_scale
    if not _rows_16b_aligned(o):
        o = torch.empty(q.shape, device=q.device, dtype=q.dtype)
    p = _describe(q, k, v, o, lse, logit_scale, bias, mask, _flags_for(mask), scale_type, scale_dim=_scale_dim)
    if _events is not None:
        p.ev_start, p.ev_stop = _events
    with _on_device(q.device) as stream:
        p.stream = stream
        _abi.check(lib.fwa2_forward(p), "fwa2_forward")
    return o, lse, logit_scale


def _flash_attn_backward(do, q, k, v, logit_scale, o, lse, dq, dk, dv, dscale, db, bias=None, mask=None,
                         scale_type="scalar", _scale_dim=0, _events=None):
    """Fills dq, dk, dv (and dscale, db when given) in place, as the reference's launcher does
    (attn_kernel_backward.py:567-711); dscale already carries the clamp mask (l <= ln 100).
    `_events`: an optional pair of raw hipEvent_t handles recorded around the main backward kernel of this call."""
    if q.shape[0] == 0:     # an empty batch: the sums over units are empty
        for t in (db, dscale):
            if t is not None:
                t.zero_()
        return
    d = q.shape[-1]
    if d % 8:               # zero-padded copies, as in the forward; the gradients of the pad columns are dropped
        padded = [_pad8(x) for x in (do, q, k, v, o)]
        grads = [torch.empty_like(padded[i]) for i in (1, 2, 3)]
        _flash_attn_backward(padded[0], padded[1], padded[2], padded[3], logit_scale, padded[4], lse, *grads, dscale, db,
                             bias=bias, mask=mask, scale_type=scale_type, _scale_dim=d, _events=_events)
        for given, used in zip((dq, dk, dv), grads):
            given.copy_(used[..., :d])
        return
    do, q, k, v, o = (_kernel_ready(x) for x in (do, q, k, v, o))
    if bias is not None and bias.stride(-1) != 1:
        bias = bias.contiguous()
    if mask is not None and mask.stride(-1) != 1:
        mask = mask.contiguous()
    # gradient buffers the kernels cannot write directly (rows off 16-byte boundaries, strided dbias)
    # are filled through a compact temporary
    outs = []
    for t in (dq, dk, dv):
        outs.append(t if _rows_16b_aligned(t) else torch.empty(t.shape, device=t.device, dtype=t.dtype))
    db_k = db if db is None or db.is_contiguous() else torch.empty(db.shape, device=db.device, dtype=db.dtype)
    ds_k = dscale if dscale is None or dscale.is_contiguous() else torch.empty(dscale.shape, device=dscale.device,
                                                                               dtype=dscale.dtype)
    lib = _abi.load()
    p = _describe(q, k, v, o, lse, logit_scale, bias, mask, _flags_for(mask), scale_type, scale_dim=_scale_dim)
    _set_t4(p.d_o, do); _set_t4(p.dq, outs[0]); _set_t4(p.dk, outs[1]); _set_t4(p.dv, outs[2])
    if db_k is not None:
        p.dbias = db_k.data_ptr()
    if ds_k is not None and scale_type == "tensor":
        p.dscale = ds_k.data_ptr()
    if _events is not None:
        p.ev_start, p.ev_stop = _events
    with _on_device(q.device) as stream:
        need = lib.fwa2_backward_workspace_bytes(p)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=q.device)
        p.workspace, p.workspace_bytes = ws.data_ptr(), need
        p.stream = stream
        _abi.check(lib.fwa2_backward(p), "fwa2_backward")
    for given, used in zip((dq, dk, dv, db, dscale), (*outs, db_k, ds_k)):
        if given is not None and used is not given:
            given.copy_(used)


def _flags_for(mask):
    """The per-window flags of a square mask (the scan covers those); None otherwise."""
    return mask_window_flags(mask) if mask is not None and mask.shape[1] == mask.shape[2] else None
