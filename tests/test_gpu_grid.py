"""GPU tests of the window map: the cyclic shift and the window partition / reverse of the reference's
block (flash_win_attn_v2/swin_transformer_v2.py:419-441) done by the kernels' addressing.  The map only
changes which addresses a unit reads and writes, so every result must be bit-identical to the packed
operator run on explicitly rolled and partitioned copies, which the other GPU tests hold against the oracle."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _partition(x, grid, window, shift):
    """[B, gh*gw, ...] -> [B*nW, wh*ww, ...] as roll(-shift) + window_partition do it."""
    (gh, gw), (wh, ww), (sh, sw) = grid, window, shift
    b, rest = x.shape[0], x.shape[2:]
    x = x.reshape(b, gh, gw, *rest)
    x = torch.roll(x, shifts=(-sh, -sw), dims=(1, 2))
    x = x.reshape(b, gh // wh, wh, gw // ww, ww, *rest).transpose(2, 3)
    return x.reshape(b * (gh // wh) * (gw // ww), wh * ww, *rest).contiguous()


def _reverse(x, grid, window, shift):
    """Inverse of `_partition`: window_reverse + roll(+shift)."""
    (gh, gw), (wh, ww), (sh, sw) = grid, window, shift
    rest = x.shape[2:]
    b = x.shape[0] // ((gh // wh) * (gw // ww))
    x = x.reshape(b, gh // wh, gw // ww, wh, ww, *rest).transpose(2, 3).reshape(b, gh, gw, *rest)
    x = torch.roll(x, shifts=(sh, sw), dims=(1, 2))
    return x.reshape(b, gh * gw, *rest).contiguous()


def _inputs(batch, grid, window, heads, d, dtype, seed, with_mask):
    (gh, gw), (wh, ww) = grid, window
    n, nw = wh * ww, (gh // wh) * (gw // ww)
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(batch, gh * gw, 3, heads, d, generator=g).to(dtype).cuda()
    scale = (torch.randn(heads, 1, 1, generator=g) * 0.5 + 2.0).to(dtype).cuda()
    bias = (torch.randn(heads, n, n, generator=g) * 2).to(dtype).cuda()
    mask = None
    if with_mask:
        mask = torch.where(torch.rand(nw, n, n, generator=g) < 0.3, -100.0, 0.0)
        mask[0] = 0                                         # one window with nothing masked, as in Swin
        mask[:, torch.arange(n), torch.arange(n)] = 0       # no fully masked row
        mask = mask.cuda()
    dout = torch.randn(batch, gh * gw, heads, d, generator=g).to(dtype).cuda()
    return qkv, scale, bias, mask, dout


CASES = [
    # batch, grid, window, shift, heads, mask
    (2, (16, 16), (8, 8), (4, 4), 3, True),
    (2, (16, 16), (8, 8), (0, 0), 3, False),
    (3, (8, 24), (4, 8), (2, 3), 2, True),          # non-square window and grid, unequal shifts
    (2, (14, 21), (7, 7), (3, 3), 3, True),         # 49 tokens
    (1, (12, 8), (4, 4), (1, 3), 4, True),
    (2, (8, 8), (8, 8), (0, 0), 3, False),          # one window covers the grid
    (2, (6, 9), (3, 3), (1, 1), 2, True),           # 9 tokens
    (2, (32, 32), (16, 16), (8, 8), 3, True),       # 256 tokens: forward and one-pass backward kernels
    (2, (32, 16), (16, 16), (0, 0), 3, False),
    (2, (24, 36), (12, 12), (6, 6), 3, True),       # 144 tokens: one 16-key tile per wavefront
    (1, (20, 40), (10, 20), (5, 10), 2, True),      # 200 tokens, not a multiple of 16
    (2, (16, 24), (8, 12), (4, 6), 3, True),        # 96 tokens
    (2, (22, 11), (11, 11), (5, 5), 2, True),       # 121 tokens, odd
    (2, (36, 18), (18, 18), (9, 9), 2, True),       # 324 tokens: the streaming kernels, two key-side super-tiles
    (1, (24, 48), (24, 24), (12, 12), 3, True),     # 576 tokens
    (1, (32, 64), (32, 32), (16, 16), 2, False),    # 1024 tokens, the largest mapped window
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"b{c[0]}g{c[1][0]}x{c[1][1]}w{c[2][0]}x{c[2][1]}s{c[3][0]}_{c[3][1]}")
def test_grid_matches_partitioned_call(case, dtype):
    from flash_window_attention_v2_amd import flash_win_attn_v2_grid_func, flash_win_attn_v2_qkvpacked_func
    batch, grid, window, shift, heads, with_mask = case
    qkv, scale, bias, mask, dout = _inputs(batch, grid, window, heads, 32, dtype, 11, with_mask)

    a = qkv.clone().requires_grad_(True)
    scale_a, bias_a = scale.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    o_a = flash_win_attn_v2_grid_func(a, grid, window, shift, scale_a, bias_a, mask)
    assert o_a.shape == (batch, grid[0] * grid[1], heads, 32) and o_a.is_contiguous()
    o_a.backward(dout)

    b = qkv.clone().requires_grad_(True)
    scale_b, bias_b = scale.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    o_w = flash_win_attn_v2_qkvpacked_func(_partition(b, grid, window, shift), scale_b, bias_b, mask)
    o_b = _reverse(o_w, grid, window, shift)
    o_b.backward(dout)

    assert torch.equal(o_a, o_b)
    assert torch.equal(a.grad, b.grad)
    assert torch.equal(bias_a.grad, bias_b.grad)
    assert torch.equal(scale_a.grad, scale_b.grad)


@pytest.mark.parametrize("case", [CASES[2], CASES[7], CASES[13]], ids=["w4x8", "w16x16", "w18x18"])
def test_grid_against_the_classic_oracle(case):
    """The grid operator held directly against the fp32 classic path applied to rolled and partitioned copies
    made on the CPU (roll, window_partition, attention, window_reverse, roll back, as the reference's block
    does them, flash_win_attn_v2/swin_transformer_v2.py:419-441): no product kernel is on the checking side."""
    from oracle.classic_torch import classic_fwd_bwd
    from flash_window_attention_v2_amd import flash_win_attn_v2_grid_func
    batch, grid, window, shift, heads, with_mask = case
    dtype = torch.bfloat16
    qkv, scale, bias, mask, dout = _inputs(batch, grid, window, heads, 32, dtype, 19, with_mask)
    a = qkv.clone().requires_grad_(True)
    scale_a, bias_a = scale.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    o = flash_win_attn_v2_grid_func(a, grid, window, shift, scale_a, bias_a, mask)
    o.backward(dout)

    win = _partition(qkv.cpu(), grid, window, shift)                      # [BW, N, 3, H, d]
    q, k, v = (win[:, :, i].transpose(1, 2) for i in range(3))            # [BW, H, N, d]
    do = _partition(dout.cpu(), grid, window, shift).transpose(1, 2)
    ref = classic_fwd_bwd(q, k, v, scale.cpu(), bias.cpu(), None if mask is None else mask.cpu(), do)
    back = lambda t: _reverse(t.transpose(1, 2).contiguous(), grid, window, shift)      # -> [B, L, H, d]
    o_ref = back(ref["o"])
    dqkv_ref = torch.stack([back(ref[g]) for g in ("dq", "dk", "dv")], dim=2)
    assert float((o.detach().float().cpu() - o_ref).abs().max()) <= 2e-2
    for i, g in enumerate(("dq", "dk", "dv")):
        got, want = a.grad[:, :, i].float().cpu(), dqkv_ref[:, :, i]
        assert float((got - want).abs().max() / want.abs().max()) <= 5e-2, g
    assert float((bias_a.grad.float().cpu() - ref["dbias"]).abs().max() / ref["dbias"].abs().max()) <= 5e-2
    want = ref["dscale"].flatten()
    slack = torch.maximum(want.abs(), 0.02 * ref["dscale_l1"])
    assert bool(((scale_a.grad.float().cpu().flatten() - want).abs() <= 5e-2 * slack).all())


@pytest.mark.parametrize("d", [16, 64, 128])
@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES[7]], ids=["w8x8", "w4x8", "w16x16"])
def test_grid_with_other_head_dimensions(case, d):
    """The window map on the plain kernels that serve head dimensions other than 32."""
    from flash_window_attention_v2_amd import flash_win_attn_v2_grid_func, flash_win_attn_v2_qkvpacked_func
    batch, grid, window, shift, heads, with_mask = case
    qkv, scale, bias, mask, dout = _inputs(batch, grid, window, heads, d, torch.bfloat16, 17, with_mask)
    a = qkv.clone().requires_grad_(True)
    scale_a, bias_a = scale.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    flash_win_attn_v2_grid_func(a, grid, window, shift, scale_a, bias_a, mask).backward(dout)
    b = qkv.clone().requires_grad_(True)
    scale_b, bias_b = scale.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    o_w = flash_win_attn_v2_qkvpacked_func(_partition(b, grid, window, shift), scale_b, bias_b, mask)
    _reverse(o_w, grid, window, shift).backward(dout)
    assert torch.equal(a.grad, b.grad)
    assert torch.equal(bias_a.grad, bias_b.grad) and torch.equal(scale_a.grad, scale_b.grad)


def test_grid_rejects_windows_longer_than_1024_tokens():
    """The map's row arithmetic covers windows of up to 1024 tokens: beyond that the library must say so
    instead of computing on wrong addresses."""
    from flash_window_attention_v2_amd import flash_win_attn_v2_grid_func
    qkv, scale, bias, mask, _ = _inputs(1, (36, 72), (36, 36), 2, 32, torch.bfloat16, 12, False)
    with pytest.raises(NotImplementedError, match="window map"):
        flash_win_attn_v2_grid_func(qkv, (36, 72), (36, 36), (18, 18), scale, bias, mask)


def test_grid_argument_errors():
    from flash_window_attention_v2_amd import _abi, flash_win_attn_v2_grid_func
    qkv, scale, bias, mask, _ = _inputs(2, (16, 16), (8, 8), 3, 32, torch.bfloat16, 13, True)
    with pytest.raises(AssertionError):
        flash_win_attn_v2_grid_func(qkv, (16, 16), (5, 8), (0, 0), scale, bias, mask)       # 16 % 5
    with pytest.raises(AssertionError):
        flash_win_attn_v2_grid_func(qkv, (16, 8), (8, 8), (0, 0), scale, bias, mask)        # L != gh * gw
    with pytest.raises(AssertionError):
        flash_win_attn_v2_grid_func(qkv, (16, 16), (8, 8), (0, 0), scale, bias, mask[:2])   # mask windows
    # a shift outside [0, extent) is reduced modulo the grid, as torch.roll does
    o1 = flash_win_attn_v2_grid_func(qkv, (16, 16), (8, 8), (4 + 16, 4 - 16), scale, bias, mask)
    o2 = flash_win_attn_v2_grid_func(qkv, (16, 16), (8, 8), (4, 4), scale, bias, mask)
    assert torch.equal(o1, o2)
