"""GPU parity for head dimensions other than 32: the reference supports any head dimension up to 128
(flash_win_attn_v2/kernels/attn_kernel_forward.py:267, 298).  Same oracle, same tolerances as the d = 32 tests
(bf16: max abs 2e-2 on o, 5e-2 relative on every gradient; fp16: 5e-3 / 2e-2)."""
import pytest
import torch

from oracle.swin_inputs import make_inputs
from tests.test_gpu_parity import _run_and_check

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("d", [8, 16, 24, 48, 64, 96, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dims_with_shift_mask(d, dtype):
    inp = make_inputs(batch=2, n_windows=4, heads=3, n=64, d=d, dtype=dtype, seed=d, resolution=16, window=8, shift=4)
    _run_and_check(inp, dtype, tag=f"d{d}")


@pytest.mark.parametrize("n,res,win,shift", [(49, 14, 7, 3), (144, 24, 12, 6), (256, 32, 16, 8), (16, 8, 4, 2)])
@pytest.mark.parametrize("d", [16, 64, 128])
def test_head_dims_across_window_sizes(n, res, win, shift, d):
    nw = (res // win) ** 2
    inp = make_inputs(batch=2, n_windows=nw, heads=2, n=n, d=d, dtype=torch.bfloat16, seed=n + d, resolution=res,
                      window=win, shift=shift)
    _run_and_check(inp, torch.bfloat16, tag=f"N{n}d{d}")


@pytest.mark.parametrize("with_scale,with_bias,with_mask", [(0, 1, 1), (1, 0, 1), (1, 1, 0), (0, 0, 0)])
def test_head_dim_64_optional_arguments(with_scale, with_bias, with_mask):
    inp = make_inputs(batch=2, n_windows=4, heads=2, n=64, d=64, dtype=torch.bfloat16, seed=5, resolution=16, window=8,
                      shift=4, with_scale=bool(with_scale), with_bias=bool(with_bias), with_mask=bool(with_mask))
    _run_and_check(inp, torch.bfloat16, tag=f"opt{with_scale}{with_bias}{with_mask}")


def test_head_dim_64_ragged_window_fp32_mask_and_clamped_scale():
    """N = 37 (not a multiple of anything), fp32 mask next to bf16 inputs, many units per dbias group, and a
    logit scale above ln 100, whose gradient must be exactly zero."""
    inp = make_inputs(batch=70, n_windows=1, heads=2, n=37, d=64, dtype=torch.bfloat16, seed=8, with_mask=False)
    g = torch.Generator().manual_seed(9)
    inp["mask"] = torch.where(torch.rand(1, 37, 37, generator=g) < 0.3, -100.0, 0.0)  # fp32
    inp["logit_scale"][1] = 5.0
    _run_and_check(inp, torch.bfloat16, tag="ragged", dscale_l1_frac=0.1)


@pytest.mark.parametrize("d,with_scale", [(20, True), (20, False), (12, False), (36, True), (100, False), (5, True)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dims_that_are_not_multiples_of_8(d, with_scale, dtype):
    """Any head dimension up to 128 (attn_kernel_forward.py:267, 298): the launchers run these on zero-padded
    rows.  Without a logit scale the default 1/sqrt(d) must keep referring to the true d, not to the padded one
    (d = 12 padded to 16 would otherwise be off by 13 % in every logit)."""
    inp = make_inputs(batch=2, n_windows=4, heads=2, n=64, d=d, dtype=dtype, seed=d, resolution=16, window=8, shift=4,
                      with_scale=with_scale)
    _run_and_check(inp, dtype, tag=f"d{d}")


def test_the_library_itself_takes_multiples_of_8_only():
    """Below the Python launchers the C ABI refuses such a head dimension instead of reading past the rows."""
    from flash_window_attention_v2_amd import _abi
    from tests.test_abi import _good_problem
    lib = _abi.load()
    p = _good_problem()
    p.head_dim = 20
    assert lib.fwa2_validate(p, 0) == _abi.ERR_UNSUPPORTED and b"multiples of 8" in lib.fwa2_last_error()


@pytest.mark.parametrize("nq,nk,d", [(64, 96, 32), (100, 49, 32), (49, 128, 64), (300, 64, 32), (37, 290, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_more_or_fewer_keys_than_queries(nq, nk, d, dtype):
    """The reference's kernels take k / v with a row count of their own (attn_kernel_forward.py:263-264):
    bias is [H, Nq, Nk], mask [nW, Nq, Nk], dk / dv follow k / v.  300 queries and 290 keys also cross the
    bound up to which dbias is summed inside the dq pass."""
    from oracle.classic_torch import classic_fwd_bwd
    from tests.test_gpu_parity import TOL, _rel
    from flash_window_attention_v2_amd import flash_win_attn_v2_func
    bw, heads, nw = 6, 2, 3
    g = torch.Generator().manual_seed(nq + nk)
    rnd = lambda *s: torch.randn(*s, generator=g)
    q, do = rnd(bw, heads, nq, d).to(dtype), rnd(bw, heads, nq, d).to(dtype)
    k, v = rnd(bw, heads, nk, d).to(dtype), rnd(bw, heads, nk, d).to(dtype)
    bias = (16 * torch.sigmoid(rnd(heads, nq, nk))).to(dtype)
    scale = torch.full((heads, 1, 1), 2.3).to(dtype)
    mask = torch.where(torch.rand(nw, nq, nk, generator=g) < 0.3, -100.0, 0.0)
    mask[0] = 0
    mask[:, :, 0] = 0                                   # every row keeps a key
    mask = mask.to(dtype)
    ref = classic_fwd_bwd(q, k, v, scale, bias, mask, do)

    dq_, dk_, dv_, ds_, db_ = (t.cuda().requires_grad_() for t in (q, k, v, scale, bias))
    o = flash_win_attn_v2_func(dq_, dk_, dv_, ds_, db_, mask.cuda())
    assert o.shape == (bw, heads, nq, d)
    o.backward(do.cuda())
    tol_o, tol_g = TOL[dtype]
    assert float((o.detach().float().cpu() - ref["o"]).abs().max()) <= tol_o
    assert dk_.grad.shape == k.shape and dv_.grad.shape == v.shape and db_.grad.shape == bias.shape
    for got, name in ((dq_, "dq"), (dk_, "dk"), (dv_, "dv"), (db_, "dbias")):
        assert _rel(got.grad, ref[name]) <= tol_g, name
    diff = (ds_.grad.float().cpu().flatten() - ref["dscale"].float().cpu().flatten()).abs()
    bound = torch.maximum(ref["dscale"].float().cpu().flatten().abs().max().expand_as(diff),
                          0.1 * ref["dscale_l1"].float().cpu().flatten())
    assert bool((diff <= tol_g * bound).all())
