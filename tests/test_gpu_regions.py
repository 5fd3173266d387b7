"""GPU tests of the region form of a mask: the scan that recognises mask = c * [id_i != id_j] (what the reference's
builder produces, flash_win_attn_v2/swin_transformer_v2.py:386-405) and the forward path that rebuilds such a mask
from N ids per window instead of reading N x N entries.  The scan must accept exactly that form and nothing else,
so that every other mask keeps being read entry by entry."""
import ctypes
import math

import numpy as np
import pytest
import torch

from oracle.classic_torch import classic_fwd_bwd
from oracle.swin_inputs import make_inputs, shifted_window_mask

pytestmark = pytest.mark.gpu


def _scan(mask):
    """(flags [nW], value [nW], count [nW], ids [nW, 256]) as the library's scan reports them."""
    from flash_window_attention_v2_amd import _abi, kernels
    lib = _abi.load()
    nw, n = mask.shape[0], mask.shape[1]
    live = torch.zeros(nw, dtype=torch.uint8, device="cuda")
    regions = torch.zeros(nw * _abi.MASK_REGION_BYTES, dtype=torch.uint8, device="cuda")
    st = lib.fwa2_mask_scan_regions(mask.data_ptr(), kernels._DTYPES[mask.dtype], nw, n, mask.stride(0), mask.stride(1),
                                    live.data_ptr(), regions.data_ptr(), None)
    _abi.check(st, "fwa2_mask_scan_regions")
    torch.cuda.synchronize()
    rec = regions.cpu().numpy().reshape(nw, _abi.MASK_REGION_BYTES)
    value = rec[:, 0:4].copy().view(np.float32)[:, 0]
    count = rec[:, 4:8].copy().view(np.int32)[:, 0]
    return live.cpu().numpy(), value, count, rec[:, 16:]


def _mask_from_ids(ids, value, dtype):
    ids = torch.as_tensor(ids)
    return torch.where(ids[:, :, None] != ids[:, None, :], value, 0.0).to(dtype)


@pytest.mark.parametrize("res,win,shift", [(32, 8, 4), (64, 16, 8), (48, 12, 6), (28, 14, 7), (64, 16, 3)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_scan_recognises_shifted_window_masks(res, win, shift, dtype):
    mask = shifted_window_mask(res, win, shift).to(dtype).cuda()
    flags, value, count, ids = _scan(mask)
    n = win * win
    m = mask.float().cpu()
    for w in range(mask.shape[0]):
        if not bool((m[w] != 0).any()):
            assert flags[w] == 0
            continue
        assert flags[w] == 7 and value[w] == -100.0 and 2 <= count[w] <= 4
        rebuilt = _mask_from_ids(ids[w:w + 1, :n].astype(np.int64), -100.0, torch.float32)[0]
        assert torch.equal(rebuilt, m[w])
        # ids number the regions in order of their first token
        first_seen = [int(np.argmax(ids[w, :n] == r)) for r in range(count[w])]
        assert first_seen == sorted(first_seen) and ids[w, 0] == 0 and ids[w, :n].max() == count[w] - 1


def test_scan_rejects_everything_else():
    n, nw = 64, 12
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 4, (nw, n), generator=g)
    base = _mask_from_ids(ids, -100.0, torch.float32)
    masks = base.clone()
    masks[1, 5, 9] = -100.0 if masks[1, 5, 9] == 0 else 0.0          # one entry off the form (breaks symmetry)
    masks[2] = torch.where(torch.rand(n, n, generator=g) < 0.3, -100.0, 0.0)    # dense random
    masks[2].fill_diagonal_(0)
    masks[3] = _mask_from_ids(ids[3:4], 100.0, torch.float32)[0]      # positive value: may not only remove keys
    masks[4] = _mask_from_ids(ids[4:5], -float("inf"), torch.float32)[0]
    nine = torch.arange(n) % 9                                         # nine regions: one too many
    masks[5] = _mask_from_ids(nine[None], -100.0, torch.float32)[0]
    eight = torch.arange(n) % 8                                        # eight regions: the most a record holds
    masks[6] = _mask_from_ids(eight[None], -100.0, torch.float32)[0]
    masks[7] = base[7] * 0                                             # all zero
    two = base[8].clone()
    two[two != 0] = torch.where(torch.rand(int((two != 0).sum()), generator=g) < 0.5, -100.0, -50.0)   # two values
    masks[8] = two
    masks[9] = _mask_from_ids(ids[9:10], -1e6, torch.float32)[0]       # too large for the fp16 operand
    masks[10] = _mask_from_ids(ids[10:11], -0.375, torch.float32)[0]   # a soft mask is fine
    masks[11, 3, 3] = -100.0                                           # non-zero diagonal
    flags, value, count, rec_ids = _scan(masks.cuda())
    want = {0: 7, 1: 3, 2: 3, 3: 1, 4: 3, 5: 3, 6: 7, 7: 0, 8: 3, 9: 3, 10: 7, 11: 3}
    assert {w: int(flags[w]) for w in want} == want
    assert count[6] == 8 and value[10] == -0.375
    assert np.array_equal(rec_ids[6, :n], eight.numpy())


@pytest.mark.parametrize("n", [64, 144, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_forward_from_region_records(n, dtype, monkeypatch):
    """Random labellings with up to 8 regions and a soft value (so that masked keys keep weight and an error in the
    rebuilt term would show), one all-zero window and one window off the form: the forward output must match the
    fp32 classic path on the dense mask, and the run that reads the dense mask instead."""
    from flash_window_attention_v2_amd import flash_win_attn_v2_func, kernels
    win = int(math.isqrt(n))
    nw = 6
    inp = make_inputs(batch=3, n_windows=nw, heads=2, n=n, dtype=dtype, seed=60 + n, with_mask=False)
    g = torch.Generator().manual_seed(n)
    ids = torch.stack([torch.randint(0, r, (n,), generator=g) for r in (2, 4, 8, 3, 1, 5)])
    value = -2.625
    mask = _mask_from_ids(ids, value, torch.float32)
    mask[5, 1, 2] = value if mask[5, 1, 2] == 0 else 0.0               # window 5 is not of the form
    inp["mask"] = mask.to(dtype)
    flags, _, count, _ = _scan(inp["mask"].cuda())
    assert list(flags) == [7, 7, 7, 7, 0, 3] and list(count[:4]) == [2, 4, 8, 3]
    ref = classic_fwd_bwd(inp["q"], inp["k"], inp["v"], inp["logit_scale"], inp["bias"], inp["mask"], inp["do"])
    dev = {k: (None if v is None else v.cuda()) for k, v in inp.items()}
    with torch.no_grad():
        o = flash_win_attn_v2_func(dev["q"], dev["k"], dev["v"], dev["logit_scale"], dev["bias"], dev["mask"])
        monkeypatch.setattr(kernels, "_flags_for", lambda m: None)     # every window read entry by entry
        o_dense = flash_win_attn_v2_func(dev["q"], dev["k"], dev["v"], dev["logit_scale"], dev["bias"], dev["mask"])
    tol = 2e-2 if dtype == torch.bfloat16 else 5e-3
    err = float((o.float().cpu() - ref["o"]).abs().max())
    err_dense = float((o_dense.float().cpu() - ref["o"]).abs().max())
    assert err <= tol and err <= 1.5 * err_dense + 1e-3, (err, err_dense)
    assert float((o.float() - o_dense.float()).abs().max()) <= tol


def test_region_units_beyond_the_gap_limit_take_the_exact_maximum():
    """With a wide bias range the row bound, which ignores the mask, may sit far above the largest logit of a
    region unit: those units must then find the exact maximum instead of trusting the bound."""
    from flash_window_attention_v2_amd import flash_win_attn_v2_func
    n, dtype = 256, torch.bfloat16
    inp = make_inputs(batch=2, n_windows=4, heads=2, n=n, dtype=dtype, seed=77, resolution=32, window=16, shift=8)
    g = torch.Generator().manual_seed(3)
    inp["bias"] = (torch.randn(2, n, n, generator=g) * 30).to(dtype)   # range far beyond the limit of 96 / log2 e
    ref = classic_fwd_bwd(inp["q"], inp["k"], inp["v"], inp["logit_scale"], inp["bias"], inp["mask"], inp["do"])
    dev = {k: (None if v is None else v.cuda()) for k, v in inp.items()}
    with torch.no_grad():
        o = flash_win_attn_v2_func(dev["q"], dev["k"], dev["v"], dev["logit_scale"], dev["bias"], dev["mask"])
    assert torch.isfinite(o).all()
    assert float((o.float().cpu() - ref["o"]).abs().max()) <= 2e-2
