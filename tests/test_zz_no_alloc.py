"""fwa2_backward_static, the backward entry point that allocates nothing: called through the C ABI
and compared with fwa2_backward (caller-owned workspace) on the same inputs, twice in a row with the
second problem smaller than the first, so that whatever the first call left in the library's static
scratch is what the second one starts from."""
import ctypes

import pytest
import torch

from flash_window_attention_v2_amd import _abi, kernels
from oracle.classic_torch import classic_fwd_bwd
from oracle.swin_inputs import make_inputs

pytestmark = pytest.mark.gpu


def _backward_through(entry, dev, o, lse, workspace):
    """dq, dk, dv, dbias, dscale of one call of `entry` (a libfwa2 backward entry point)."""
    q, k, v = dev["q"], dev["k"], dev["v"]
    grads = [torch.full_like(t, float("nan")) for t in (q, k, v, dev["bias"], dev["logit_scale"])]
    p = kernels._describe(q, k, v, o, lse, dev["logit_scale"], dev["bias"], dev["mask"],
                          kernels._flags_for(dev["mask"]), "tensor")
    kernels._set_t4(p.d_o, dev["do"])
    for dst, t in zip((p.dq, p.dk, p.dv), grads):
        kernels._set_t4(dst, t)
    p.dbias, p.dscale = grads[3].data_ptr(), grads[4].data_ptr()
    if workspace is not None:
        p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel()
    p.stream = torch.cuda.current_stream().cuda_stream
    _abi.check(entry(ctypes.byref(p)), "backward")
    torch.cuda.synchronize()
    return grads


def _case(lib, batch, n_windows, heads, n, resolution, window, shift, dtype, seed):
    inp = make_inputs(batch=batch, n_windows=n_windows, heads=heads, n=n, d=32, dtype=dtype, seed=seed,
                      resolution=resolution, window=window, shift=shift)
    dev = {k: (None if v is None else v.cuda()) for k, v in inp.items()}
    o, lse, _ = kernels._flash_attn_forward(dev["q"], dev["k"], dev["v"], dev["logit_scale"], dev["bias"], dev["mask"],
                                            scale_type="tensor")
    p = kernels._describe(dev["q"], dev["k"], dev["v"], o, lse, dev["logit_scale"], dev["bias"], dev["mask"], None, "tensor")
    need = lib.fwa2_backward_workspace_bytes(ctypes.byref(p))
    assert 0 < need <= _abi.STATIC_SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = _backward_through(lib.fwa2_backward, dev, o, lse, ws)
    # the allocation-free call: no workspace passed, and torch's allocator must not see a request either
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    got = _backward_through(lib.fwa2_backward_static, dev, o, lse, None)
    # the five gradient tensors the caller passes in, and nothing else
    assert torch.cuda.memory_stats()["allocation.all.allocated"] - before == 5
    for name, a, b in zip(("dq", "dk", "dv", "dbias", "dscale"), got, want):
        assert torch.isfinite(a.float()).all(), name
        assert torch.equal(a, b), f"{name}: static-scratch call differs from fwa2_backward, max abs diff " \
                                  f"{float((a.float() - b.float()).abs().max())}"
    # ... and both agree with the fp32 classic oracle within the operator's tolerances
    ref = classic_fwd_bwd(inp["q"], inp["k"], inp["v"], inp["logit_scale"], inp["bias"], inp["mask"], inp["do"])
    tol = 5e-2 if dtype == torch.bfloat16 else 2e-2
    for name, a in zip(("dq", "dk", "dv", "dbias", "dscale"), got):
        rel = float((a.float().cpu() - ref[name]).abs().max() / ref[name].abs().max())
        assert rel <= tol, f"{name}: relative error {rel} against the oracle"


def test_static_scratch_backward_matches_workspace_backward_twice():
    lib = _abi.load()
    # first windows of 256 tokens with a 16-window mask (the one-pass backward with its score tables; about
    # 77 MiB of scratch on a 256-CU part) ...
    _case(lib, batch=4, n_windows=16, heads=3, n=256, resolution=64, window=16, shift=8, dtype=torch.bfloat16, seed=11)
    # ... then a smaller problem on the fused kernel, which finds the first call's leftovers in the scratch
    _case(lib, batch=2, n_windows=4, heads=2, n=64, resolution=16, window=8, shift=4, dtype=torch.float16, seed=12)
    # ... and once more the larger shape class at 144 tokens (padded tiles, other offsets into the scratch)
    _case(lib, batch=2, n_windows=4, heads=2, n=144, resolution=24, window=12, shift=6, dtype=torch.bfloat16, seed=13)


def test_static_scratch_backward_refuses_what_does_not_fit():
    lib = _abi.load()
    inp = make_inputs(batch=1, n_windows=4, heads=2, n=64, d=32, dtype=torch.bfloat16, seed=0, resolution=16, window=8,
                      shift=4)
    dev = {k: (None if v is None else v.cuda()) for k, v in inp.items()}
    o, lse, _ = kernels._flash_attn_forward(dev["q"], dev["k"], dev["v"], dev["logit_scale"], dev["bias"], dev["mask"],
                                            scale_type="tensor")
    p = kernels._describe(dev["q"], dev["k"], dev["v"], o, lse, dev["logit_scale"], dev["bias"], dev["mask"], None, "tensor")
    # the same pointers described as 256 windows of 576 tokens: refused on its size before anything is launched
    p.bw, p.heads, p.n, p.n_windows = 256, 6, 576, 4
    for t in (p.q, p.k, p.v, p.o):
        t.stride_bw, t.stride_h, t.stride_n = 6 * 576 * 32, 576 * 32, 32
    p.bias.stride_a = p.mask.stride_a = 576 * 576
    p.bias.stride_n = p.mask.stride_n = 576
    p.lse_stride_bw, p.lse_stride_h = 6 * 576, 576
    assert lib.fwa2_backward_workspace_bytes(ctypes.byref(p)) > _abi.STATIC_SCRATCH_BYTES
    with pytest.raises(NotImplementedError, match="static buffer holds"):
        _abi.check(lib.fwa2_backward_static(ctypes.byref(p)), "fwa2_backward_static")
    torch.cuda.synchronize()
