"""Host-side layout decisions of the launchers (no GPU): which tensors the kernels address directly, which are
copied, and how bias / mask rows of odd window lengths are padded."""
import torch

from flash_window_attention_v2_amd import kernels


def test_rows_the_kernels_address_directly():
    ok = kernels._rows_16b_aligned
    a = torch.empty(4, 3, 64, 32, dtype=torch.bfloat16)
    assert ok(a)
    assert ok(a[:, :, ::2])                                # a row stride of 64 elements
    assert ok(a.transpose(1, 2))                           # [B, N, H, d] viewed as [B, H, N, d]: inner stride still 1
    assert ok(torch.empty(4, 3, 64, 40, dtype=torch.bfloat16)[..., :32])       # padded rows, 80 bytes apart
    assert not ok(a[..., 1:])                              # rows start 2 bytes off a 16-byte boundary
    assert not ok(a.transpose(2, 3))                       # inner stride 64
    assert not ok(torch.empty(4, 3, 64, 36, dtype=torch.bfloat16)[..., :32])   # rows 72 bytes apart
    packed = torch.empty(4, 64, 3, 3, 32, dtype=torch.bfloat16).permute(2, 0, 3, 1, 4)      # qkv projection output
    assert all(ok(packed[i]) for i in range(3))
    assert ok(torch.empty(3, 64, 64, dtype=torch.bfloat16))                    # the 3-d form (bias, mask)
    assert not ok(torch.empty(3, 14, 14, dtype=torch.bfloat16))


def test_kernel_ready_copies_only_what_it_must():
    a = torch.randn(2, 3, 16, 32).to(torch.float16)
    assert kernels._kernel_ready(a) is a
    view = a[..., 1:]
    ready = kernels._kernel_ready(view)
    assert ready is not view and ready.is_contiguous() and torch.equal(ready, view)


def test_rows_of_8_pads_and_caches_by_version(monkeypatch):
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)      # no device in this test
    bias = torch.randn(3, 14, 14)
    padded = kernels._rows_of_8(bias, cache=True)
    assert padded.shape == (3, 14, 16) and padded.stride() == (224, 16, 1)
    assert torch.equal(padded[..., :14], bias) and padded[..., 14:].abs().sum() == 0
    assert kernels._rows_of_8(bias, cache=True) is padded              # same tensor, same version: the cached copy
    bias.add_(1.0)                                                     # edited in place: padded again
    again = kernels._rows_of_8(bias, cache=True)
    assert again is not padded and torch.equal(again[..., :14], bias)
    assert kernels._rows_of_8(bias, cache=False) is not again          # a bias is rebuilt every call
    even = torch.randn(3, 16, 16)
    assert kernels._rows_of_8(even, cache=True) is even and kernels._rows_of_8(None, cache=True) is None
