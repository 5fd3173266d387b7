"""The operator under HIP graph capture: the library allocates nothing, never synchronises and records no
memset, so forward + backward can be captured once and replayed.  Every replay, with the program's own eager
work and synchronisations in between, must reproduce the eager result bit for bit."""
import pytest
import torch

from oracle.swin_inputs import make_inputs

pytestmark = pytest.mark.gpu


def _fresh(n, res, win, d, seed, scale):
    nw = (res // win) ** 2
    inp = make_inputs(batch=2, n_windows=nw, heads=3, n=n, d=d, dtype=torch.bfloat16, seed=seed, resolution=res,
                      window=win, shift=win // 2, with_scale=scale)
    return {k: (v.cuda() if v is not None else None) for k, v in inp.items()}


def _eager(func, t):
    q, k, v = (t[x].clone().requires_grad_() for x in "qkv")
    bias = t["bias"].clone().requires_grad_()
    scale = t["logit_scale"].clone().requires_grad_() if t["logit_scale"] is not None else None
    o = func(q, k, v, scale, bias, t["mask"])
    o.backward(t["do"])
    return [o.detach(), q.grad, k.grad, v.grad, bias.grad] + ([scale.grad] if scale is not None else [])


@pytest.mark.parametrize("n,res,win,d,scale", [(64, 16, 8, 32, True), (256, 32, 16, 32, True), (144, 24, 12, 32, False),
                                               (64, 16, 8, 64, True)])
def test_forward_backward_replay(n, res, win, d, scale):
    from flash_window_attention_v2_amd import flash_win_attn_v2_func as func
    st = _fresh(n, res, win, d, 100, scale)          # static tensors of the graph
    leaves = [st[x].requires_grad_() for x in "qkv"] + [st["bias"].requires_grad_()]
    if scale:
        leaves.append(st["logit_scale"].requires_grad_())

    def step():
        o = func(st["q"], st["k"], st["v"], st["logit_scale"], st["bias"], st["mask"])
        o.backward(st["do"])
        return o

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                    # warm-up: mask flags and launch plans are cached here
        for _ in range(3):
            for x in leaves:
                x.grad = None
            step()
    torch.cuda.current_stream().wait_stream(side)
    for x in leaves:
        x.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_static = step()
    outs = [o_static] + [x.grad for x in leaves]

    for seed in (1, 2, 3):
        new = _fresh(n, res, win, d, seed, scale)
        with torch.no_grad():
            for name in ("q", "k", "v", "do", "bias"):
                st[name].copy_(new[name])
        graph.replay()
        torch.cuda.synchronize()
        want = _eager(func, new)                     # eager work between the replays
        torch.cuda.synchronize()
        for got, ref in zip(outs, want):
            assert torch.equal(got, ref), f"replay with seed {seed} differs from eager"
