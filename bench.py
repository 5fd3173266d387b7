#!/usr/bin/env python3
"""Benchmark of the hot path: Swin V2 scaled-cosine window attention, forward +
backward, on one MI355X.

A "step" is one forward + backward of the operator on the benchmark's
synthetic batch (benchmark configuration 3: B=64 images x 64 windows of N=256 tokens,
3 heads, head dim 32, bf16, shifted-window mask, bias = 16*sigmoid(N(0,1)),
logit_scale = ln 10), inputs already resident in HBM.  One JSON line goes to
stdout; progress goes to stderr.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras | --basic-extras]
                    [--sweep [--sweep-n N ...]] [--copy-bytes B]

`extras` carries the forward-only and N = 64 figures, peak memory, the window-size sweep of the reference's
operator benchmark as HIP graph replays and one end-to-end model step; `--sweep` prints the sweep alone, with
the eager timings beside the replays (`--sweep-n`: only those window lengths, replays only, for a profiler);
`--copy-bytes` adds a plain device copy of that size, timed, as the reference point for HBM counters and for the
time the step's bytes would take at copy speed.
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "fwd+bwd ms & TFLOPS (% MFMA peak), B64 nW64 H3 d32 N256 bf16, 1 GPU"
MFMA_BF16_PEAK_TFLOPS = 2500.0     # MI355X dense bf16
HBM_PEAK_GBS = 8000.0              # MI355X HBM3E
# HBM bytes per launch of the backward kernel at the benchmark shape, from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a copy kernel of known size
# (profiles/kernels_C3_fwd_bwd.txt: FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0).
BWD_KERNEL_TRAFFIC_BYTES = 1.805e9
# device memory the library holds on every GPU whether or not it is used (the scratch of fwa2_backward_static)
STATIC_SCRATCH_MB = 128.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def flops_matmul(bw, heads, n, d, fwd=True, bwd=True):
    """Algorithmic matmul flops: 4 N^2 d forward (QK^T, PV), 10 N^2 d backward."""
    per = (4 if fwd else 0) + (10 if bwd else 0)
    return per * n * n * d * bw * heads


def flops_reference_convention(bw, heads, n, d, fwd_bwd=True):
    """FLOP count the reference's own benchmark quotes (benchmark/utils.py:26-67): per (bw, head)
    6 N d + 4 N^2 d + 6 N^2, and three times that for forward+backward (benchmark/bench_attn.py:99)."""
    per = 6 * n * d + 4 * n * n * d + 6 * n * n
    return per * bw * heads * (3 if fwd_bwd else 1)


def bytes_min(bw, heads, n, d, n_windows, fwd=True, bwd=True, e=2):
    """Algorithmic HBM bytes: q,k,v,o (+lse) forward; q,k,v,o,do,dq,dk,dv (+lse, dbias) backward;
    bias and mask once per pass."""
    unit = bw * heads
    side = heads * n * n * e + n_windows * n * n * e
    tot = 0
    if fwd:
        tot += unit * (4 * n * d * e + 4 * n) + side
    if bwd:
        tot += unit * (8 * n * d * e + 4 * n) + side + heads * n * n * e
    return tot


class HipEvents:
    """Raw hipEvent pairs (torch.cuda.Event would only see torch's current stream; these are
    recorded by the library on the stream the kernel is launched on)."""

    def __init__(self, count):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]
        self.pairs = []
        for _ in range(count):
            a, b = ctypes.c_void_p(), ctypes.c_void_p()
            assert self.hip.hipEventCreate(ctypes.byref(a)) == 0 and self.hip.hipEventCreate(ctypes.byref(b)) == 0
            self.pairs.append((a, b))

    def elapsed_ms(self):
        out = []
        for a, b in self.pairs:
            assert self.hip.hipEventSynchronize(b) == 0
            ms = ctypes.c_float()
            assert self.hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
            out.append(ms.value)
        return out


def time_steps(fn, steps, warmup, torch):
    for _ in range(warmup):
        fn(-1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def cpu_baseline(cfg, torch):
    """The oracle's classic fp32 path (forward + autograd backward) on the host cores, on a
    bounded batch slice of the same workload."""
    from oracle.classic_torch import classic_fwd_bwd
    from oracle.swin_inputs import make_inputs

    cores = len(os.sched_getaffinity(0))
    torch.set_num_threads(cores)
    sample_batch = 8     # about 0.4 GB per N x N fp32 tensor; 10-20 s of host work in all
    small = dict(cfg, batch=sample_batch)
    inp = make_inputs(**small, dtype=torch.bfloat16, seed=0)
    args = (inp["q"], inp["k"], inp["v"], inp["logit_scale"], inp["bias"], inp["mask"], inp["do"])
    classic_fwd_bwd(*args)                       # warm-up
    times = []
    t_end = time.perf_counter() + 15.0
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 20):
        t0 = time.perf_counter()
        classic_fwd_bwd(*args)
        times.append(time.perf_counter() - t0)
    sec = sorted(times)[len(times) // 2]
    fl = flops_matmul(sample_batch * cfg["n_windows"], cfg["heads"], cfg["n"], cfg["d"])
    return {
        "value": round(fl / sec * 1e-12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"classic fp32 torch forward+backward on batch {sample_batch} of {cfg['batch']} "
                  f"(BW={sample_batch * cfg['n_windows']}), median of {len(times)} runs, {sec * 1e3:.1f} ms each; "
                  f"scaled to the full batch: {sec * 1e3 * cfg['batch'] / sample_batch:.0f} ms per step",
    }


class L2Flush:
    """Overwrites a buffer larger than every cache level between timed calls (the 8 x 4 MB L2s and the
    256 MB memory-side cache), as triton.testing.do_bench does for the reference's own operator benchmark
    (benchmark/bench_attn.py:93): small shapes are then timed from HBM, not from a warm cache."""

    def __init__(self, torch, nbytes=512 << 20):
        self.buf = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda")

    def __call__(self):
        self.buf.zero_()


def timed_calls(torch, fn, steps, warmup, flush=None):
    """One event pair per call (recorded on torch's current stream, which is where `fn` enqueues), an optional
    cache flush before each call outside the pair.  Returns (median ms, mean ms)."""
    for _ in range(warmup):
        fn()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for e0, e1 in pairs:
        if flush is not None:
            flush()
        e0.record()
        fn()
        e1.record()
    torch.cuda.synchronize()
    ms = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    return ms[len(ms) // 2], sum(ms) / len(ms)


def captured(torch, fn):
    """`fn` as one HIP graph: warmed up on a side stream, captured once; returns the replay callable."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return graph.replay


def window_sweep(torch, steps, warmup, eager=True, windows=(64, 144, 256, 576, 1024)):
    """The reference's window-size sweep (benchmark/config.py: B16 x 16 windows, H6, d32, windows of 8, 12, 16, 24
    and 32 tokens a side, bias = 16 sigmoid(randn), tensor logit scale ln 10, no mask) in bf16 and fp16, forward
    and forward + backward.  Every case is timed as one captured HIP graph replayed `steps` times, which takes the
    host out of the figure (at 1 536 units the eager calls are bound by it up to 256 tokens), each replay from
    flushed caches; with `eager` also as plain calls.  Median and mean per call; TFLOP/s (of the median) count the
    matrix products only (4 N^2 d forward, 14 N^2 d forward + backward)."""
    from flash_window_attention_v2_amd import flash_win_attn_v2_func

    flush = L2Flush(torch)
    bw, heads, d = 16 * 16, 6, 32
    rows = []
    for dtype in (torch.bfloat16, torch.float16):
        for n in windows:
            g = torch.Generator(device="cpu").manual_seed(0)
            q, k, v, do = (torch.randn(bw, heads, n, d, generator=g).to(dtype).cuda() for _ in range(4))
            bias = (16 * torch.sigmoid(torch.randn(heads, n, n, generator=g))).to(dtype).cuda()
            ls = torch.full((heads, 1, 1), math.log(10.0), dtype=dtype, device="cuda")
            leaves = (q, k, v, bias, ls)
            for t in leaves:
                t.requires_grad_(True)

            def fwd():
                with torch.no_grad():
                    return flash_win_attn_v2_func(q, k, v, ls, bias, None)

            def fwd_bwd():
                for t in leaves:
                    t.grad = None
                flash_win_attn_v2_func(q, k, v, ls, bias, None).backward(do)

            fl = flops_matmul(bw, heads, n, d, bwd=False)
            fl_all = flops_matmul(bw, heads, n, d)
            row = {"dtype": str(dtype).split(".")[-1], "n": n}
            for tag, fn, f in (("fwd", fwd, fl), ("fwd_bwd", fwd_bwd, fl_all)):
                if eager:
                    med, mean = timed_calls(torch, fn, steps, warmup, flush)
                    row[tag + "_eager_ms"] = [round(med, 4), round(mean, 4)]
                    row[tag + "_eager_tflops"] = round(f / med * 1e-9, 1)
                med, mean = timed_calls(torch, captured(torch, fn), steps, warmup, flush)
                row[tag + "_ms"] = [round(med, 4), round(mean, 4)]
                row[tag + "_tflops"] = round(f / med * 1e-9, 1)
                row[tag + "_pct_peak"] = round(f / med * 1e-9 / MFMA_BF16_PEAK_TFLOPS * 100, 2)
            log(f"[bench] sweep {row}")
            rows.append(row)
    return {"sweep": "B16 x 16 windows, H6, d32, bias, tensor scale, no mask; one HIP graph replay per call, caches "
                     "flushed before each; *_ms = [median, mean]; TFLOP/s of the matrix products at the median; "
                     "pct_peak against 2.5 PFLOP/s (bf16 and fp16 dense)",
            "steps": steps, "warmup": warmup, "rows": rows}


def model_step(torch, steps, warmup, batch=64):
    """The end-to-end case (Swin V2-T layout: 256 x 256 images, patch 4, depths 2/2/6/2, heads 3/6/12/24, windows
    of 16 x 16 tokens, bf16, batch 64) timed the way the reference times its model (benchmark/bench_model.py:23-38:
    zero_grad, forward, cross-entropy, backward, Adam step; peak memory of the loop), with this library's operator
    and with the classic one.  Median and mean of per-step event pairs."""
    from flash_window_attention_v2_amd import SwinTransformerV2

    out = {"config": f"img 256, patch 4, embed 96, depths 2/2/6/2, heads 3/6/12/24, window 16, bf16, batch {batch}, "
                     "random weights and images; training step with Adam; *_ms = [median, mean]"}
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(batch, 3, 256, 256, generator=g).to(torch.bfloat16).cuda()
    y = torch.randint(0, 1000, (batch,), generator=g).cuda()
    for tag, flash in (("flash", True), ("classic", False)):
        torch.manual_seed(0)
        model = SwinTransformerV2(img_size=256, patch_size=4, embed_dim=96, depths=[2, 2, 6, 2], num_heads=[3, 6, 12, 24],
                                  window_size=16, is_flash=flash).to(dtype=torch.bfloat16, device="cuda")
        opt = torch.optim.Adam(model.parameters(), lr=1e-4)

        def step():
            opt.zero_grad()
            loss = torch.nn.functional.cross_entropy(model(x), y)
            loss.backward()
            opt.step()

        step()
        torch.cuda.synchronize(); torch.cuda.empty_cache(); torch.cuda.reset_peak_memory_stats()
        med, mean = timed_calls(torch, step, steps, warmup)
        out[tag + "_step_ms"] = [round(med, 3), round(mean, 3)]
        out[tag + "_peak_mem_gb"] = round(torch.cuda.max_memory_allocated() / 2**30, 3)
        with torch.no_grad():
            med, mean = timed_calls(torch, lambda: model(x), steps, warmup)
        out[tag + "_fwd_ms"] = [round(med, 3), round(mean, 3)]
        log(f"[bench] model {tag}: step {out[tag + '_step_ms']} ms, {out[tag + '_peak_mem_gb']} GB")
        del model, opt
        torch.cuda.empty_cache()
    out["step_speedup"] = round(out["classic_step_ms"][0] / out["flash_step_ms"][0], 3)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip forward-only, N=64 and memory figures")
    ap.add_argument("--basic-extras", action="store_true",
                    help="extras without the window-size sweep and the model step (forward-only, N=64 and memory figures only)")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the benchmark line, print the window-size sweep (TFLOP/s versus N) as one JSON line")
    ap.add_argument("--sweep-n", type=int, nargs="+", default=None,
                    help="with --sweep: only these window lengths (tokens), graph replays only")
    ap.add_argument("--copy-bytes", type=int, default=0,
                    help="also run one plain device copy of this many bytes (reference point for HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the hot path has no cross-GPU step); use --gpus 1")

    import torch

    from flash_window_attention_v2_amd import _abi, flash_win_attn_v2_func
    from oracle.swin_inputs import CONFIGS, make_inputs

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    lib = _abi.load()
    torch.cuda.set_device(0)
    if args.sweep:
        if args.sweep_n:
            out = window_sweep(torch, min(args.steps, 30), min(args.warmup, 5), eager=False, windows=tuple(args.sweep_n))
        else:
            out = window_sweep(torch, min(args.steps, 30), min(args.warmup, 5))
        print(json.dumps(out), flush=True)
        return

    def setup(cfg):
        inp = make_inputs(**cfg, dtype=torch.bfloat16, seed=0)
        dev = {k: (None if v is None else v.cuda()) for k, v in inp.items()}
        for name in ("q", "k", "v", "bias", "logit_scale"):
            dev[name].requires_grad_(True)
        return dev

    def make_step(dev):
        leaves = [dev[n] for n in ("q", "k", "v", "bias", "logit_scale")]

        def step(i):
            o = flash_win_attn_v2_func(dev["q"], dev["k"], dev["v"], dev["logit_scale"], dev["bias"], dev["mask"])
            o.backward(dev["do"])
            for t in leaves:
                t.grad = None
        return step

    def kernel_times(dev, steps, warmup):
        """The main kernels of one step, each between a pair of HIP events that the library records on the launch
        stream around them (fwa2_problem.ev_start / ev_stop): the same two library calls a step makes, issued
        through the launchers under the reference's names.  Returns (forward ms list, backward-kernel ms list)."""
        from flash_window_attention_v2_amd.kernels import _flash_attn_backward, _flash_attn_forward
        q, k, v, ls, bias, mask, do = (dev[n].detach() for n in ("q", "k", "v", "logit_scale", "bias", "mask", "do"))
        dq, dk, dv = (torch.empty_like(x) for x in (q, k, v))
        ds, db = torch.empty_like(ls), torch.empty_like(bias)
        ev_f, ev_b = HipEvents(steps), HipEvents(steps)
        for i in range(-warmup, steps):
            o, lse, _ = _flash_attn_forward(q, k, v, ls, bias=bias, mask=mask, scale_type="tensor",
                                            _events=ev_f.pairs[i] if i >= 0 else None)
            _flash_attn_backward(do, q, k, v, ls, o, lse, dq, dk, dv, ds, db, bias=bias, mask=mask, scale_type="tensor",
                                 _events=ev_b.pairs[i] if i >= 0 else None)
        torch.cuda.synchronize()
        return ev_f.elapsed_ms(), ev_b.elapsed_ms()

    cfg = CONFIGS["C3"]
    bw = cfg["batch"] * cfg["n_windows"]
    log(f"[bench] building inputs {cfg}")
    dev = setup(cfg)
    log("[bench] timing forward+backward")
    ms = time_steps(make_step(dev), args.steps, args.warmup, torch)
    log("[bench] timing the kernels of a step")
    fwd_kern_ms, bwd_kern_ms = kernel_times(dev, args.steps, min(args.warmup, 5))
    kern_avg = sum(bwd_kern_ms) / len(bwd_kern_ms)
    fl_all = flops_matmul(bw, cfg["heads"], cfg["n"], cfg["d"])
    # the dominant kernel is the whole backward in one pass (S recomputed once, dP, dV, dK, dQ): 10 N^2 d flops
    # per unit; its algorithmic bytes are the backward's (q, k, v, o, dO in; dq, dk, dv, dbias out; lse, bias, mask)
    fl_bwd = flops_matmul(bw, cfg["heads"], cfg["n"], cfg["d"], fwd=False)
    by_bwd = bytes_min(bw, cfg["heads"], cfg["n"], cfg["d"], cfg["n_windows"], fwd=False)
    tflops = fl_all / (ms * 1e-3) * 1e-12
    achieved = fl_bwd / (kern_avg * 1e-3) * 1e-12

    def kernel_row(name, ms_list, flops, nbytes):
        avg = sum(ms_list) / len(ms_list)
        med = sorted(ms_list)[len(ms_list) // 2]
        return {"kernel": name, "ms": round(avg, 4), "ms_median": round(med, 4), "flops": flops, "bytes": nbytes,
                "tflops": round(flops / avg * 1e-9, 1), "frac_mfma_peak": round(flops / avg * 1e-9 / MFMA_BF16_PEAK_TFLOPS, 4),
                "gbs": round(nbytes / avg * 1e-6, 1), "frac_hbm_peak": round(nbytes / avg * 1e-6 / HBM_PEAK_GBS, 4)}

    kernels = [
        kernel_row("forward: fwd_resident_kernel (masked and unmasked units in one launch)", fwd_kern_ms,
                   flops_matmul(bw, cfg["heads"], cfg["n"], cfg["d"], bwd=False),
                   bytes_min(bw, cfg["heads"], cfg["n"], cfg["d"], cfg["n_windows"], bwd=False)),
        kernel_row("backward: bwd_one_kernel (dq, dk, dv, dbias partials, dlogit_scale terms in one pass)", bwd_kern_ms,
                   fl_bwd, by_bwd),
    ]

    result = {
        "metric": METRIC, "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C3: B64 x 64 windows, H3, N256, d32, bf16, shift-8 mask, fwd+bwd", "bw": bw,
                   "heads": cfg["heads"], "n": cfg["n"], "head_dim": cfg["d"]},
        "pct_mfma_peak": round(100 * tflops / MFMA_BF16_PEAK_TFLOPS, 2),
        "roofline": {"bound": "mfma", "kernel": "bwd_one_kernel (the whole backward in one pass, one launch)",
                     "achieved": round(achieved, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": BWD_KERNEL_TRAFFIC_BYTES,
                     "kernel_ms": round(kern_avg, 4),
                     "hbm_frac_of_8TBs": round(by_bwd / (kern_avg * 1e-3) / (HBM_PEAK_GBS * 1e9), 4),
                     "kernels": kernels},
    }

    if not args.no_extras:
        extras = {}
        log("[bench] forward only")
        with torch.no_grad():
            f_ms = time_steps(lambda i: flash_win_attn_v2_func(dev["q"], dev["k"], dev["v"], dev["logit_scale"],
                                                               dev["bias"], dev["mask"]), args.steps, args.warmup, torch)
        extras["fwd_ms"] = round(f_ms, 4)
        extras["fwd_tflops"] = round(flops_matmul(bw, cfg["heads"], cfg["n"], cfg["d"], bwd=False) / f_ms * 1e-9, 2)
        extras["tflops_reference_convention"] = round(flops_reference_convention(bw, cfg["heads"], cfg["n"], cfg["d"]) / ms * 1e-9, 2)
        extras["fwd_tflops_reference_convention"] = round(
            flops_reference_convention(bw, cfg["heads"], cfg["n"], cfg["d"], fwd_bwd=False) / f_ms * 1e-9, 2)
        extras["fwd_hbm_gbs"] = round(bytes_min(bw, cfg["heads"], cfg["n"], cfg["d"], cfg["n_windows"], bwd=False) / f_ms * 1e-6, 1)
        extras["fwd_bwd_hbm_gbs"] = round(bytes_min(bw, cfg["heads"], cfg["n"], cfg["d"], cfg["n_windows"]) / ms * 1e-6, 1)
        # peak memory of the op against the classic path in the same dtype on the GPU
        step = make_step(dev)
        torch.cuda.synchronize(); torch.cuda.empty_cache(); torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        step(-1); torch.cuda.synchronize()
        extras["peak_mem_mb_new"] = round((torch.cuda.max_memory_allocated() - base) / 2**20, 1)
        extras["static_scratch_mb"] = STATIC_SCRATCH_MB
        extras["peak_mem_mb_new_with_static_scratch"] = round(extras["peak_mem_mb_new"] + STATIC_SCRATCH_MB, 1)
        from flash_window_attention_v2_amd import win_attention_torch
        torch.cuda.empty_cache(); torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        o = win_attention_torch(dev["q"], dev["k"], dev["v"], dev["logit_scale"], dev["bias"], dev["mask"])
        o.backward(dev["do"]); torch.cuda.synchronize()
        extras["peak_mem_mb_classic_bf16"] = round((torch.cuda.max_memory_allocated() - base) / 2**20, 1)
        del o
        for n_ in ("q", "k", "v", "bias", "logit_scale"):
            dev[n_].grad = None
        extras["peak_mem_ratio"] = round(extras["peak_mem_mb_new_with_static_scratch"] / extras["peak_mem_mb_classic_bf16"], 4)
        del dev
        torch.cuda.empty_cache()
        # N = 64 (config 2) is bandwidth-bound: report achieved HBM GB/s
        log("[bench] config 2 (N=64)")
        c2 = CONFIGS["C2"]
        dev2 = setup(c2)
        # one event pair per call, caches flushed before every call (the step touches 0.6 GB against a 256 MB
        # memory-side cache), median and mean
        step2 = make_step(dev2)
        ms2, ms2_mean = timed_calls(torch, lambda: step2(0), args.steps, args.warmup, L2Flush(torch))
        bw2 = c2["batch"] * c2["n_windows"]
        extras["c2_fwd_bwd_ms"] = round(ms2, 4)
        extras["c2_fwd_bwd_ms_mean"] = round(ms2_mean, 4)
        extras["c2_timing"] = "per-call event pairs, 512 MiB flush before each call, median (and mean)"
        extras["c2_hbm_gbs"] = round(bytes_min(bw2, c2["heads"], c2["n"], c2["d"], c2["n_windows"]) / ms2 * 1e-6, 1)
        extras["c2_hbm_frac"] = round(extras["c2_hbm_gbs"] / HBM_PEAK_GBS, 4)
        extras["c2_tflops"] = round(flops_matmul(bw2, c2["heads"], c2["n"], c2["d"]) / ms2 * 1e-9, 2)
        del dev2
        torch.cuda.empty_cache()
        if not args.basic_extras:
            log("[bench] window-size sweep as graph replays")
            extras["window_sweep"] = window_sweep(torch, 10, 2, eager=False)
            log("[bench] end-to-end model step")
            extras["model"] = model_step(torch, 8, 2)
        result["extras"] = extras

    if args.copy_bytes:
        src = torch.empty(args.copy_bytes, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        result["copy_bytes"] = args.copy_bytes
        # The same copy timed: what the HBM gives a kernel that only reads and writes (read + written bytes per second).
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        result["copy_gbs"] = round(2 * args.copy_bytes * 10 / e0.elapsed_time(e1) * 1e-6, 1)
        del src, dst

    if not args.no_cpu:
        log("[bench] CPU baseline (classic fp32 on host cores)")
        result["cpu_baseline"] = cpu_baseline(cfg, torch)
    else:
        result["cpu_baseline"] = None

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
