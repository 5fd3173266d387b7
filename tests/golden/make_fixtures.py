"""Writes the golden fixtures of this directory from the float64 oracle.

    python tests/golden/make_fixtures.py

Each .npz holds seeded operator inputs (float32 arrays whose values are exactly representable in
the case's low-precision dtype) and the oracle's float64 results rounded to float32: o, lse, dq,
dk, dv, dbias, dscale.  The reference project ships no vectors of its own; these are regression
anchors for the oracle and a device-side comparison that needs no recomputation on the GPU box.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import window_attention_np as wnp          # noqa: E402
from oracle.swin_inputs import make_inputs              # noqa: E402

CASES = {
    # name: (make_inputs kwargs, dtype)
    "bf16_n16_shift_mask": (dict(batch=1, n_windows=4, heads=2, n=16, resolution=8, window=4, shift=2, seed=11),
                            torch.bfloat16),
    "f16_n49_no_mask": (dict(batch=2, n_windows=1, heads=1, n=49, with_mask=False, seed=12), torch.float16),
}


def build(name):
    kwargs, dtype = CASES[name]
    inp = make_inputs(dtype=dtype, **kwargs)
    if name.startswith("bf16"):
        # one head past the clamp, so the gate on the logit-scale gradient is part of the fixture
        inp["logit_scale"][1] = 5.0
    arrays = {k: v.float().numpy() for k, v in inp.items() if v is not None}
    args = [arrays.get(k) for k in ("logit_scale", "bias", "mask")]
    o, lse = wnp.forward(arrays["q"], arrays["k"], arrays["v"], *args)
    grads = wnp.backward(arrays["q"], arrays["k"], arrays["v"], arrays["do"], *args)
    out = {"in_" + k: v for k, v in arrays.items()}
    out["o"], out["lse"] = o.astype(np.float32), lse.astype(np.float32)
    for k, v in grads.items():
        if v is not None:
            out[k] = v.astype(np.float32)
    return out


if __name__ == "__main__":
    for case in CASES:
        path = os.path.join(HERE, case + ".npz")
        np.savez_compressed(path, **build(case))
        print(case, os.path.getsize(path), "bytes")
