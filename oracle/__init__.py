"""CPU oracle for Swin V2 scaled-cosine window attention.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is used by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, always as the checker and never as the thing
being measured or shipped.

Modules
-------
window_attention_np   float64 numpy restatement: forward, log-sum-exp and the
                      hand-derived backward (dq, dk, dv, dbias, dlogit_scale).
classic_torch         restatement of the classic PyTorch definition (normalise,
                      matmul, scale, bias, mask, softmax, matmul) run in
                      whatever dtype it is given; in fp32 it is the parity bar
                      and the CPU baseline.
swin_inputs           closed-form shifted-window mask, relative-position index
                      and seeded input factories for the benchmark configs.

Pinning status (what each function is checked against, see tests/test_oracle_*):
  forward         brute-force scalar loops (tiny shapes), torch SDPA special
                  case, softmax/normalisation invariants
  backward        torch.autograd of the classic restatement in float64,
                  finite differences, orthogonality / zero-row-sum invariants
  mask generator  the slice-painting construction vs the closed form, plus
                  structural properties (symmetry, zero windows count)
  The reference repository holds no golden vectors or asserted tests for this
  path, so nothing here is pinned against reference-produced numbers; the
  achieved error of the reference's Triton kernels is "parity unpinned".
"""
