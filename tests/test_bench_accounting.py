"""Known answers for the flop and byte accounting the benchmark reports."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import bench


def test_reference_convention_flops_known_answer():
    # benchmark/utils.py:26-67 counts, per (unit, head), 6 N d (two normalisations and the scale) +
    # 4 N^2 d (two matmuls) + 6 N^2 (bias, mask, softmax); benchmark/bench_attn.py:99 triples it for
    # forward + backward.  N = 256, d = 32 by hand: 49 152 + 8 388 608 + 393 216.
    assert bench.flops_reference_convention(1, 1, 256, 32, fwd_bwd=False) == 8_830_976
    total = bench.flops_reference_convention(4096, 3, 256, 32)
    assert total == 3 * 4096 * 3 * 8_830_976
    assert round(total / 1e9, 2) == 325.55


def test_matmul_flops_known_answer():
    # 14 N^2 d per (unit, head): 4 forward, 10 backward; the benchmark shape gives 360.78 GFLOP
    assert bench.flops_matmul(1, 1, 256, 32) == 14 * 256 * 256 * 32
    assert round(bench.flops_matmul(4096, 3, 256, 32) / 1e9, 2) == 360.78
    assert bench.flops_matmul(4096, 3, 256, 32, bwd=False) * 10 == bench.flops_matmul(4096, 3, 256, 32, fwd=False) * 4
