"""The throughput sweeps (``python -m flagattention_amd.benchmarks``) as a checked component.

The counted FLOPs and bytes are compared with the closed forms of the reference's benchmark scripts
(``benchmark/flash_benchmark.py:95-103``, ``benchmark/paged_benchmark.py:184``) written out for
fixed shapes; on a GPU every sweep runs for one point."""
import math

import pytest
import torch

from flagattention_amd import benchmarks


def test_flash_flop_count_follows_the_reference_convention():
    # flash_benchmark.py:96-103: macs = 2 B H T^2 D, x2.5 backward, flops = 2 macs, halved if causal
    B, H, T, D = 4, 16, 2048, 128
    assert benchmarks.flash_flops(B, H, T, D, False, "fwd") == 4 * 4 * 16 * 2048 * 2048 * 128
    assert benchmarks.flash_flops(B, H, T, D, True, "fwd") == 2 * 4 * 16 * 2048 * 2048 * 128
    assert benchmarks.flash_flops(B, H, T, D, False, "bwd") == 10 * 4 * 16 * 2048 * 2048 * 128
    assert benchmarks.flash_flops(B, H, T, D, True, "bwd") == 5 * 4 * 16 * 2048 * 2048 * 128
    # forward + backward of the headline shape: 7 products' worth of 2 B H (T^2 / 2) D
    c3 = benchmarks.flash_flops(1, 32, 8192, 128, True, "fwd") + benchmarks.flash_flops(1, 32, 8192, 128, True, "bwd")
    assert c3 == 7 * 2 * 32 * (8192 * 8192 // 2) * 128


def test_decode_byte_and_pseudo_flop_counts():
    # every key and value row of every kv head once, two bytes per element
    assert benchmarks.kv_bytes(rows=64 * 4096, heads_kv=8, D=128) == 2 * 64 * 4096 * 8 * 128 * 2
    # paged_benchmark.py:184: 2.0 * num_seqs * num_query_heads * 2 * context_len * head_size
    assert benchmarks.paged_pseudo_flops(32, 64, 4096, 128) == 2.0 * 32 * 64 * 2 * 4096 * 128


def test_point_budget_stops_a_sweep():
    b = benchmarks._Budget(2)
    assert [b.spent() for _ in range(4)] == [False, False, True, True]
    assert not benchmarks._Budget(None).spent()


@pytest.mark.gpu
@pytest.mark.parametrize("which", benchmarks.SWEEPS)
def test_every_sweep_runs_one_point(which):
    records = benchmarks.run(which, quick=True, points=1)
    assert len(records) == 1
    r = records[0]
    assert math.isfinite(r["ms"]) and r["ms"] > 0
    if which in ("flash", "piecewise"):
        # first point of the sweep: forward, not causal, D = 64, T = 512 at 32768 tokens
        assert (r["mode"], r["causal"], r["D"], r["T"], r["B"], r["H"]) == ("fwd", False, 64, 512, 64, 32)
        assert r["flops"] == 4.0 * 64 * 32 * 512 * 512 * 64
        assert r["tflops"] == pytest.approx(r["flops"] / (r["ms"] * 1e-3) / 1e12)
        assert 1.0 < r["tflops"] < 2500.0          # below the chip's dense bf16 peak
    elif which == "decode":
        assert (r["D"], r["N"], r["B"], r["H"]) == (64, 512, 2, 32)
        assert r["bytes"] == 2 * 2 * 32 * 512 * 64 * 2
        assert 0 < r["gbs"] < 8000.0 * 8          # tiny inputs are served from cache, HBM peak does not bound them
    else:
        assert (r["num_seqs"], r["group"], r["D"], r["block"], r["ctx"]) == (1, 1, 64, 16, 512)
        assert r["bytes"] == 2 * 1 * 512 * 64 * 64 * 2
        assert r["pseudo_tflops"] == pytest.approx(2.0 * 1 * 64 * 2 * 512 * 64 / (r["ms"] * 1e-3) / 1e12)
