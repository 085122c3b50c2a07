"""Every kernel under adversarial wavefront schedules on the host lane simulator.

The wavefronts of a workgroup share tiles in LDS and meet at workgroup barriers.  The simulator's default
schedule advances them nearly in step, which is the schedule least likely to show a missing barrier.  Here
each case runs again with every wavefront running ahead alone until it has to wait (lowest index first, then
highest first: the largest skew the barriers allow) and under random interleavings; a correctly synchronised
kernel gives bit-identical results under all of them.
"""
import contextlib
import os
import subprocess
import sys

import pytest
import torch

import flag_attn
from flagattention_amd import _lib, flash, paged, piecewise
from tests.sim import simlib

SCHEDULES = [("ahead", 0), ("ahead_descending", 0), ("random", 1), ("random", 2)]


@pytest.fixture(autouse=True)
def simulator_behind_the_public_api(monkeypatch):
    lib = simlib.get()
    monkeypatch.setattr(_lib, "get", lambda: lib)
    monkeypatch.setattr(torch.cuda, "device", lambda device: contextlib.nullcontext())


@contextlib.contextmanager
def schedule(mode, seed):
    os.environ["HWSIM_SCHEDULE"], os.environ["HWSIM_SEED"] = mode, str(seed)
    try:
        yield
    finally:
        del os.environ["HWSIM_SCHEDULE"], os.environ["HWSIM_SEED"]


def same_under_every_schedule(run):
    expected = run()
    for mode, seed in SCHEDULES:
        with schedule(mode, seed):
            got = run()
        for i, (a, b) in enumerate(zip(got, expected)):
            assert torch.equal(a, b), f"output {i} differs under schedule {mode} (seed {seed})"


def rnd(*shape, dtype=torch.bfloat16, seed=0):
    gen = torch.Generator().manual_seed(seed + sum(shape))
    return torch.randn(*shape, generator=gen).to(dtype)


CHILD = """
import contextlib, torch, flag_attn
from flagattention_amd import _lib
from tests.sim import simlib
lib = simlib.get()
_lib.get = lambda: lib
torch.cuda.device = lambda device: contextlib.nullcontext()
q = torch.randn(1, 1, 32, 16).half()
flag_attn.flash_attention(q, q, q)
"""


def test_the_simulator_reads_the_schedule():
    """An unknown name ends the process that launches a kernel (so ask a child): the variable is honoured."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    good = subprocess.run([sys.executable, "-c", CHILD], cwd=root, capture_output=True, text=True,
                          env=dict(os.environ, HWSIM_SCHEDULE="ahead"))
    assert good.returncode == 0, good.stderr
    bad = subprocess.run([sys.executable, "-c", CHILD], cwd=root, capture_output=True, text=True,
                         env=dict(os.environ, HWSIM_SCHEDULE="no such schedule"))
    assert bad.returncode != 0 and "HWSIM_SCHEDULE must be" in bad.stderr


@pytest.mark.parametrize("D,M,N,causal,block_m,route", [
    (128, 200, 200, True, 128, "whole"),
    (128, 300, 270, False, 256, "sliced"),       # the 256-row forward; dS handed over in slices
    (128, 129, 257, True, 256, "recompute"),
    (64, 150, 190, True, None, "default"),
    (32, 130, 130, False, None, "default"),
    (16, 100, 140, True, None, "default"),
])
def test_flash_attention(monkeypatch, D, M, N, causal, block_m, route):
    B, H, Hk = 1, 2, 1
    q, k, v = rnd(B, H, M, D).requires_grad_(), rnd(B, Hk, N, D, seed=1).requires_grad_(), rnd(B, Hk, N, D, seed=2).requires_grad_()
    do = rnd(B, H, M, D, seed=3)
    if route != "default":
        heads = {"whole": B * H, "sliced": H // Hk, "recompute": 0}[route]
        monkeypatch.setattr(flash, "ds_heads_per_launch", lambda *a, **kw: heads)
    if block_m is not None:
        monkeypatch.setattr(flash, "get_fwd_config", lambda *a: (block_m, 64, 2, 4))
    monkeypatch.setattr(flash, "num_splits_heuristic", lambda *a: 1)    # the dense forward, however few workgroups

    def run():
        o, L, tot, _, _ = flag_attn.flash_attention(q, k, v, causal=causal, return_log_normalizer=True,
                                                    return_total_attention=True)
        return (o, L, tot) + torch.autograd.grad(o, (q, k, v), do)

    same_under_every_schedule(run)


def test_flash_attention_with_dropout(monkeypatch):
    q, k, v = (rnd(1, 2, 140, 64, dtype=torch.float16, seed=s).requires_grad_() for s in range(3))
    do = rnd(1, 2, 140, 64, dtype=torch.float16, seed=3)
    monkeypatch.setattr(flash, "philox_cuda_seed_offset", lambda n, device: (1234, 8))   # the same mask in every run
    monkeypatch.setattr(flash, "num_splits_heuristic", lambda *a: 1)    # a shape this small would be split, without dropout

    def run():
        o = flag_attn.flash_attention(q, k, v, causal=True, dropout_p=0.2)
        return (o,) + torch.autograd.grad(o, (q, k, v), do)

    same_under_every_schedule(run)


@pytest.mark.parametrize("route", ["whole", "recompute"])
def test_piecewise_attention(monkeypatch, route):
    B, H, M, N, D, w = 1, 2, 150, 170, 128, 40
    ins = [rnd(B, H, M if i in (0, 2) else N, D, seed=i).requires_grad_() for i in range(5)]   # q1, k1, q2, k2, v
    do = rnd(B, H, M, D, seed=9)
    monkeypatch.setattr(piecewise, "ds_heads_per_launch", lambda *a, **kw: {"whole": B * H, "recompute": 0}[route])

    def run():
        o = flag_attn.piecewise_attention(*ins, w, causal=True)
        return (o,) + torch.autograd.grad(o, ins, do)

    same_under_every_schedule(run)


def test_split_kv_forward():
    q = rnd(1, 4, 3, 128, dtype=torch.float16)
    k, v = rnd(1, 2, 1500, 128, dtype=torch.float16, seed=1), rnd(1, 2, 1500, 128, dtype=torch.float16, seed=2)

    def run():
        o, L, *_ = flag_attn.flash_attention(q, k, v, causal=False, return_log_normalizer=True)
        return (o, L, flag_attn.flash_attention_split_kv(q, k, v, causal=True))

    same_under_every_schedule(run)


@pytest.mark.parametrize("launch", [("balanced", 5), ("single", 0), ("partitioned", 4)])
def test_paged_attention(monkeypatch, launch):
    seqs, Hq, Hkv, D, bs = 3, 8, 2, 128, 16
    ctx = torch.tensor([300, 1, 133], dtype=torch.int32)
    blocks = [(int(c) + bs - 1) // bs for c in ctx]
    num_blocks = sum(blocks) + 2
    perm = torch.randperm(num_blocks, generator=torch.Generator().manual_seed(5))
    table = torch.zeros(seqs, max(blocks), dtype=torch.int32)
    at = 0
    for s, n in enumerate(blocks):
        table[s, :n] = perm[at:at + n]
        at += n
    q = rnd(seqs, Hq, D, dtype=torch.float16)
    kc, vc = rnd(num_blocks, Hkv, bs, D, dtype=torch.float16, seed=1), rnd(num_blocks, Hkv, bs, D, dtype=torch.float16, seed=2)
    num_splits = 0
    if launch[0] == "partitioned":
        num_splits = launch[1]
    else:
        monkeypatch.setattr(paged, "choose_launch", lambda *a: launch)   # a handful of workgroups instead of a full chip's

    def run():
        return (flag_attn.paged_attention(q, kc, vc, ctx, table, D ** -0.5, int(ctx.max()), num_splits),)

    same_under_every_schedule(run)
