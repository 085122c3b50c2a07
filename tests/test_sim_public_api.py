"""The public operators (``flag_attn.flash_attention`` / ``piecewise_attention`` / ``paged_attention``)
end to end on the host lane simulator: the same Python host logic the GPU path runs -- hooks, split
decision, dS hand-over policy, slicing, autograd wiring, group sums -- with CPU tensors and the kernel
sources compiled for the simulator.  Two test-only substitutions make that possible: the library
handle is the simulator build, and ``torch.cuda.device`` (a no-op for these tensors) is a null context.
The shipped package has no such path: without the HIP library it raises.
"""
import contextlib
import math

import pytest
import torch

import flag_attn
from flagattention_amd import _lib, flash, paged, piecewise
from oracle import flash_attention as oracle_flash, paged_attention as oracle_paged, piecewise_attention as oracle_pw
from oracle import within_two_x
from tests.sim import simlib

torch.manual_seed(20240)


@pytest.fixture(autouse=True)
def simulator_behind_the_public_api(monkeypatch):
    lib = simlib.get()
    monkeypatch.setattr(_lib, "get", lambda: lib)
    monkeypatch.setattr(torch.cuda, "device", lambda device: contextlib.nullcontext())
    return lib


def check(name, hyp, same, ref, strict=False):
    ok, e_hyp, e_same = within_two_x(hyp, same, ref, strict=strict)
    assert ok, f"{name}: kernel err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


def rnd(*shape, dtype=torch.bfloat16, grad=False):
    t = torch.randn(*shape).to(dtype)
    return t.requires_grad_() if grad else t


def flash_case(B, H, Hk, M, N, D, causal, dtype=torch.bfloat16):
    q, k, v = rnd(B, H, M, D, dtype=dtype, grad=True), rnd(B, Hk, N, D, dtype=dtype, grad=True), rnd(B, Hk, N, D, dtype=dtype, grad=True)
    do = rnd(B, H, M, D, dtype=dtype)
    ref = oracle_flash(q, k, v, causal, upcast=True, return_log_normalizer=True, return_total_attention=True)
    same = oracle_flash(q, k, v, causal, upcast=False, return_log_normalizer=True, return_total_attention=True)
    g_ref = torch.autograd.grad(ref[0], (q, k, v), do)
    g_same = torch.autograd.grad(same[0], (q, k, v), do)
    return (q, k, v, do), ref, same, g_ref, g_same


@pytest.mark.parametrize("B,H,Hk,M,N,D,causal", [
    (1, 4, 2, 70, 90, 64, True),       # grouped heads: dK/dV summed over each kv head's query heads
    (2, 2, 2, 65, 40, 128, False),
    (1, 2, 1, 40, 130, 32, True),
])
def test_flash_attention_forward_backward(B, H, Hk, M, N, D, causal):
    (q, k, v, do), ref, same, g_ref, g_same = flash_case(B, H, Hk, M, N, D, causal)
    o, L, tot, seed, offset = flag_attn.flash_attention(q, k, v, causal=causal, return_log_normalizer=True,
                                                        return_total_attention=True)
    assert seed is None and offset is None
    grads = torch.autograd.grad(o, (q, k, v), do)
    check("o", o, same[0], ref[0], strict=True)
    check("L", L, same[1], ref[1])
    check("total", tot, same[2], ref[2])
    for name, h, s, r in zip(("dq", "dk", "dv"), grads, g_same, g_ref):
        assert h.shape == r.shape and h.dtype == s.dtype
        check(name, h, s, r, strict=True)
    # plain call: the tensor alone (flash.py:150-160 of the reference)
    assert torch.equal(flag_attn.flash_attention(q, k, v, causal=causal), o)


@pytest.mark.parametrize("route", ["whole", "sliced", "recompute", "no memory"])
def test_flash_backward_routes_agree(monkeypatch, route):
    """The dS hand-over, its sliced form, the recomputing pair and the fall-back taken when the workspace
    cannot be allocated are four ways through ``FlashAttention.backward``; all meet the 2x rule and the
    two hand-over forms agree bit for bit."""
    B, H, Hk, M, N, D = 2, 4, 2, 64, 96, 128
    (q, k, v, do), ref, same, g_ref, g_same = flash_case(B, H, Hk, M, N, D, True)
    heads = {"whole": B * H, "sliced": 2, "recompute": 0, "no memory": B * H}[route]
    monkeypatch.setattr(flash, "ds_heads_per_launch", lambda *a, **kw: heads)
    if route == "no memory":
        monkeypatch.setattr(flash, "_ds_workspace", lambda *a, **kw: None)
    o = flag_attn.flash_attention(q, k, v, causal=True)
    grads = torch.autograd.grad(o, (q, k, v), do)
    for name, h, s, r in zip(("dq", "dk", "dv"), grads, g_same, g_ref):
        check(name, h, s, r, strict=True)
    if route == "sliced":
        monkeypatch.setattr(flash, "ds_heads_per_launch", lambda *a, **kw: B * H)
        whole = torch.autograd.grad(flag_attn.flash_attention(q, k, v, causal=True), (q, k, v), do)
        for a, b in zip(grads, whole):
            assert torch.equal(a, b)


def test_flash_attention_decode_shape_takes_the_split_path(monkeypatch):
    calls = []
    real = flash.split_kv_forward
    monkeypatch.setattr(flash, "split_kv_forward", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    q, k, v = rnd(1, 4, 1, 64, dtype=torch.float16), rnd(1, 2, 1100, 64, dtype=torch.float16), rnd(1, 2, 1100, 64, dtype=torch.float16)
    o, L, *_ = flag_attn.flash_attention(q, k, v, causal=False, return_log_normalizer=True)
    assert calls
    ref = oracle_flash(q, k, v, False, upcast=True, return_log_normalizer=True)
    same = oracle_flash(q, k, v, False, upcast=False, return_log_normalizer=True)
    check("o", o, same[0], ref[0])
    check("L", L, same[1], ref[1])
    # the forward-only entry point of split_kv.py:266-330
    o2 = flag_attn.flash_attention_split_kv(q, k, v, causal=False)
    check("o (split_kv entry)", o2, same[0], ref[0])


def test_replaced_hooks_are_called_per_launch(monkeypatch):
    seen = []

    def fwd(B, H, M, N, D, causal):
        seen.append(("fwd", B, H, M, N, D, causal))
        return (128, 64, 2, 4)

    def bwd(B, H, M, N, D, causal):
        seen.append(("bwd", B, H, M, N, D, causal))
        return (64, 128, 3, 4)

    monkeypatch.setattr(flash, "get_fwd_config", fwd)
    monkeypatch.setattr(flash, "get_bwd_config", bwd)
    q, k, v = rnd(1, 2, 40, 32, grad=True), rnd(1, 2, 50, 32, grad=True), rnd(1, 2, 50, 32, grad=True)
    o = flag_attn.flash_attention(q, k, v, causal=True)
    torch.autograd.grad(o, (q, k, v), torch.ones_like(o))
    assert seen == [("fwd", 1, 2, 40, 50, 32, True), ("bwd", 1, 2, 40, 50, 32, True)]


@pytest.mark.parametrize("route", ["whole", "sliced", "recompute", "no memory"])
def test_piecewise_attention_routes(monkeypatch, route):
    B, H, M, N, D, w = 1, 2, 70, 70, 128, 24
    ins = [rnd(B, H, M if i in (0, 2) else N, D, grad=True) for i in range(5)]   # q1, k1, q2, k2, v
    do = rnd(B, H, M, D)
    heads = {"whole": B * H, "sliced": 1, "recompute": 0, "no memory": B * H}[route]
    monkeypatch.setattr(piecewise, "ds_heads_per_launch", lambda *a, **kw: heads)
    if route == "no memory":
        monkeypatch.setattr(piecewise, "_ds_workspace", lambda *a, **kw: None)
    o = flag_attn.piecewise_attention(*ins, w, causal=True)
    grads = torch.autograd.grad(o, ins, do)
    ref = oracle_pw(*ins, w, causal=True, upcast=True)
    same = oracle_pw(*ins, w, causal=True)
    g_ref = torch.autograd.grad(ref, ins, do)
    g_same = torch.autograd.grad(same, ins, do)
    check("o", o, same, ref)
    for name, h, s, r in zip(("dq1", "dk1", "dq2", "dk2", "dv"), grads, g_same, g_ref):
        check(name, h, s, r)


def test_paged_attention_public_call():
    seqs, Hq, Hkv, D, bs = 3, 4, 2, 64, 16
    ctx = torch.tensor([37, 1, 160], dtype=torch.int32)
    blocks = [(int(c) + bs - 1) // bs for c in ctx]
    num_blocks = sum(blocks) + 2
    perm = torch.randperm(num_blocks)
    table = torch.zeros(seqs, max(blocks), dtype=torch.int32)
    at = 0
    for s, n in enumerate(blocks):
        table[s, :n] = perm[at:at + n]
        at += n
    q = rnd(seqs, Hq, D, dtype=torch.float16)
    kc, vc = rnd(num_blocks, Hkv, bs, D, dtype=torch.float16), rnd(num_blocks, Hkv, bs, D, dtype=torch.float16)
    scale = D ** -0.5
    out = flag_attn.paged_attention(q, kc, vc, ctx, table, scale, int(ctx.max()))
    ref = oracle_paged(q.float(), kc.float(), vc.float(), table, ctx, scale)
    assert torch.allclose(out.float(), ref, atol=2e-3, rtol=1e-5)   # tests/flag_attn/test_paged_attention.py:62


@pytest.mark.parametrize("launch", [("balanced", 3), ("single", 0), ("partitioned", 2)])
def test_paged_attention_zero_length_contexts(monkeypatch, launch):
    """A sequence without keys gets a zero row in every launch form, and does not disturb its neighbours."""
    seqs, Hq, Hkv, D, bs = 4, 4, 2, 64, 16
    ctx = torch.tensor([0, 100, 0, 33], dtype=torch.int32)
    num_blocks = 24
    table = torch.randint(0, num_blocks, (seqs, 8), dtype=torch.int32, generator=torch.Generator().manual_seed(3))
    q = rnd(seqs, Hq, D, dtype=torch.float16)
    kc, vc = rnd(num_blocks, Hkv, bs, D, dtype=torch.float16), rnd(num_blocks, Hkv, bs, D, dtype=torch.float16)
    num_splits = launch[1] if launch[0] == "partitioned" else 0
    if launch[0] != "partitioned":
        monkeypatch.setattr(paged, "choose_launch", lambda *a: launch)
    out = flag_attn.paged_attention(q, kc, vc, ctx, table, D ** -0.5, 100, num_splits)
    live = ctx > 0
    assert not out[~live].any()
    ref = oracle_paged(q[live].float(), kc.float(), vc.float(), table[live], ctx[live], D ** -0.5)
    assert torch.allclose(out[live].float(), ref, atol=2e-3, rtol=1e-5)


@pytest.mark.parametrize("num_wgs", [1, 7, 40])
def test_paged_attention_many_empty_sequences(monkeypatch, num_wgs):
    """Empty sequences are dealt round-robin to the workgroups of the balanced launch, also to those that
    have no keys to stream; more sequences than one scan step (64) and than workgroups."""
    seqs, Hq, Hkv, D, bs = 130, 4, 2, 32, 16
    gen = torch.Generator().manual_seed(11)
    ctx = torch.zeros(seqs, dtype=torch.int32)
    live_at = [0, 63, 64, 97, 129]
    ctx[live_at] = torch.tensor([5, 130, 1, 40, 77], dtype=torch.int32)
    num_blocks = 32
    table = torch.randint(0, num_blocks, (seqs, 9), dtype=torch.int32, generator=gen)
    q = rnd(seqs, Hq, D, dtype=torch.float16)
    kc, vc = rnd(num_blocks, Hkv, bs, D, dtype=torch.float16), rnd(num_blocks, Hkv, bs, D, dtype=torch.float16)
    monkeypatch.setattr(paged, "choose_launch", lambda *a: ("balanced", num_wgs))
    real_empty = torch.empty
    monkeypatch.setattr(torch, "empty", lambda *a, **kw: real_empty(*a, **kw).fill_(7) if kw.get("dtype") == q.dtype else real_empty(*a, **kw))
    out = flag_attn.paged_attention(q, kc, vc, ctx, table, D ** -0.5, 130)
    live = ctx > 0
    assert not out[~live].any()          # the output buffer started out as sevens
    ref = oracle_paged(q[live].float(), kc.float(), vc.float(), table[live], ctx[live], D ** -0.5)
    assert torch.allclose(out[live].float(), ref, atol=2e-3, rtol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_dense_forward_in_key_pieces(monkeypatch, causal):
    """A dense launch whose 256-row workgroups would leave half the compute units idle runs the 256-row kernel
    over pieces of the key axis and merges them (flash.wide_key_splits): the cross-length shape of the workload
    list in small.  The last piece ends in a partial tile."""
    B, H, Hk, M, N, D = 1, 2, 1, 300, 2100, 128
    monkeypatch.setattr(flash, "_num_cus", lambda: 8)
    assert flash.wide_key_splits(B, H, M, N, D, 8) == 2
    calls = []
    lib = _lib.get()

    class Spy:
        def __getattr__(self, name):
            fn = getattr(lib, name)
            if name in ("fa_fwd", "fa_splitkv_fwd", "fa_splitkv_combine"):
                return lambda *a: (calls.append(name), fn(*a))[1]
            return fn

    monkeypatch.setattr(_lib, "get", lambda: Spy())
    (q, k, v, do), ref, same, g_ref, g_same = flash_case(B, H, Hk, M, N, D, causal)
    o, L, *_ = flag_attn.flash_attention(q, k, v, causal=causal, return_log_normalizer=True)
    assert calls == ["fa_splitkv_fwd", "fa_splitkv_combine"]
    check("o", o, same[0], ref[0])
    check("L", L, same[1], ref[1])
    grads = torch.autograd.grad(o, (q, k, v), do)
    for name, h, s, r in zip(("dq", "dk", "dv"), grads, g_same, g_ref):
        check(name, h, s, r)


def test_key_pieces_that_some_rows_do_not_see():
    """The split entry point with at least 256 query rows runs the 256-row kernel per piece.  Under the causal mask
    with M = N the first row block sees nothing of the second piece: that piece reports zeros and a log-normalizer
    of -inf for those rows and drops out of the merge."""
    from flagattention_amd import _abi
    lib = _lib.get()
    B, H, M, N, D = 1, 1, 512, 512, 128
    (q, k, v, do), ref, same, _, _ = flash_case(B, H, H, M, N, D, True, dtype=torch.float16)
    part_o = torch.full((B, H, 2, M, D), float("nan"), dtype=torch.float16)
    part_lse = torch.full((B, H, 2, M), float("nan"), dtype=torch.float32)
    _abi.fa_splitkv_fwd(lib, q, k, v, part_o, part_lse, True, D ** -0.5, 2, 256)
    assert bool((part_lse[0, 0, 1, :256] == -math.inf).all()) and not part_o[0, 0, 1, :256].any()
    assert bool(torch.isfinite(part_lse[0, 0, 1, 256:]).all()) and bool(torch.isfinite(part_lse[0, 0, 0]).all())
    o, L = torch.empty_like(q), torch.empty(B, H, M)
    _abi.fa_splitkv_combine(lib, part_o, part_lse, o, L, 2)
    check("o", o, same[0], ref[0])
    check("L", L, same[1], ref[1])
