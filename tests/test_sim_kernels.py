"""Runs the unchanged kernel sources in the host lane simulator (tests/sim) and checks them against
the oracle under the 2x rule.  This covers, without a GPU: tile index arithmetic, key/query tails,
bottom-right causal masking, rows without keys, grouped heads, strided (BTHD) views, every head
size, both dtypes, the piecewise regime switch, split merging and block-table gathers -- through the
same C entry points and Python marshalling the GPU path uses.  Sizes are small: the simulator runs
one lane at a time.
"""
import math

import pytest
import torch

from flagattention_amd import _abi
from flagattention_amd.split_kv import _split_size
from oracle import (flash_attention, paged_attention, piecewise_attention, within_two_x)
from tests.sim import simlib

torch.manual_seed(10086)


@pytest.fixture(scope="module")
def lib():
    return simlib.get()


def rnd(shape, dtype, bthd=False, std=1.0):
    B, H, T, D = shape
    if bthd:
        return (torch.randn(B, T, H, D) * std).to(dtype).transpose(1, 2)
    return (torch.randn(B, H, T, D) * std).to(dtype)


def check(name, hyp, same, ref):
    ok, e_hyp, e_same = within_two_x(hyp, same, ref)
    assert ok, f"{name}: kernel err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


FLASH_CASES = [
    # B, H, Hk, M, N, D, causal, dtype, bthd
    (1, 2, 1, 100, 150, 128, True, torch.bfloat16, False),
    (1, 2, 2, 130, 70, 64, True, torch.float16, True),      # M > N: rows without keys
    (2, 2, 1, 70, 40, 32, False, torch.bfloat16, True),
    (1, 1, 1, 33, 200, 16, True, torch.float16, False),
    (1, 1, 1, 129, 129, 64, False, torch.bfloat16, False),
]


@pytest.mark.parametrize("B,H,Hk,M,N,D,causal,dtype,bthd", FLASH_CASES)
def test_flash_forward_backward_total(lib, B, H, Hk, M, N, D, causal, dtype, bthd):
    q = rnd((B, H, M, D), dtype, bthd).requires_grad_()
    k = rnd((B, Hk, N, D), dtype, bthd).requires_grad_()
    v = rnd((B, Hk, N, D), dtype, bthd).requires_grad_()
    do = rnd((B, H, M, D), dtype, bthd)
    sc = 1 / math.sqrt(D)
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    o = torch.full_like(qd, float("nan"))
    lse = torch.full((B, H, M), float("nan"))
    _abi.fa_fwd(lib, qd, kd, vd, o, lse, causal, sc)
    tot = torch.full((B, H, N), float("nan"))
    _abi.fa_total_attn(lib, qd, kd, lse, tot, causal, sc)
    delta = torch.full((B, H, M), float("nan"))
    _abi.fa_bwd_delta(lib, o, do, delta)
    dk = torch.full((B, Hk, N, D), float("nan"), dtype=dtype)   # group-summed by the kernel
    dv = torch.full((B, Hk, N, D), float("nan"), dtype=dtype)
    dq = torch.full((B, H, M, D), float("nan"), dtype=dtype)
    _abi.fa_bwd_dkdv(lib, qd, kd, vd, do, lse, delta, dk, dv, causal, sc)
    _abi.fa_bwd_dq(lib, qd, kd, vd, do, lse, delta, dq, causal, sc)

    ref = flash_attention(q, k, v, causal, upcast=True, return_log_normalizer=True, return_total_attention=True)
    same = flash_attention(q, k, v, causal, upcast=False, return_log_normalizer=True, return_total_attention=True)
    g_ref = torch.autograd.grad(ref[0], (q, k, v), do)
    g_same = torch.autograd.grad(same[0], (q, k, v), do)
    check("o", o, same[0], ref[0])
    check("lse", lse, same[1], ref[1])
    check("total", tot, same[2], ref[2])
    assert torch.allclose(delta, (o.float() * do.float()).sum(-1), atol=1e-4, rtol=1e-4)
    for name, h, s, r in zip(("dq", "dk", "dv"), (dq, dk, dv), g_same, g_ref):
        check(name, h, s, r)
    if causal and M > N:
        assert torch.all(o[:, :, : M - N] == 0) and torch.all(dq[:, :, : M - N] == 0)
        assert torch.all(torch.isinf(lse[:, :, : M - N]))


WIDE_CASES = [
    # B, H, Hk, M, N, causal, dtype, bthd, std
    (1, 1, 1, 64, 64, False, torch.bfloat16, False, 1.0),     # one tile
    (1, 2, 1, 100, 150, True, torch.bfloat16, False, 1.0),    # grouped heads, ragged rows and keys
    (1, 1, 1, 300, 300, True, torch.float16, True, 1.0),      # two row blocks, diagonal tiles, strided views
    (1, 1, 1, 40, 1, False, torch.float16, False, 1.0),       # a single key
    (1, 1, 1, 257, 520, True, torch.bfloat16, False, 1.0),    # steady loop, then masked tiles, then the last one
    (1, 1, 1, 256, 640, False, torch.float16, False, 4.0),    # large late scores: the reference maximum is raised late
    (1, 1, 1, 330, 130, True, torch.float16, False, 1.0),     # M > N: rows without keys
]


@pytest.mark.parametrize("B,H,Hk,M,N,causal,dtype,bthd,std", WIDE_CASES)
def test_flash_forward_256_row_kernel(lib, B, H, Hk, M, N, causal, dtype, bthd, std):
    """fa_fwd with block_m = 256: the slot-structured kernel with 64 query rows per wavefront (head
    size 128), against the oracle and against the 128-row kernel."""
    D = 128
    q, k, v = rnd((B, H, M, D), dtype, bthd, std), rnd((B, Hk, N, D), dtype, bthd, std), rnd((B, Hk, N, D), dtype, bthd)
    if std > 1:
        k[..., N // 2:, :] *= 1.5
    sc = 1 / math.sqrt(D)
    o = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, M), float("nan"))
    _abi.fa_fwd(lib, q, k, v, o, lse, causal, sc, block_m=256)
    ref = flash_attention(q, k, v, causal, upcast=True, return_log_normalizer=True)
    same = flash_attention(q, k, v, causal, upcast=False, return_log_normalizer=True)
    check("o", o, same[0], ref[0])
    check("lse", lse, same[1], ref[1])
    o128, lse128 = torch.empty_like(o), torch.empty_like(lse)
    _abi.fa_fwd(lib, q, k, v, o128, lse128, causal, sc, block_m=128)
    assert torch.equal(torch.isinf(lse), torch.isinf(lse128))
    fin = torch.isfinite(lse)
    assert (lse[fin] - lse128[fin]).abs().max() < 1e-4
    if causal and M > N:
        assert torch.all(o[:, :, : M - N] == 0) and torch.all(torch.isinf(lse[:, :, : M - N]))


def test_flash_forward_tile_argument_is_checked(lib):
    q = rnd((1, 1, 64, 64), torch.float16)
    o, lse = torch.empty_like(q), torch.empty(1, 1, 64)
    with pytest.raises(AssertionError):   # the 256-row kernel exists for head size 128 only
        _abi.fa_fwd(lib, q, q, q, o, lse, False, 0.125, block_m=256)
    with pytest.raises(AssertionError):   # no such tile
        _abi.fa_fwd(lib, q, q, q, o, lse, False, 0.125, block_m=64)
    _abi.fa_fwd(lib, q, q, q, o, lse, False, 0.125, block_m=128)


DS_CASES = [
    # B, H, Hk, M, N, D, causal, dtype, bthd
    (1, 2, 1, 100, 150, 128, True, torch.bfloat16, False),
    (1, 2, 2, 130, 70, 64, True, torch.float16, True),      # M > N: rows without keys
    (2, 1, 1, 70, 200, 32, False, torch.bfloat16, True),
    (1, 1, 1, 257, 129, 16, True, torch.float16, False),    # three query blocks, key tail of one
    (1, 1, 1, 270, 200, 128, False, torch.bfloat16, False), # head 128: four whole query tiles and a tail (slotted body)
    (1, 2, 1, 200, 260, 128, True, torch.float16, True),    # head 128, causal, grouped heads
]


@pytest.mark.parametrize("B,H,Hk,M,N,D,causal,dtype,bthd", DS_CASES)
def test_flash_backward_with_stored_ds(lib, B, H, Hk, M, N, D, causal, dtype, bthd):
    """dK/dV kernel that leaves dS in the workspace + dQ computed from it, against the oracle and
    against the recomputing dQ kernel (the two round dS to the input dtype at the same place)."""
    q = rnd((B, H, M, D), dtype, bthd).requires_grad_()
    k = rnd((B, Hk, N, D), dtype, bthd).requires_grad_()
    v = rnd((B, Hk, N, D), dtype, bthd).requires_grad_()
    do = rnd((B, H, M, D), dtype, bthd)
    sc = 1 / math.sqrt(D)
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    o = torch.full_like(qd, float("nan"))
    lse = torch.full((B, H, M), float("nan"))
    _abi.fa_fwd(lib, qd, kd, vd, o, lse, causal, sc)
    delta = torch.full((B, H, M), float("nan"))
    _abi.fa_bwd_delta(lib, o, do, delta)
    dk = torch.full((B, Hk, N, D), float("nan"), dtype=dtype)   # group-summed by the kernel
    dv = torch.full((B, Hk, N, D), float("nan"), dtype=dtype)
    dq = torch.full((B, H, M, D), float("nan"), dtype=dtype)
    mib = lib.fa_bwd_ds_workspace_mib(B, H, M, N)
    assert mib > 0
    ds = torch.full((mib << 19,), float("nan"), dtype=dtype)   # unwritten chunks hold NaN
    _abi.fa_bwd_dkdv_ds(lib, qd, kd, vd, do, lse, delta, dk, dv, ds, causal, sc)
    _abi.fa_bwd_dq_from_ds(lib, kd, ds, dq, causal, sc)
    dk_plain, dv_plain = torch.empty_like(dk), torch.empty_like(dv)
    dq_plain = torch.empty_like(dq)
    _abi.fa_bwd_dkdv(lib, qd, kd, vd, do, lse, delta, dk_plain, dv_plain, causal, sc)
    _abi.fa_bwd_dq(lib, qd, kd, vd, do, lse, delta, dq_plain, causal, sc)
    assert torch.equal(dk, dk_plain) and torch.equal(dv, dv_plain)
    assert not torch.isnan(dq).any()
    ref = flash_attention(q, k, v, causal, upcast=True)
    same = flash_attention(q, k, v, causal, upcast=False)
    g_ref = torch.autograd.grad(ref, (q, k, v), do)
    g_same = torch.autograd.grad(same, (q, k, v), do)
    check("dq", dq, g_same[0], g_ref[0])
    check("dk", dk, g_same[1], g_ref[1])
    check("dv", dv, g_same[2], g_ref[2])
    # same products, same rounding of dS; only the summation order over keys inside the MFMA differs
    assert (dq.float() - dq_plain.float()).abs().max() <= 2e-2 * dq_plain.float().abs().max() + 1e-6


@pytest.mark.parametrize("dtype,causal,M,N", [
    (torch.float16, False, 64, 40), (torch.float16, False, 128, 200), (torch.float16, True, 100, 170),
    (torch.bfloat16, False, 64, 40)])
def test_stored_ds_is_zero_for_keys_past_the_end(lib, dtype, causal, M, N):
    """Head size 128, a key count that is no multiple of 32 and strongly negative log-normalizers: the
    lanes of keys past N see zero K/V rows, so exp2(score - L) there is exp(-L), far above fp16's range
    once rounded.  The dK/dV kernel must leave exact zeroes for them in the dS workspace, or the
    dQ-from-dS kernel multiplies infinities by its zeroed K rows."""
    D, sc = 128, 128 ** -0.5
    q = (torch.randn(1, 1, M, D) * 0.1 + 1.0).to(dtype)
    k = (torch.randn(1, 1, N, D) * 0.1 - 1.8).to(dtype)
    v = torch.randn(1, 1, N, D).to(dtype)
    do = torch.randn(1, 1, M, D).to(dtype)
    o = torch.empty_like(q)
    lse = torch.empty(1, 1, M)
    _abi.fa_fwd(lib, q, k, v, o, lse, causal, sc)
    assert lse.max() < -11.5   # exp(-L) does not fit fp16
    delta = torch.empty(1, 1, M)
    _abi.fa_bwd_delta(lib, o, do, delta)
    dk, dv, dq, dq_plain = (torch.empty_like(t) for t in (k, v, q, q))
    ds = torch.full((lib.fa_bwd_ds_workspace_mib(1, 1, M, N) << 19,), float("nan"), dtype=dtype)
    _abi.fa_bwd_dkdv_ds(lib, q, k, v, do, lse, delta, dk, dv, ds, causal, sc)
    _abi.fa_bwd_dq_from_ds(lib, k, ds, dq, causal, sc)
    _abi.fa_bwd_dq(lib, q, k, v, do, lse, delta, dq_plain, causal, sc)
    assert torch.isfinite(dq.float()).all()
    assert (dq.float() - dq_plain.float()).abs().max() <= 2e-2 * dq_plain.float().abs().max() + 1e-6


@pytest.mark.parametrize("B,H,M,N,pd,seed,offset", [
    (1, 2, 7, 33, 0.3, 1234, 40),                                   # 462 elements: a vector tail
    (2, 1, 16, 16, 0.5, 987654321987, 123456789123456789),          # 64-bit counter, whole vectors only
    (1, 1, 3, 5, 0.9, 7, (1 << 32) - 4),                             # the counter's low word wraps
])
def test_dropout_mask_kernel_is_bit_exact_with_the_oracle(lib, B, H, M, N, pd, seed, offset):
    """fa_dropout_mask (the reference's recompute_mask_kernel, testing/dropout.py:5-25) against the
    numpy restatement of Triton's Philox in oracle/dropout.py."""
    from oracle import keep_mask
    mask = torch.zeros((B, H, M, N), dtype=torch.bool)
    _abi.fa_dropout_mask(lib, mask, pd, seed, offset)
    assert torch.equal(mask, keep_mask(B, H, M, N, pd, seed, offset))


DROPOUT_CASES = [
    # B, H, Hk, M, N, D, causal, dtype, p, seed, offset
    (1, 2, 1, 70, 100, 64, True, torch.bfloat16, 0.3, 1234, 40),
    (2, 1, 1, 40, 40, 128, False, torch.float16, 0.5, 987654321987, 123456789123456789),   # 64-bit counter
    (1, 2, 2, 130, 70, 32, True, torch.float16, 0.1, 7, 0),                               # rows without keys
]


@pytest.mark.parametrize("B,H,Hk,M,N,D,causal,dtype,pd,seed,offset", DROPOUT_CASES)
def test_flash_dropout(lib, B, H, Hk, M, N, D, causal, dtype, pd, seed, offset):
    """Forward, both backward routes (dS recomputed / dS kept) with dropout, against the oracle given
    the mask that oracle.dropout restates from (seed, offset)."""
    from oracle import keep_mask
    q = rnd((B, H, M, D), dtype).requires_grad_()
    k = rnd((B, Hk, N, D), dtype).requires_grad_()
    v = rnd((B, Hk, N, D), dtype).requires_grad_()
    do = rnd((B, H, M, D), dtype)
    sc = 1 / math.sqrt(D)
    drop = (pd, seed, offset)
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    o = torch.full_like(qd, float("nan"))
    lse = torch.full((B, H, M), float("nan"))
    _abi.fa_fwd(lib, qd, kd, vd, o, lse, causal, sc, drop)
    delta = torch.full((B, H, M), float("nan"))
    _abi.fa_bwd_delta(lib, o, do, delta)
    # with dropout the kernels leave one dK/dV slice per query head
    dk, dv = torch.empty(B, H, N, D, dtype=dtype), torch.empty(B, H, N, D, dtype=dtype)
    dq = torch.empty(B, H, M, D, dtype=dtype)
    if H > Hk:
        with pytest.raises(AssertionError):
            _abi.fa_bwd_dkdv(lib, qd, kd, vd, do, lse, delta, dk[:, :Hk], dv[:, :Hk], causal, sc, drop)
    _abi.fa_bwd_dkdv(lib, qd, kd, vd, do, lse, delta, dk, dv, causal, sc, drop)
    _abi.fa_bwd_dq(lib, qd, kd, vd, do, lse, delta, dq, causal, sc, drop)
    dk2, dv2, dq2 = torch.empty_like(dk), torch.empty_like(dv), torch.empty_like(dq)
    ds = torch.full((lib.fa_bwd_ds_workspace_mib(B, H, M, N) << 19,), float("nan"), dtype=dtype)
    _abi.fa_bwd_dkdv_ds(lib, qd, kd, vd, do, lse, delta, dk2, dv2, ds, causal, sc, drop)
    _abi.fa_bwd_dq_from_ds(lib, kd, ds, dq2, causal, sc)
    assert torch.equal(dk, dk2) and torch.equal(dv, dv2)
    dk, dv = dk.reshape(B, Hk, H // Hk, N, D).sum(2), dv.reshape(B, Hk, H // Hk, N, D).sum(2)

    mask = keep_mask(B, H, M, N, pd, seed, offset)
    assert 0 < (~mask).float().mean() < 1
    ref = flash_attention(q, k, v, causal, upcast=True, return_log_normalizer=True, dropout_p=pd, dropout_mask=mask)
    same = flash_attention(q, k, v, causal, upcast=False, return_log_normalizer=True, dropout_p=pd, dropout_mask=mask)
    g_ref = torch.autograd.grad(ref[0], (q, k, v), do)
    g_same = torch.autograd.grad(same[0], (q, k, v), do)
    check("o", o, same[0], ref[0])
    check("lse", lse, same[1], ref[1])
    for name, h, s_, r in (("dq", dq, g_same[0], g_ref[0]), ("dq (dS kept)", dq2, g_same[0], g_ref[0]),
                           ("dk", dk, g_same[1], g_ref[1]), ("dv", dv, g_same[2], g_ref[2])):
        check(name, h, s_, r)
    # a different seed gives a different output: the mask is really applied
    o2 = torch.empty_like(o)
    _abi.fa_fwd(lib, qd, kd, vd, o2, lse, causal, sc, (pd, seed + 1, offset))
    assert not torch.equal(o, o2)


PW_CASES = [
    # B, H, M, N, D, w, causal, dtype
    (1, 2, 200, 200, 64, 50, True, torch.bfloat16),
    (1, 1, 130, 260, 32, 100, False, torch.float16),
    (1, 1, 260, 130, 16, 190, True, torch.bfloat16),
    (1, 1, 150, 150, 128, -20, False, torch.float16),
    (1, 1, 300, 300, 32, 70, True, torch.float16),      # threshold crosses several row and key blocks
    (1, 1, 140, 200, 64, 0, True, torch.bfloat16),      # every visible pair is far
    (1, 1, 140, 140, 16, 1000, True, torch.float16),    # every pair is near
    (1, 1, 70, 330, 32, -1000, False, torch.bfloat16),  # non-causal, every pair far
    (1, 1, 330, 70, 32, 129, False, torch.float16),     # M > N, threshold on a block edge
    (2, 2, 200, 330, 128, 64, True, torch.bfloat16),    # head size 128, threshold on a block edge, two heads
    (1, 1, 270, 300, 128, 200, False, torch.bfloat16),  # head size 128: whole tiles in the near regime, and in the far one
    # thresholds of 95 and more with head sizes 128 and 64: every tile of the backward in slots, the ones a regime
    # begins or ends in with one select per element
    (1, 2, 330, 330, 128, 100, True, torch.bfloat16),
    (1, 1, 300, 400, 64, 130, True, torch.float16),
    (1, 1, 260, 300, 64, 95, False, torch.bfloat16),
    (1, 1, 330, 290, 128, 95, True, torch.float16),     # M > N, key tail block beside blocks in slots
]


@pytest.mark.parametrize("B,H,M,N,D,w,causal,dtype", PW_CASES)
def test_piecewise_forward_backward(lib, B, H, M, N, D, w, causal, dtype):
    ts = [rnd((B, H, M if i in (0, 2) else N, D), dtype).requires_grad_() for i in range(5)]
    do = rnd((B, H, M, D), dtype)
    sc = 1 / math.sqrt(D)
    d = [t.detach() for t in ts]
    o = torch.full_like(d[0], float("nan"))
    lse = torch.full((B, H, M), float("nan"))
    _abi.pw_fwd(lib, *d, o, lse, w, causal, sc)
    delta = torch.empty(B, H, M)
    _abi.fa_bwd_delta(lib, o, do, delta)
    dk1, dk2, dv = (torch.full_like(d[1], float("nan")) for _ in range(3))
    dq1, dq2 = (torch.full_like(d[0], float("nan")) for _ in range(2))
    _abi.pw_bwd_dkdv(lib, *d, do, lse, delta, dk1, dk2, dv, w, causal, sc)
    _abi.pw_bwd_dq(lib, *d, do, lse, delta, dq1, dq2, w, causal, sc)
    ref = piecewise_attention(*ts, w, causal, upcast=True)
    g_ref = torch.autograd.grad(ref, ts, do)
    same = piecewise_attention(*ts, w, causal, upcast=False)
    g_same = torch.autograd.grad(same, ts, do)
    check("o", o, same, ref)
    for name, h, s, r in zip(("dq1", "dk1", "dq2", "dk2", "dv"), (dq1, dk1, dq2, dk2, dv), g_same, g_ref):
        check(name, h, s, r)
    # the same backward with dS handed over in the workspace (unwritten chunks hold NaN)
    mib = lib.fa_bwd_ds_workspace_mib(B, H, M, N)
    ds = torch.full((2 * (mib << 19),), float("nan"), dtype=dtype)
    ek1, ek2, ev = (torch.full_like(d[1], float("nan")) for _ in range(3))
    eq1, eq2 = (torch.full_like(d[0], float("nan")) for _ in range(2))
    _abi.pw_bwd_dkdv_ds(lib, *d, do, lse, delta, ek1, ek2, ev, ds, w, causal, sc)
    _abi.pw_bwd_dq_from_ds(lib, d[1], d[3], ds, eq1, eq2, w, causal, sc)
    assert torch.equal(ek1, dk1) and torch.equal(ek2, dk2) and torch.equal(ev, dv)
    assert not torch.isnan(eq1).any() and not torch.isnan(eq2).any()
    check("dq1 from dS", eq1, g_same[0], g_ref[0])
    check("dq2 from dS", eq2, g_same[2], g_ref[2])
    for e, h in ((eq1, dq1), (eq2, dq2)):
        assert (e.float() - h.float()).abs().max() <= 2e-2 * h.float().abs().max() + 1e-6


SPLIT_CASES = [
    (2, 4, 2, 1, 612, 128, False, 3, torch.float16),
    (1, 4, 1, 2, 400, 64, True, 2, torch.bfloat16),
    (1, 2, 2, 4, 300, 16, True, 4, torch.float16),
    (1, 40, 1, 1, 200, 32, False, 2, torch.bfloat16),   # 40 rows share one kv head: two row blocks
    (1, 2, 2, 40, 100, 64, True, 2, torch.float16),     # early rows see no key of the late split
]


@pytest.mark.parametrize("B,H,Hk,M,N,D,causal,S,dtype", SPLIT_CASES)
def test_split_kv_and_merge(lib, B, H, Hk, M, N, D, causal, S, dtype):
    q, k, v = rnd((B, H, M, D), dtype, std=3), rnd((B, Hk, N, D), dtype, std=3), rnd((B, Hk, N, D), dtype, std=3)
    sc = 1 / math.sqrt(D)
    po = torch.full((B, H, S, M, D), float("nan"), dtype=torch.float16)
    pl = torch.full((B, H, S, M), float("nan"))
    _abi.fa_splitkv_fwd(lib, q, k, v, po, pl, causal, sc, S, _split_size(N, S))
    o = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, M), float("nan"))
    _abi.fa_splitkv_combine(lib, po, pl, o, lse, S)
    ref = flash_attention(q, k, v, causal, upcast=True, return_log_normalizer=True)
    same = flash_attention(q, k, v, causal, upcast=False, return_log_normalizer=True)
    check("o", o, same[0], ref[0])
    check("lse", lse, same[1], ref[1])
    assert not torch.isnan(po).any()


PAGED_CASES = [
    # seqs, Hq, G, D, block, max_len, splits, partition, dtype, table dtype
    (3, 8, 1, 64, 16, 100, 1, 0, torch.float16, torch.int64),
    (3, 8, 4, 128, 16, 300, 1, 0, torch.float16, torch.int64),
    (2, 8, 8, 32, 16, 300, 3, 128, torch.float16, torch.int32),
    (2, 4, 1, 64, 16, 2, 1, 0, torch.float16, torch.int64),
    (2, 6, 2, 16, 32, 200, 2, 128, torch.bfloat16, torch.int64),
    (1, 40, 40, 64, 16, 70, 2, 64, torch.float16, torch.int64),
    (2, 4, 2, 256, 16, 150, 1, 0, torch.float16, torch.int64),
    (2, 4, 2, 512, 16, 150, 1, 0, torch.float16, torch.int64),   # 16-key steps
    (2, 2, 1, 512, 16, 200, 2, 128, torch.bfloat16, torch.int32),
]


@pytest.mark.parametrize("seqs,Hq,G,D,bs,max_len,splits,psize,dtype,tdtype", PAGED_CASES)
def test_paged_attention_and_reduce(lib, seqs, Hq, G, D, bs, max_len, splits, psize, dtype, tdtype):
    Hk = Hq // G
    lens = torch.randint(1, max_len + 1, (seqs,), dtype=torch.int32)
    lens[0] = max_len
    nb = 50
    sc = D ** -0.5
    q = torch.empty(seqs, Hq, D).uniform_(-sc, sc).to(dtype)
    kc = torch.empty(nb, Hk, bs, D).uniform_(-sc, sc).to(dtype)
    vc = torch.empty(nb, Hk, bs, D).uniform_(-sc, sc).to(dtype)
    bt = torch.randint(0, nb, (seqs, (max_len + bs - 1) // bs)).to(tdtype)
    out = torch.full_like(q, float("nan"))
    if splits == 1:
        _abi.paged_attn(lib, out, q, kc, vc, lens, bt, sc, 0, 1, None, None, None)
    else:
        shape = (seqs, Hk, splits, G)
        ml, es = torch.full(shape, float("nan")), torch.full(shape, float("nan"))
        tmp = torch.full(shape + (D,), float("nan"), dtype=dtype)
        _abi.paged_attn(lib, out, q, kc, vc, lens, bt, sc, psize, splits, tmp, ml, es)
        _abi.paged_reduce(lib, out, tmp, ml, es, lens, Hk, psize, splits)
    ref = paged_attention(q, kc, vc, bt, lens, sc)
    same = paged_attention(q, kc, vc, bt, lens, sc, same_precision=True)
    check("out", out, same, ref)
    if dtype == torch.float16:
        assert torch.allclose(out, ref, atol=2e-3, rtol=1e-5)


BALANCED_CASES = [
    # seqs, Hq, G, D, block, lens, workgroups, dtype, table dtype
    (4, 4, 2, 64, 16, [700, 1, 300, 129], 7, torch.float16, torch.int64),   # pairs cut at both ends
    (3, 2, 1, 128, 16, [1000, 0, 260], 3, torch.float16, torch.int32),      # an empty sequence
    (2, 40, 40, 32, 8, [200, 90], 4, torch.bfloat16, torch.int64),          # 3 row blocks per kv head
    (5, 2, 2, 16, 16, [40, 50, 60, 70, 80], 64, torch.float16, torch.int64),  # more workgroups than work
    (1, 2, 1, 64, 16, [1500], 5, torch.float16, torch.int64),               # one pair over many workgroups
    (2, 4, 4, 512, 16, [300, 77], 3, torch.float16, torch.int64),           # 16-key steps
]


@pytest.mark.parametrize("seqs,Hq,G,D,bs,lens,wgs,dtype,tdtype", BALANCED_CASES)
def test_paged_attention_balanced(lib, seqs, Hq, G, D, bs, lens, wgs, dtype, tdtype):
    Hk = Hq // G
    lens = torch.tensor(lens, dtype=torch.int32)
    max_len = int(lens.max())
    nb = 120
    sc = D ** -0.5
    q = torch.empty(seqs, Hq, D).uniform_(-sc, sc).to(dtype)
    kc = torch.empty(nb, Hk, bs, D).uniform_(-sc, sc).to(dtype)
    vc = torch.empty(nb, Hk, bs, D).uniform_(-sc, sc).to(dtype)
    bt = torch.randint(0, nb, (seqs, (max_len + bs - 1) // bs)).to(tdtype)
    out = torch.full_like(q, float("nan"))
    nbytes = lib.paged_attn_balanced_workspace(wgs, D)
    assert nbytes > 0
    ws = torch.full((nbytes // 4,), float("nan"))
    _abi.paged_attn_balanced(lib, out, q, kc, vc, lens, bt, sc, ws, wgs)
    live = lens > 0
    assert (out[~live] == 0).all()
    ref = paged_attention(q[live], kc, vc, bt[live], lens[live], sc)
    same = paged_attention(q[live], kc, vc, bt[live], lens[live], sc, same_precision=True)
    check("out", out[live], same, ref)
    if dtype == torch.float16:
        assert torch.allclose(out[live], ref, atol=2e-3, rtol=1e-5)


def test_paged_attention_balanced_static_scratch(lib):
    """The entry point without a workspace argument (static scratch inside the library) against the one
    with a caller-provided workspace: bit-equal, on two calls in a row, the second one smaller, with the
    scratch still holding the first call's partial results; and the size limit is enforced."""
    from flagattention_amd import _lib
    calls = [  # seqs, Hq, G, D, block, lens, workgroups
        (4, 4, 2, 64, 16, [700, 1, 300, 129], 7),
        (2, 4, 2, 64, 16, [130, 260], 3),
    ]
    for seqs, Hq, G, D, bs, lens, wgs in calls:
        Hk = Hq // G
        lens = torch.tensor(lens, dtype=torch.int32)
        nb, sc = 60, D ** -0.5
        q = torch.empty(seqs, Hq, D).uniform_(-sc, sc).to(torch.float16)
        kc = torch.empty(nb, Hk, bs, D).uniform_(-sc, sc).to(torch.float16)
        vc = torch.empty(nb, Hk, bs, D).uniform_(-sc, sc).to(torch.float16)
        bt = torch.randint(0, nb, (seqs, (int(lens.max()) + bs - 1) // bs))
        out_ws = torch.full_like(q, float("nan"))
        ws = torch.full((lib.paged_attn_balanced_workspace(wgs, D) // 4,), float("nan"))
        _abi.paged_attn_balanced(lib, out_ws, q, kc, vc, lens, bt, sc, ws, wgs)
        out_static = torch.full_like(q, float("nan"))
        _abi.paged_attn_balanced_static(lib, out_static, q, kc, vc, lens, bt, sc, wgs)
        assert torch.equal(out_ws, out_static)
        ref = paged_attention(q, kc, vc, bt, lens, sc)
        assert torch.allclose(out_static, ref, atol=2e-3, rtol=1e-5)
    # 4096 workgroups at head size 64 need 4096 * 8464 bytes: more than the array holds
    assert lib.paged_attn_balanced_workspace(4096, D) > _lib.STATIC_SCRATCH_BYTES
    with pytest.raises(AssertionError, match="scratch"):
        _abi.paged_attn_balanced_static(lib, out_static, q, kc, vc, lens, bt, sc, 4096)
    # the sizes the host wrapper launches fit: one resident wave of a 256-CU device
    assert lib.paged_attn_balanced_workspace(512, 128) <= _lib.STATIC_SCRATCH_BYTES
    assert lib.paged_attn_balanced_workspace(256, 512) <= _lib.STATIC_SCRATCH_BYTES


def test_entry_points_reject_bad_arguments(lib):
    q = rnd((1, 2, 32, 64), torch.float16)
    k = rnd((1, 2, 32, 64), torch.float16)
    o = torch.empty_like(q)
    lse = torch.empty(1, 2, 32)
    with pytest.raises(AssertionError):  # head size outside {16, 32, 64, 128}
        _abi.fa_fwd(lib, q[..., :48].contiguous(), k[..., :48].contiguous(), k[..., :48].contiguous(),
                    o[..., :48].contiguous(), lse, False, 1.0)
    with pytest.raises(AssertionError):  # 3 query heads over 2 kv heads
        _abi.fa_fwd(lib, rnd((1, 3, 32, 64), torch.float16), k, k, rnd((1, 3, 32, 64), torch.float16),
                    torch.empty(1, 3, 32), False, 1.0)


def test_matrix_pipe_probe_runs_and_fills_its_sink():
    """The rate probe of the benchmark: one float per thread comes back; constant operands give a value that can be
    written down -- per wavefront accumulator, iters * 4 products of A (rows (lane + e) & 3) and B (+-0.5)."""
    from flagattention_amd import _abi
    lib = simlib.get()
    cus = lib.fa_num_cus()
    sink = torch.full((cus * 256,), float("nan"))
    flop = _abi.fa_probe_mfma(lib, sink, 1, random_operands=False)
    assert flop == cus * 4 * 16 * 32768
    assert bool(torch.isfinite(sink).all()) and bool((sink == sink[:256].repeat(cus)).all())
    _abi.fa_probe_mfma(lib, sink, 1, random_operands=True)
    assert bool(torch.isfinite(sink).all()) and sink.abs().max() > 0
    with pytest.raises(AssertionError):
        _abi.fa_probe_mfma(lib, sink[:10], 1)
