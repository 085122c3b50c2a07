"""GPU parity tests of piecewise_attention, forward and backward.

Shapes and the threshold rule follow tests/flag_attn/test_piecewise_attention.py:12-124 of the
reference.  Acceptance: max|x_hip - x_fp32| <= 2 * max|x_torch_same_precision - x_fp32| + 1e-5 for
o, dq1, dk1, dq2, dk2, dv.
"""
import pytest
import torch

import flagattention_amd as flag_attn
from oracle import piecewise_attention as oracle_pw, flash_attention as oracle_flash, within_two_x

pytestmark = pytest.mark.gpu

SHAPES = [
    (2, 4, 512, 612, 128), (2, 4, 1024, 1034, 64), (2, 4, 2048, 2048, 32), (2, 4, 4096, 4096, 16),
    (2, 4, 4096, 4001, 16), (1, 2, 8192, 8192, 16), (1, 2, 8192, 8192, 32), (1, 2, 8192, 3867, 32),
]


def make(shape, dtype, order, std, seed, grad=False):
    g = torch.Generator(device="cuda").manual_seed(seed)
    B, H, T, D = shape
    if order == "BHTD":
        t = torch.empty((B, H, T, D), dtype=dtype, device="cuda").normal_(0.0, std, generator=g)
    else:
        t = torch.empty((B, T, H, D), dtype=dtype, device="cuda").normal_(0.0, std, generator=g).transpose(1, 2)
    return t.requires_grad_() if grad else t


def inputs(B, H, M, N, D, dtype, order, scale, grad):
    return (make((B, H, M, D), dtype, order, scale, 1, grad), make((B, H, N, D), dtype, order, scale, 2, grad),
            make((B, H, M, D), dtype, order, scale, 3, grad), make((B, H, N, D), dtype, order, scale, 4, grad),
            make((B, H, N, D), dtype, order, scale, 5, grad))


def check(name, hyp, same, ref):
    ok, e_hyp, e_same = within_two_x(hyp, same, ref)
    assert ok, f"{name}: hip err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


@pytest.mark.parametrize("scale", [1.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("B,H,M,N,D", SHAPES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attention_fwd(B, H, M, N, D, causal, order, dtype, scale):
    q1, k1, q2, k2, v = inputs(B, H, M, N, D, dtype, order, scale, False)
    w = (M // 2) if M < N else (M - N // 2)
    ref = oracle_pw(q1, k1, q2, k2, v, w, causal=causal, upcast=True)
    same = oracle_pw(q1, k1, q2, k2, v, w, causal=causal)
    hyp = flag_attn.piecewise_attention(q1, k1, q2, k2, v, w, causal=causal)
    check("o", hyp, same, ref)


@pytest.mark.parametrize("scale", [1.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("B,H,M,N,D", SHAPES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attention_bwd(B, H, M, N, D, causal, order, dtype, scale):
    ts = inputs(B, H, M, N, D, dtype, order, scale, True)
    do = make((B, H, M, D), dtype, order, scale, 6)
    w = (M // 2) if M < N else (M - N // 2)
    o_ref = oracle_pw(*ts, w, causal=causal, upcast=True)
    g_ref = torch.autograd.grad(o_ref, ts, do)
    o_same = oracle_pw(*ts, w, causal=causal, upcast=False)
    g_same = torch.autograd.grad(o_same, ts, do)
    o_hyp = flag_attn.piecewise_attention(*ts, w, causal=causal)
    g_hyp = torch.autograd.grad(o_hyp, ts, do)
    check("o", o_hyp, o_same, o_ref)
    for name, h, s, r in zip(("dq1", "dk1", "dq2", "dk2", "dv"), g_hyp, g_same, g_ref):
        check(name, h, s, r)


@pytest.mark.parametrize("causal", [True, False])
def test_reduces_to_flash_when_threshold_is_out_of_range(causal):
    """A threshold above (below) every distance must give plain attention on the first (second)
    pair; checked with the 2x rule against the flash oracle."""
    q1, k1, q2, k2, v = inputs(1, 2, 700, 900, 64, torch.bfloat16, "BHTD", 1.0, False)
    near = flag_attn.piecewise_attention(q1, k1, q2, k2, v, 900, causal=causal)
    far = flag_attn.piecewise_attention(q1, k1, q2, k2, v, -900, causal=causal)
    check("near", near, oracle_flash(q1, k1, v, causal), oracle_flash(q1, k1, v, causal, upcast=True))
    check("far", far, oracle_flash(q2, k2, v, causal), oracle_flash(q2, k2, v, causal, upcast=True))


@pytest.mark.parametrize("M,N,w,causal", [
    (1100, 1300, 300, True),      # threshold inside blocks
    (1024, 1024, 256, True),      # threshold on a block edge
    (1200, 1100, 0, True),        # M > N: rows without keys; every visible pair far
    (1100, 1300, -100, False),    # non-causal: future keys within 100 are far as well
    (1100, 1300, 5000, False),    # every pair near: the far grid stays unread
])
def test_backward_with_stored_ds(monkeypatch, M, N, w, causal):
    """Head size 128 and >= 2^20 scores: the dK/dV kernel leaves dS in a workspace (one chunk grid per
    regime) for the dQ kernels.  Checked against the oracle, against the recomputing route, and with
    a workspace bound that forces one (batch, head) slice per launch."""
    from flagattention_amd import flash
    B, H, D, dtype = 2, 2, 128, torch.bfloat16
    ts = inputs(B, H, M, N, D, dtype, "BTHD", 1.0, True)
    do = make((B, H, M, D), dtype, "BHTD", 1.0, 6)
    assert flash.ds_heads_per_launch(flag_attn._lib.get(), B, H, 1, M, N, D, grids=2) >= B * H
    g_ds = torch.autograd.grad(flag_attn.piecewise_attention(*ts, w, causal=causal), ts, do)
    g_ref = torch.autograd.grad(oracle_pw(*ts, w, causal=causal, upcast=True), ts, do)
    g_same = torch.autograd.grad(oracle_pw(*ts, w, causal=causal, upcast=False), ts, do)
    for name, h, s, r in zip(("dq1", "dk1", "dq2", "dk2", "dv"), g_ds, g_same, g_ref):
        assert not torch.isnan(h).any(), name
        check(name, h, s, r)
    per_slice = 2 * flag_attn._lib.get().fa_bwd_ds_workspace_mib(1, 1, M, N)
    monkeypatch.setattr(flash, "DS_WORKSPACE_LIMIT_MIB", per_slice)
    g_sliced = torch.autograd.grad(flag_attn.piecewise_attention(*ts, w, causal=causal), ts, do)
    monkeypatch.setattr(flash, "DS_WORKSPACE_LIMIT_MIB", 0)
    g_rec = torch.autograd.grad(flag_attn.piecewise_attention(*ts, w, causal=causal), ts, do)
    for name, a, b, c in zip(("dq1", "dk1", "dq2", "dk2", "dv"), g_ds, g_sliced, g_rec):
        assert torch.equal(a, b), name          # same kernels on slices
        if name.startswith("dq"):  # same products and rounding; the summation order inside the MFMA differs
            assert (a.float() - c.float()).abs().max() <= 2e-2 * c.float().abs().max() + 1e-6, name
        else:
            assert torch.equal(a, c), name
