"""The ways the reference's own example scripts call the operators (examples/*.py), through the
reference's package name: tensors created under a default device and dtype, int64 block tables from
``torch.randint``, the 5-tuple of auxiliary outputs, a replaced ``get_fwd_config`` hook, and the
piecewise call with its threshold as a positional argument.  Results are checked with the 2x rule
against the oracle.
"""
import pytest
import torch

import flag_attn
from oracle import flash_attention as oracle_flash, piecewise_attention as oracle_pw
from oracle import paged_attention as oracle_paged, within_two_x

pytestmark = pytest.mark.gpu


def check(name, hyp, same, ref):
    ok, e_hyp, e_same = within_two_x(hyp, same, ref)
    assert ok, f"{name}: hip err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


def test_paged_call_under_default_device_and_dtype():
    """examples/paged_example.py:20-52: everything allocated through torch's defaults."""
    old_dtype = torch.get_default_dtype()
    try:
        torch.set_default_dtype(torch.float16)
        torch.set_default_device("cuda:0")
        torch.cuda.manual_seed(0)
        num_seqs, hq, hkv, D, bs, num_blocks, max_len = 7, 16, 4, 128, 16, 2000, 4096
        lens = torch.randint(1, max_len, [num_seqs], dtype=torch.int32)
        max_ctx = lens.max().item()
        scale = D ** -0.5
        q = torch.empty(num_seqs, hq, D).uniform_(-scale, scale)
        kc = torch.empty(num_blocks, hkv, bs, D).uniform_(-scale, scale)
        vc = torch.empty_like(kc).uniform_(-scale, scale)
        table = torch.randint(0, num_blocks, (num_seqs, (max_ctx + bs - 1) // bs))
        out = flag_attn.paged_attention(q, kc, vc, lens, table, scale, max_ctx)
    finally:
        torch.set_default_device(None)
        torch.set_default_dtype(old_dtype)
    ref = oracle_paged(q, kc, vc, table, lens, scale)
    assert out.dtype == torch.float16 and out.shape == q.shape
    assert torch.allclose(out.float(), ref.float(), atol=2e-3, rtol=1e-5)


def test_auxiliary_outputs_come_as_a_five_tuple():
    """examples/flash_attention_with_aux_outputs.py (which unpacks three values; the reference returns
    five, src/flag_attn/flash.py:150-160)."""
    B, H, M, N, D = 2, 4, 10, 20, 128
    q, k, v = (torch.randn((B, H, T, D), dtype=torch.bfloat16, device="cuda", requires_grad=True) for T in (M, N, N))
    res = flag_attn.flash_attention(q, k, v, causal=False, return_log_normalizer=True, return_total_attention=True)
    assert isinstance(res, tuple) and len(res) == 5 and res[3] is None and res[4] is None
    o, logz, tot = res[:3]
    ref = oracle_flash(q, k, v, False, upcast=True, return_log_normalizer=True, return_total_attention=True)
    same = oracle_flash(q, k, v, False, upcast=False, return_log_normalizer=True, return_total_attention=True)
    for name, h, s, r in zip(("o", "log_normalizer", "total_attention"), (o, logz, tot), same, ref):
        check(name, h, s, r)


def test_replaced_config_hook_is_called_and_reported(monkeypatch):
    """examples/use_cutom_config_func.py: callers may assign ``flash.get_fwd_config``.  The hook is
    called before the launch like in the reference (flash.py:64-66); a tile that no compiled kernel has
    is reported once and the default tile is launched, with correct results."""
    import warnings
    from flag_attn import flash
    calls = []

    def hook(B, H, M, N, D, causal):
        calls.append((B, H, M, N, D, causal))
        return (64, 64, 1, 4)
    monkeypatch.setattr(flash, "get_fwd_config", hook)
    B, H, T, D = 2, 16, 1024, 128
    q, k, v = (torch.randn(B, H, T, D, dtype=torch.bfloat16, device="cuda:0", requires_grad=True) for _ in range(3))
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        o = flag_attn.flash_attention(q, k, v, causal=True)
        flag_attn.flash_attention(q, k, v, causal=True)
    assert calls == [(B, H, T, T, D, True)] * 2
    assert len([w for w in seen if "BLOCK_M=64, BLOCK_N=64" in str(w.message)]) <= 1   # once per distinct answer
    go = torch.randn_like(o)
    grads = torch.autograd.grad(o, (q, k, v), go)
    g_ref = torch.autograd.grad(oracle_flash(q, k, v, True, upcast=True), (q, k, v), go)
    g_same = torch.autograd.grad(oracle_flash(q, k, v, True, upcast=False), (q, k, v), go)
    for name, h, s, r in zip(("dq", "dk", "dv"), grads, g_same, g_ref):
        check(name, h, s, r)


def test_piecewise_call_with_positional_threshold():
    """examples/piecewise_example.py at a quarter of its length."""
    from flag_attn import piecewise_attention
    B, H, T, D = 2, 4, 2048, 128
    ts = [torch.randn((B, H, T, D), dtype=torch.float16, device="cuda:0").requires_grad_() for _ in range(5)]
    o = piecewise_attention(*ts, T // 2, causal=True)
    go = torch.randn((B, H, T, D), dtype=torch.float16, device="cuda:0")
    grads = torch.autograd.grad(o, ts, go)
    g_ref = torch.autograd.grad(oracle_pw(*ts, T // 2, causal=True, upcast=True), ts, go)
    g_same = torch.autograd.grad(oracle_pw(*ts, T // 2, causal=True, upcast=False), ts, go)
    assert len(grads) == 5
    for name, h, s, r in zip(("dq1", "dk1", "dq2", "dk2", "dv"), grads, g_same, g_ref):
        check(name, h, s, r)
