"""The benchmark configurations as parity cases, at their full sizes.

Every case runs the HIP path through the public API on the full configuration.  Where the fp32
oracle fits the device for the whole problem it checks everything; where it does not (8192^2 score
matrices over 32 heads) the kernels still run at full size and a slice of heads / sequences is
compared.  Acceptance: max|hip - fp32| <= 2 * max|same-precision torch - fp32| + 1e-5 for every
output (o, log-normalizer, total attention, dq, dk, dv).
"""
import math

import pytest
import torch

import flagattention_amd as flag_attn
from oracle import flash_attention as oracle_flash, piecewise_attention as oracle_pw
from oracle import paged_attention as oracle_paged, within_two_x

pytestmark = pytest.mark.gpu


def randn(shape, dtype, seed, grad=False):
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = torch.empty(shape, dtype=dtype, device="cuda").normal_(0.0, 1.0, generator=g)
    return t.requires_grad_() if grad else t


def check(name, hyp, same, ref, strict=False):
    ok, e_hyp, e_same = within_two_x(hyp, same, ref, strict=strict)
    assert ok, f"{name}: hip err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


def test_c1_forward_noncausal_fp16_against_the_cpu_fp32_oracle():
    B, H, T, D = 2, 4, 512, 64
    q, k, v = (randn((B, H, T, D), torch.float16, s) for s in (1, 2, 3))
    o, L, *_ = flag_attn.flash_attention(q, k, v, causal=False, sm_scale=1 / math.sqrt(D), return_log_normalizer=True)
    qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
    ref = oracle_flash(qc, kc, vc, False, 1 / math.sqrt(D), upcast=True, return_log_normalizer=True)
    same = oracle_flash(q, k, v, False, 1 / math.sqrt(D), upcast=False, return_log_normalizer=True)
    check("o", o.cpu(), same[0].cpu(), ref[0])
    check("L", L.cpu(), same[1].cpu(), ref[1])


def _flash_fwd_bwd_case(B, H, M, N, D, head_slice=None):
    q = randn((B, H, M, D), torch.bfloat16, 1, grad=True)
    k = randn((B, H, N, D), torch.bfloat16, 2, grad=True)
    v = randn((B, H, N, D), torch.bfloat16, 3, grad=True)
    do = randn((B, H, M, D), torch.bfloat16, 4)
    o, L, tot, *_ = flag_attn.flash_attention(q, k, v, causal=True, sm_scale=1 / math.sqrt(D),
                                             return_log_normalizer=True, return_total_attention=True)
    grads = torch.autograd.grad(o, (q, k, v), do)
    hs = slice(None) if head_slice is None else head_slice
    qs, ks, vs = (t[:, hs].detach().requires_grad_() for t in (q, k, v))
    ref = oracle_flash(qs, ks, vs, True, upcast=True, return_log_normalizer=True, return_total_attention=True)
    g_ref = torch.autograd.grad(ref[0], (qs, ks, vs), do[:, hs])
    same = oracle_flash(qs, ks, vs, True, upcast=False, return_log_normalizer=True, return_total_attention=True)
    g_same = torch.autograd.grad(same[0], (qs, ks, vs), do[:, hs])
    check("o", o[:, hs], same[0], ref[0])
    check("L", L[:, hs], same[1], ref[1])
    check("total", tot[:, hs], same[2], ref[2])
    for name, h, s, r in zip(("dq", "dk", "dv"), grads, g_same, g_ref):
        check(name, h[:, hs], s, r, strict=True)   # "<" as in test_flash_attention.py:174-177 of the reference


def test_c2_forward_backward_causal_bf16():
    _flash_fwd_bwd_case(4, 16, 2048, 2048, 128)


@pytest.mark.parametrize("D", [128, 64])
def test_c3_long_sequence(D):
    _flash_fwd_bwd_case(1, 32, 8192, 8192, D, head_slice=slice(5, 8))


@pytest.mark.parametrize("D", [128, 64])
def test_c3_cross_length(D):
    _flash_fwd_bwd_case(1, 32, 1024, 8192, D)


def test_c4_piecewise_forward_backward():
    B, H, T, D, w = 2, 32, 4096, 128, 1024
    q1, k1, q2, k2, v = (randn((B, H, T, D), torch.bfloat16, s, grad=True) for s in (1, 2, 3, 4, 5))
    do = randn((B, H, T, D), torch.bfloat16, 6)
    o = flag_attn.piecewise_attention(q1, k1, q2, k2, v, w, causal=True)
    grads = torch.autograd.grad(o, (q1, k1, q2, k2, v), do)
    hs = slice(12, 16)
    ins = [t[:, hs].detach().requires_grad_() for t in (q1, k1, q2, k2, v)]
    ref = oracle_pw(*ins, w, causal=True, upcast=True)
    g_ref = torch.autograd.grad(ref, ins, do[:, hs])
    same = oracle_pw(*ins, w, causal=True)
    g_same = torch.autograd.grad(same, ins, do[:, hs])
    check("o", o[:, hs], same, ref)
    for name, h, s, r in zip(("dq1", "dk1", "dq2", "dk2", "dv"), grads, g_same, g_ref):
        check(name, h[:, hs], s, r)


def test_c5a_paged_decode_normal_inputs_permuted_blocks():
    g = torch.Generator(device="cuda").manual_seed(10086)
    seqs, Hq, Hkv, D, bs = 64, 32, 8, 128, 16
    ctx = torch.randint(512, 8193, (seqs,), device="cuda", generator=g, dtype=torch.int32)
    blocks_per_seq = (ctx + bs - 1) // bs
    num_blocks = int(blocks_per_seq.sum())
    max_ctx = int(ctx.max())
    perm = torch.randperm(num_blocks, device="cuda", generator=g)
    bt = torch.zeros(seqs, (max_ctx + bs - 1) // bs, dtype=torch.int64, device="cuda")
    start = 0
    for s, n in enumerate(blocks_per_seq.tolist()):
        bt[s, :n] = perm[start:start + n]
        start += n
    q = randn((seqs, Hq, D), torch.float16, 1)
    kc = randn((num_blocks, Hkv, bs, D), torch.float16, 2)
    vc = randn((num_blocks, Hkv, bs, D), torch.float16, 3)
    scale = D ** -0.5
    out = flag_attn.paged_attention(q, kc, vc, ctx, bt, scale, max_ctx)
    sub = torch.tensor([0, 7, 13, 21, 34, 42, 55, 63], device="cuda")
    ref = oracle_paged(q[sub], kc, vc, bt[sub], ctx[sub], scale)
    same = oracle_paged(q[sub], kc, vc, bt[sub], ctx[sub], scale, same_precision=True)
    check("out", out[sub], same, ref)


def test_c5b_dense_split_kv_decode_through_flash_attention():
    q = randn((4, 32, 1, 128), torch.float16, 1)
    k = randn((4, 8, 32768, 128), torch.float16, 2)
    v = randn((4, 8, 32768, 128), torch.float16, 3)
    o, L, *_ = flag_attn.flash_attention(q, k, v, causal=False, return_log_normalizer=True)
    ref = oracle_flash(q, k, v, False, upcast=True, return_log_normalizer=True)
    same = oracle_flash(q, k, v, False, upcast=False, return_log_normalizer=True)
    check("o", o, same[0], ref[0])
    check("L", L, same[1], ref[1])
    o2 = flag_attn.flash_attention_split_kv(q, k, v, causal=False)
    check("o (split_kv entry)", o2, same[0], ref[0])
