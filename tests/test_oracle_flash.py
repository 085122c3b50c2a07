"""Pins the flash-attention oracle without the reference: library routine, fp64 brute force,
invariants and closed-form gradients.  Each check is chosen so that a plausible mistake (top-left
instead of bottom-right causal alignment, a dropped scale, wrong head grouping, a transposed
operand) fails it."""
import math

import pytest
import torch

from oracle import flash_attention, max_abs_diff

torch.manual_seed(10086)


def brute_force(q, k, v, causal, sm_scale):
    """fp64 loops straight from the definition; returns out, lse, total attention."""
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    g = H // Hk
    out = torch.zeros(B, H, M, D, dtype=torch.float64)
    lse = torch.full((B, H, M), -math.inf, dtype=torch.float64)
    tot = torch.zeros(B, H, N, dtype=torch.float64)
    q, k, v = q.double(), k.double(), v.double()
    for b in range(B):
        for h in range(H):
            hk = h // g
            for m in range(M):
                last = N - M + m if causal else N - 1  # last visible key
                if last < 0:
                    continue
                s = [sm_scale * float(torch.dot(q[b, h, m], k[b, hk, n])) for n in range(last + 1)]
                top = max(s)
                e = [math.exp(x - top) for x in s]
                z = sum(e)
                lse[b, h, m] = top + math.log(z)
                for n, en in enumerate(e):
                    p = en / z
                    tot[b, h, n] += p
                    out[b, h, m] += p * v[b, hk, n]
    return out, lse, tot


@pytest.mark.parametrize("M,N", [(5, 5), (3, 7), (7, 3), (1, 6)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Hq,Hk", [(2, 2), (4, 2), (4, 1)])
def test_matches_brute_force(M, N, causal, Hq, Hk):
    B, D = 2, 8
    q = torch.randn(B, Hq, M, D)
    k = torch.randn(B, Hk, N, D)
    v = torch.randn(B, Hk, N, D)
    scale = 0.37
    o, lse, tot = flash_attention(q, k, v, causal, scale, upcast=True,
                                  return_log_normalizer=True, return_total_attention=True)
    o_bf, lse_bf, tot_bf = brute_force(q, k, v, causal, scale)
    assert max_abs_diff(o, o_bf.float()) < 2e-6
    assert max_abs_diff(lse, lse_bf.float()) < 2e-6
    assert max_abs_diff(tot, tot_bf.float()) < 2e-6
    assert not torch.isnan(o).any()


def test_empty_rows_are_zero_with_minus_inf_normalizer():
    q, k, v = torch.randn(1, 1, 6, 4), torch.randn(1, 1, 2, 4), torch.randn(1, 1, 2, 4)
    o, lse, tot = flash_attention(q, k, v, True, upcast=True,
                                  return_log_normalizer=True, return_total_attention=True)
    assert torch.all(o[0, 0, :4] == 0)          # rows 0..3 see no key (m + N - M < 0)
    assert torch.all(torch.isinf(lse[0, 0, :4]) & (lse[0, 0, :4] < 0))
    assert torch.isfinite(lse[0, 0, 4:]).all()
    assert abs(tot.sum().item() - 2.0) < 1e-6   # only the two non-empty rows contribute


@pytest.mark.parametrize("causal,M,N", [(False, 33, 47), (True, 40, 40)])
def test_matches_sdpa(causal, M, N):
    q, k, v = torch.randn(2, 3, M, 16), torch.randn(2, 3, N, 16), torch.randn(2, 3, N, 16)
    o = flash_attention(q, k, v, causal, upcast=True)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=causal)
    assert max_abs_diff(o, ref) < 2e-6


def test_default_scale_and_explicit_scale():
    q, k, v = torch.randn(1, 2, 9, 16), torch.randn(1, 2, 11, 16), torch.randn(1, 2, 11, 16)
    assert max_abs_diff(flash_attention(q, k, v), flash_attention(q, k, v, sm_scale=0.25)) == 0.0
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=0.7)
    assert max_abs_diff(flash_attention(q, k, v, sm_scale=0.7), ref) < 2e-6


def test_lse_and_total_attention_invariants():
    q, k, v = torch.randn(2, 2, 12, 8), torch.randn(2, 2, 20, 8), torch.randn(2, 2, 20, 8)
    for causal in (False, True):
        o, lse, tot = flash_attention(q, k, v, causal, return_log_normalizer=True, return_total_attention=True)
        assert max_abs_diff(tot.sum(-1), torch.full((2, 2), 12.0)) < 1e-5  # every row sums to one
        s = torch.einsum("bhmd,bhnd->bhmn", q, k) / math.sqrt(8)
        if causal:
            keep = torch.arange(12)[:, None] + 8 >= torch.arange(20)[None, :]
            s = s.masked_fill(~keep, -math.inf)
        assert max_abs_diff(lse, torch.logsumexp(s, -1)) < 1e-5


def test_grouped_heads_equal_repeated_heads():
    q, k, v = torch.randn(2, 6, 10, 8), torch.randn(2, 2, 13, 8), torch.randn(2, 2, 13, 8)
    a = flash_attention(q, k, v, True)
    b = flash_attention(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1), True)
    assert max_abs_diff(a, b) == 0.0
    # head h uses kv head h // 3, not h % 2
    c = flash_attention(q[:, 3:4], k[:, 1:2], v[:, 1:2], True)
    assert max_abs_diff(a[:, 3:4], c) < 1e-6


def test_same_precision_path_rounds_scores_to_input_dtype():
    q = torch.randn(1, 1, 16, 32).bfloat16()
    k = torch.randn(1, 1, 16, 32).bfloat16()
    v = torch.randn(1, 1, 16, 32).bfloat16()
    ref = flash_attention(q, k, v, upcast=True)
    sp = flash_attention(q, k, v, upcast=False)
    assert ref.dtype == sp.dtype == torch.bfloat16
    s16 = (torch.matmul(q, k.transpose(-1, -2)) * (1 / math.sqrt(32))).float()
    manual = torch.matmul(torch.softmax(s16, -1).bfloat16(), v)
    assert max_abs_diff(sp, manual) == 0.0


@pytest.mark.parametrize("causal,M,N", [(False, 6, 9), (True, 6, 9), (True, 9, 6)])
def test_closed_form_gradients(causal, M, N):
    """dV = P^T dO, dS = P*(dP - delta)*scale, dQ = dS K, dK = dS^T Q (group-summed)."""
    B, Hq, Hk, D = 2, 4, 2, 8
    g = Hq // Hk
    scale = 0.3
    q = torch.randn(B, Hq, M, D, dtype=torch.float64, requires_grad=True)
    k = torch.randn(B, Hk, N, D, dtype=torch.float64, requires_grad=True)
    v = torch.randn(B, Hk, N, D, dtype=torch.float64, requires_grad=True)
    do = torch.randn(B, Hq, M, D, dtype=torch.float64)
    o = flash_attention(q, k, v, causal, scale)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), do)

    kk, vv = k.detach().repeat_interleave(g, 1), v.detach().repeat_interleave(g, 1)
    s = torch.einsum("bhmd,bhnd->bhmn", q.detach(), kk) * scale
    keep = torch.ones(M, N, dtype=torch.bool)
    if causal:
        keep = torch.arange(M)[:, None] + (N - M) >= torch.arange(N)[None, :]
        s = s.masked_fill(~keep, -math.inf)
    p = torch.softmax(s, -1)
    p = torch.where(keep, p, torch.zeros_like(p)).nan_to_num(0.0)
    dp = torch.einsum("bhmd,bhnd->bhmn", do, vv)
    delta = (do * o.detach()).sum(-1, keepdim=True)
    ds = p * (dp - delta) * scale
    dq_cf = torch.einsum("bhmn,bhnd->bhmd", ds, kk)
    dk_cf = torch.einsum("bhmn,bhmd->bhnd", ds, q.detach()).reshape(B, Hk, g, N, D).sum(2)
    dv_cf = torch.einsum("bhmn,bhmd->bhnd", p, do).reshape(B, Hk, g, N, D).sum(2)
    # the softmax itself runs in fp32 (as in the reference), hence the 1e-6 scale of the bound
    assert (dq - dq_cf).abs().max() < 2e-6
    assert (dk - dk_cf).abs().max() < 2e-6
    assert (dv - dv_cf).abs().max() < 2e-6
    if causal and M > N:
        assert torch.all(dq[:, :, : M - N] == 0)  # empty rows get no gradient
    assert torch.isfinite(dk).all() and torch.isfinite(dv).all()


def test_gradcheck_fp64():
    q = torch.randn(1, 2, 4, 4, dtype=torch.float64, requires_grad=True)
    k = torch.randn(1, 1, 5, 4, dtype=torch.float64, requires_grad=True)
    v = torch.randn(1, 1, 5, 4, dtype=torch.float64, requires_grad=True)
    # the softmax inside runs in fp32 whatever the input dtype (as in the reference), so the finite
    # differences need a coarse step and matching tolerances
    assert torch.autograd.gradcheck(lambda a, b, c: flash_attention(a, b, c, True, 0.5), (q, k, v),
                                    eps=1e-2, atol=2e-3, rtol=1e-2)
