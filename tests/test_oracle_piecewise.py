"""Pins the piecewise-attention oracle: reductions to plain attention, an fp64 loop, and the
closed-form gradients against autograd."""
import math

import pytest
import torch

from oracle import flash_attention, piecewise_attention, piecewise_attention_grad, max_abs_diff

torch.manual_seed(10086)


def make(B, H, M, N, D, dtype=torch.float32):
    return (torch.randn(B, H, M, D, dtype=dtype), torch.randn(B, H, N, D, dtype=dtype),
            torch.randn(B, H, M, D, dtype=dtype), torch.randn(B, H, N, D, dtype=dtype),
            torch.randn(B, H, N, D, dtype=dtype))


def brute_force(q1, k1, q2, k2, v, w, causal, scale):
    B, H, M, D = q1.shape
    N = k1.shape[2]
    out = torch.zeros(B, H, M, D, dtype=torch.float64)
    q1, k1, q2, k2, v = (t.double() for t in (q1, k1, q2, k2, v))
    for b in range(B):
        for h in range(H):
            for m in range(M):
                s = []
                for n in range(N):
                    dist = m + (N - M) - n
                    if causal and dist < 0:
                        continue
                    far = dist >= w
                    s.append((n, scale * float(torch.dot((q2 if far else q1)[b, h, m], (k2 if far else k1)[b, h, n]))))
                if not s:
                    continue
                top = max(x for _, x in s)
                z = sum(math.exp(x - top) for _, x in s)
                for n, x in s:
                    out[b, h, m] += math.exp(x - top) / z * v[b, h, n]
    return out


@pytest.mark.parametrize("M,N,w", [(6, 6, 3), (4, 9, 2), (9, 4, 5), (5, 5, 0), (5, 8, -2)])
@pytest.mark.parametrize("causal", [False, True])
def test_matches_brute_force(M, N, w, causal):
    q1, k1, q2, k2, v = make(1, 2, M, N, 8)
    o = piecewise_attention(q1, k1, q2, k2, v, w, causal, 0.4, upcast=True)
    assert max_abs_diff(o, brute_force(q1, k1, q2, k2, v, w, causal, 0.4).float()) < 2e-6


@pytest.mark.parametrize("causal", [False, True])
def test_reductions_to_plain_attention(causal):
    M, N = 10, 14
    q1, k1, q2, k2, v = make(2, 2, M, N, 8)
    # identical pairs: the threshold is irrelevant
    assert max_abs_diff(piecewise_attention(q1, k1, q1, k1, v, 3, causal), flash_attention(q1, k1, v, causal)) < 1e-6
    # threshold above every distance (max distance is N - 1): only the first pair is used
    assert max_abs_diff(piecewise_attention(q1, k1, q2, k2, v, N, causal), flash_attention(q1, k1, v, causal)) < 1e-6
    # threshold below every distance (min distance is -(M - 1) + (N - M) ... >= -N): only the second pair
    assert max_abs_diff(piecewise_attention(q1, k1, q2, k2, v, -N, causal), flash_attention(q2, k2, v, causal)) < 1e-6
    if causal:  # visible keys all have distance >= 0
        assert max_abs_diff(piecewise_attention(q1, k1, q2, k2, v, 0, True), flash_attention(q2, k2, v, True)) < 1e-6


def test_distance_is_signed_and_threshold_is_inclusive_for_far():
    # one query (m = 0), three keys, N - M = 2: distances are 2, 1, 0
    q1, k1, q2, k2, v = make(1, 1, 1, 3, 4)
    o = piecewise_attention(q1, k1, q2, k2, v, 1, False, 1.0, upcast=True)
    s = torch.stack([q2[0, 0, 0] @ k2[0, 0, 0], q2[0, 0, 0] @ k2[0, 0, 1], q1[0, 0, 0] @ k1[0, 0, 2]])
    assert max_abs_diff(o[0, 0, 0], torch.softmax(s, 0) @ v[0, 0]) < 1e-6


@pytest.mark.parametrize("causal,M,N,w", [(False, 7, 7, 3), (True, 7, 7, 3), (True, 6, 10, 4), (False, 6, 10, 4)])
def test_closed_form_grads_match_autograd(causal, M, N, w):
    q1, k1, q2, k2, v = (t.requires_grad_() for t in make(2, 2, M, N, 8))
    do = torch.randn(2, 2, M, 8)
    o = piecewise_attention(q1, k1, q2, k2, v, w, causal, 0.5)
    auto = torch.autograd.grad(o, (q1, k1, q2, k2, v), do)
    closed = piecewise_attention_grad(q1.detach(), k1.detach(), q2.detach(), k2.detach(), v.detach(),
                                      w, causal, 0.5, o.detach(), do)
    for a, c in zip(auto, closed):
        assert max_abs_diff(a, c) < 1e-5
