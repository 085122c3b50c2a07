"""Plain-torch statement of piecewise (two-regime) attention and its closed-form gradients.

Test infrastructure only (see the package docstring).  Follows
``src/flag_attn/testing/piecewise.py:5-34`` (forward) and ``:36-78`` (gradient formulae) of the
reference:

* the score of (m, n) is ``q2[m].k2[n]`` when the signed distance ``m + (N - M) - n`` is at least
  ``dist_threshold`` and ``q1[m].k1[n]`` otherwise (``:21-24``); the distance is signed, so keys
  in the future of a query always use the first pair;
* both score matrices are produced in the working dtype, selected, then scaled (``:21-24``);
* causal masking fills with the most negative finite value of the working dtype rather than
  ``-inf`` (``:26-27``) and zeroes the masked probabilities afterwards (``:31-32``);
* the softmax runs in fp32 and is rounded to the value dtype at once (``:30``).
"""
import math

import torch


def _regimes(M, N, dist_threshold, device):
    rows = torch.arange(M, device=device)[:, None]
    cols = torch.arange(N, device=device)[None, :]
    signed_distance = rows + (N - M) - cols
    return signed_distance >= dist_threshold, signed_distance >= 0


def _probabilities(q1, k1, q2, k2, v_dtype, dist_threshold, causal, sm_scale):
    M, N = q1.shape[-2], k1.shape[-2]
    far, visible = _regimes(M, N, dist_threshold, q1.device)
    near_scores = torch.matmul(q1, k1.transpose(-1, -2))
    far_scores = torch.matmul(q2, k2.transpose(-1, -2))
    scores = torch.where(far, far_scores, near_scores) * sm_scale
    if causal:
        scores = torch.where(visible, scores, torch.finfo(scores.dtype).min)
    probs = torch.softmax(scores, dim=-1, dtype=torch.float32).to(v_dtype)
    return probs, far, visible


def piecewise_attention(q1, k1, q2, k2, v, dist_threshold, causal=False, sm_scale=None, upcast=False):
    """q1, q2 (B, H, M, D); k1, k2, v (B, H, N, D).  Returns out (B, H, M, D) in q1's dtype."""
    out_dtype = q1.dtype
    if upcast:
        q1, k1, q2, k2, v = (t.to(torch.float32) for t in (q1, k1, q2, k2, v))
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q1.shape[-1])
    probs, _, visible = _probabilities(q1, k1, q2, k2, v.dtype, dist_threshold, causal, sm_scale)
    if causal:
        probs = torch.where(visible, probs, 0.0)
    return torch.matmul(probs, v).to(out_dtype)


def piecewise_attention_grad(q1, k1, q2, k2, v, dist_threshold, causal, sm_scale, o, do, upcast=False):
    """Closed-form (dq1, dk1, dq2, dk2, dv) for the op above, given its output ``o`` and ``do``.

    dV = P^T dO;  dP = dO V^T;  delta = rowsum(dO * O);  dS = P * (dP - delta) * sm_scale;
    dS is routed to the pair that produced the score (``src/flag_attn/testing/piecewise.py:60-75``).
    """
    out_dtype = q1.dtype
    if upcast:
        q1, k1, q2, k2, v, o, do = (t.to(torch.float32) for t in (q1, k1, q2, k2, v, o, do))
    probs, far, _ = _probabilities(q1, k1, q2, k2, v.dtype, dist_threshold, causal, sm_scale)
    dv = torch.matmul(probs.transpose(-1, -2), do)
    dprobs = torch.matmul(do, v.transpose(-1, -2))
    delta = (do * o).sum(dim=-1, keepdim=True)
    dscores = probs * (dprobs - delta) * sm_scale
    dfar = torch.where(far, dscores, 0.0)
    dnear = torch.where(far, 0.0, dscores)
    dq1 = torch.matmul(dnear, k1)
    dk1 = torch.matmul(dnear.transpose(-1, -2), q1)
    dq2 = torch.matmul(dfar, k2)
    dk2 = torch.matmul(dfar.transpose(-1, -2), q2)
    return tuple(t.to(out_dtype) for t in (dq1, dk1, dq2, dk2, dv))
