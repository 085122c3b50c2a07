"""Plain-torch statement of scaled-dot-product attention with the reference's conventions.

Test infrastructure only (see the package docstring).  Follows
``src/flag_attn/testing/flash.py:5-70`` of the reference:

* grouped heads: every kv head serves ``Hq // Hk`` consecutive query heads (``:22-30``);
* the causal mask is aligned to the bottom-right corner, query row ``m`` sees key ``n`` iff
  ``m + (N - M) >= n`` (``:31-41``);
* scores are formed and scaled in the working dtype, then moved to fp32 for the softmax
  (``:39-47``) -- with ``upcast=False`` and bf16/fp16 inputs the scores are therefore rounded to
  16 bits before the softmax, and that sets the error budget of the acceptance rule;
* rows that see no key (``M > N`` with the causal mask) give an all ``-inf`` row, the softmax makes
  them NaN and a second select zeroes the masked probabilities (``:48-50``), so such rows produce an
  all-zero output and a log-normalizer of ``-inf``;
* probabilities are rounded to the value dtype before the second product (``:60``);
* dropout (``:55-60``): dropped probabilities are zeroed after the normaliser, total attention and
  log-normalizer have been taken, and the output is scaled by ``1 / (1 - dropout_p)``.  The mask is an
  input (``oracle.dropout.keep_mask`` restates how the kernels derive it from seed and offset).
"""
import math

import torch


def _visible(M, N, device):
    """Boolean (M, N) matrix, True where query row m may attend key n under the causal rule."""
    rows = torch.arange(M, device=device)[:, None]
    cols = torch.arange(N, device=device)[None, :]
    return rows + (N - M) >= cols


def flash_attention(q, k, v, causal=False, sm_scale=None, upcast=False,
                    return_log_normalizer=False, return_total_attention=False,
                    dropout_p=0.0, dropout_mask=None):
    """q (B, Hq, M, D); k, v (B, Hk, N, D).  Returns ``out`` or ``(out, lse|None, total|None)``.

    ``upcast=True`` is the fp32 reference, ``upcast=False`` the same-precision implementation that
    the 2x rule measures against.
    """
    out_dtype = q.dtype
    if upcast:
        q, k, v = (t.to(torch.float32) for t in (q, k, v))
    B, Hq, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    if Hq % Hk:
        raise AssertionError("query heads must be a multiple of key/value heads")
    group = Hq // Hk
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    if group > 1:
        k = k.repeat_interleave(group, dim=1)
        v = v.repeat_interleave(group, dim=1)

    keep = _visible(M, N, q.device) if causal else None

    scores = torch.matmul(q, k.transpose(-1, -2)) * sm_scale
    if causal:
        scores = torch.where(keep, scores, float("-inf"))
    scores = scores.to(torch.float32)

    lse = torch.logsumexp(scores, dim=-1) if return_log_normalizer else None

    probs = torch.softmax(scores, dim=-1, dtype=torch.float32)
    if causal:
        probs = torch.where(keep, probs, 0.0)

    total = probs.sum(dim=-2) if return_total_attention else None

    if dropout_mask is not None:
        probs = probs.masked_fill(~dropout_mask, 0.0)
    out = (torch.matmul(probs.to(v.dtype), v) * (1.0 / (1.0 - dropout_p))).to(out_dtype)
    if return_log_normalizer or return_total_attention:
        return out, lse, total
    return out
