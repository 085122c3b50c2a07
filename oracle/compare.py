"""The reference's acceptance rule, restated.

Test infrastructure only.  ``tests/flag_attn/test_flash_attention.py:8-9,57-65`` of the reference:
a result passes when its largest absolute deviation from the fp32 reference is at most twice the
deviation of the same-precision PyTorch implementation, plus 1e-5.
"""
import torch


def max_abs_diff(a, b):
    a, b = a.to(torch.float32), b.to(torch.float32)
    # -inf == -inf must count as equal (log-normalizer of rows that see no key)
    same = (a == b)
    d = torch.where(same, torch.zeros_like(a), (a - b).abs())
    return d.max().item() if d.numel() else 0.0


def within_two_x(hyp, same_precision, ref, slack=1e-5):
    """Returns (ok, err_hyp, err_same_precision)."""
    e_hyp = max_abs_diff(hyp, ref)
    e_sp = max_abs_diff(same_precision, ref)
    ok = (e_hyp <= 2.0 * e_sp + slack) and not torch.isnan(hyp.to(torch.float32)).any().item()
    return ok, e_hyp, e_sp
