"""The reference's acceptance rule, restated.

Test infrastructure only.  ``tests/flag_attn/test_flash_attention.py:8-9,57-65`` of the reference:
a result passes when its largest absolute deviation from the fp32 reference is at most twice the
deviation of the same-precision PyTorch implementation, plus 1e-5.  The forward tests compare with
``<=`` (``test_flash_attention.py:65,113,214-222,262``, ``test_piecewise_attention.py:50,119-124``);
the flash backward tests compare with ``<`` (``test_flash_attention.py:174-177,317-320``):
``strict=True`` selects the latter.
"""
import torch


def max_abs_diff(a, b):
    a, b = a.to(torch.float32), b.to(torch.float32)
    # -inf == -inf must count as equal (log-normalizer of rows that see no key)
    same = (a == b)
    d = torch.where(same, torch.zeros_like(a), (a - b).abs())
    return d.max().item() if d.numel() else 0.0


def within_two_x(hyp, same_precision, ref, slack=1e-5, strict=False):
    """Returns (ok, err_hyp, err_same_precision)."""
    e_hyp = max_abs_diff(hyp, ref)
    e_sp = max_abs_diff(same_precision, ref)
    bound = 2.0 * e_sp + slack
    ok = (e_hyp < bound if strict else e_hyp <= bound) and not torch.isnan(hyp.to(torch.float32)).any().item()
    return ok, e_hyp, e_sp
