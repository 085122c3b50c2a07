"""``total_attention``: column sums of the attention matrix from q, k and the saved log-normalizer.

Host-side counterpart of ``src/flag_attn/total.py:9-47`` of the reference.
"""
import math

import torch

from . import _abi, _config, _lib

# (BLOCK_M, BLOCK_N) the kernel is compiled for: queries per pipeline step, keys per workgroup
FWD_TILES = ((64, 128),)


def get_fwd_config(B, H, M, N, D, causal):
    """(BLOCK_M, BLOCK_N, num_stages, num_warps): the overridable hook of ``total.py:6-7``, called before
    every launch (``total.py:29``).  The kernel is compiled for one tile; any other answer is reported
    once and the compiled one is launched."""
    return (64, 128, 2, 4)


def _total_attention(lib, q, k, l, causal, sm_scale):
    B, H, M, D = q.shape
    N = k.shape[2]
    _config.resolve(get_fwd_config, FWD_TILES, "total_attention", (B, H, M, N, D, causal))
    tot = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    _abi.fa_total_attn(lib, q, k, l, tot, causal, sm_scale)
    return tot


def total_attention(q, k, l, causal=False, sm_scale=None):
    """q (B, H, M, D), k (B, Hk, N, D), l (B, H, M) fp32 log-normalizer -> (B, H, N) fp32."""
    Dq, Dk = q.shape[-1], k.shape[-1]
    assert Dq == Dk
    assert Dk in (16, 32, 64, 128)
    assert q.shape[1] % k.shape[1] == 0, "number of heads in q must be a multiple of that in k"
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(Dq)
    if q.numel() == 0 or k.shape[2] == 0:   # an empty batch, query or key axis: nothing attends to anything
        return torch.zeros((q.shape[0], q.shape[1], k.shape[2]), dtype=torch.float32, device=q.device)
    lib = _lib.get()
    q, k = _abi.kernel_ready(q), _abi.kernel_ready(k)
    l = l.contiguous()
    with torch.cuda.device(q.device):
        return _total_attention(lib, q, k, l, causal, sm_scale)
