"""``piecewise_attention``: attention whose score switches between two (q, k) pairs at a distance
threshold, on gfx950 HIP kernels.

Host-side counterpart of ``src/flag_attn/piecewise.py:25-191`` of the reference (same signature and
autograd contract: five gradients, none for the threshold / flags).
"""
import math

import torch

from . import _abi, _config, _lib
from .flash import NothingToAttend, _ds_workspace, ds_heads_per_launch

__all__ = ["attention"]


FWD_TILES = ((128, 64),)
BWD_TILES = ((64, 128),)


def get_fwd_config(B, H, M, N, D, causal):
    """(BLOCK_M, BLOCK_N, num_stages, num_warps); overridable hook called before the forward launch
    (``piecewise.py:44, 194-221``).  Only ``FWD_TILES`` are compiled; another answer is reported once."""
    return (128, 64, 2, 4)


def get_bwd_config(B, H, M, N, D, causal):
    """The same for the dK/dV kernel (``piecewise.py:98-99, 373-405``; ``BWD_TILES``)."""
    return (64, 128, 2, 4)


class PiecewiseAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q1, k1, q2, k2, v, w, causal, sm_scale):
        Dq1, Dk1, Dq2, Dk2, Dv = (t.shape[-1] for t in (q1, k1, q2, k2, v))
        assert Dq1 == Dk1 == Dq2 == Dk2 == Dv
        assert Dk1 in (16, 32, 64, 128)
        B, H, M, D = q1.shape
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(D)
        lib = _lib.get()
        q1, k1, q2, k2, v = (_abi.kernel_ready(t) for t in (q1, k1, q2, k2, v))
        with torch.cuda.device(q1.device):
            _config.resolve(get_fwd_config, FWD_TILES, "piecewise_attention forward",
                            (B, H, M, k1.shape[2], D, causal))
            o = torch.empty_like(q1)
            if not _abi.is_kernel_ready(o):
                o = torch.empty(q1.shape, dtype=q1.dtype, device=q1.device)
            L = torch.empty((B, H, M), device=q1.device, dtype=torch.float32)
            _abi.pw_fwd(lib, q1, k1, q2, k2, v, o, L, w, causal, sm_scale)
        ctx.save_for_backward(q1, k1, q2, k2, v, o, L)
        ctx.sm_scale, ctx.causal, ctx.w = sm_scale, causal, w
        return o

    @staticmethod
    def backward(ctx, do):
        q1, k1, q2, k2, v, o, L = ctx.saved_tensors
        lib = _lib.get()
        do = _abi.kernel_ready(do)
        with torch.cuda.device(q1.device):
            _config.resolve(get_bwd_config, BWD_TILES, "piecewise_attention backward",
                            (q1.shape[0], q1.shape[1], q1.shape[2], k1.shape[2], q1.shape[3], ctx.causal))
            delta = torch.empty_like(L)
            _abi.fa_bwd_delta(lib, o, do, delta)
            dk1 = torch.empty(k1.shape, dtype=k1.dtype, device=k1.device)
            dk2 = torch.empty(k2.shape, dtype=k2.dtype, device=k2.device)
            dv = torch.empty(v.shape, dtype=v.dtype, device=v.device)
            dq1 = torch.empty(q1.shape, dtype=q1.dtype, device=q1.device)
            dq2 = torch.empty(q2.shape, dtype=q2.dtype, device=q2.device)
            B, H, M, D = q1.shape
            N = k1.shape[2]
            args = (ctx.w, ctx.causal, ctx.sm_scale)
            # dS handed from the dK/dV kernel to the dQ kernels, one chunk grid per regime, when it pays
            heads = ds_heads_per_launch(lib, B, H, 1, M, N, D, grids=2)
            ds = None
            if heads >= B * H:
                ds = _ds_workspace(lib, q1.device, B, H, M, N, grids=2)
            elif heads > 0:
                heads = min(heads, H)
                ds = _ds_workspace(lib, q1.device, 1, heads, M, N, grids=2)
            if ds is None:   # dS not worth keeping for this shape, or no memory for it: recompute it
                _abi.pw_bwd_dkdv(lib, q1, k1, q2, k2, v, do, L, delta, dk1, dk2, dv, *args)
                _abi.pw_bwd_dq(lib, q1, k1, q2, k2, v, do, L, delta, dq1, dq2, *args)
            elif heads >= B * H:
                _abi.pw_bwd_dkdv_ds(lib, q1, k1, q2, k2, v, do, L, delta, dk1, dk2, dv, ds, *args)
                _abi.pw_bwd_dq_from_ds(lib, k1, k2, ds, dq1, dq2, *args)
            else:  # bounded workspace: one batch entry and `heads` heads at a time
                for b in range(B):
                    for h0 in range(0, H, heads):
                        s = (slice(b, b + 1), slice(h0, min(H, h0 + heads)))
                        _abi.pw_bwd_dkdv_ds(lib, q1[s], k1[s], q2[s], k2[s], v[s], do[s], L[s], delta[s],
                                            dk1[s], dk2[s], dv[s], ds, *args)
                        _abi.pw_bwd_dq_from_ds(lib, k1[s], k2[s], ds, dq1[s], dq2[s], *args)
        return dq1, dk1, dq2, dk2, dv, None, None, None


def attention(q1, k1, q2, k2, v, dist_threshold, causal=False, sm_scale=None):
    """Piecewise attention.

    q1, q2 (batch, heads, seqlen_q, headdim); k1, k2, v (batch, heads, seqlen_k, headdim).  The score
    of query m and key n is ``q2[m].k2[n]`` when the signed distance ``m + seqlen_k - seqlen_q - n``
    is at least ``dist_threshold`` and ``q1[m].k1[n]`` otherwise.  Returns out (batch, heads,
    seqlen_q, headdim); zero when the batch, query or key axis is empty (nothing is launched)."""
    if q1.numel() == 0 or k1.shape[2] == 0:
        assert q1.shape == q2.shape and k1.shape == k2.shape == v.shape and q1.shape[-1] == k1.shape[-1]
        return NothingToAttend.apply(q1, k1, q2, k2, v)
    return PiecewiseAttention.apply(q1, k1, q2, k2, v, dist_threshold, causal, sm_scale)
