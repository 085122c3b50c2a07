"""``flash_attention``: FlashAttention-2 forward/backward on gfx950 HIP kernels.

Host-side counterpart of ``src/flag_attn/flash.py:23-286`` of the reference: same signature, same
return convention, same autograd contract (``save_for_backward(q, k, v, o, L)``, gradients for
q, k, v only, gradients flowing into the auxiliary outputs are ignored).  The Triton launches are
replaced by calls into the C-ABI kernel library.
"""
import math
import os

import torch

from . import _abi, _config, _lib
from .split_kv import num_splits_heuristic, split_kv_forward, split_units, DECODE_MAX_ROWS
from .total import _total_attention
from .dropout import philox_cuda_seed_offset

__all__ = ["attention"]

_HEAD_DIMS = (16, 32, 64, 128)


# (BLOCK_M, BLOCK_N) the kernels are compiled for; the first entry is the fallback
FWD_TILES = ((128, 64), (256, 64))
BWD_TILES = ((64, 128),)


def wide_forward_applies(D, dropout_p=0.0):
    """The 256-row forward kernel (64 query rows per wavefront, one wavefront per SIMD) is built for
    head size 128 without dropout."""
    return D == 128 and not dropout_p > 0


def get_fwd_config(B, H, M, N, D, causal):
    """(BLOCK_M, BLOCK_N, num_stages, num_warps) of the dense forward kernel: query rows per
    workgroup, keys per pipeline stage, LDS stages, 64-lane wavefronts.

    An overridable module-level hook like ``src/flag_attn/flash.py:290-322``, called before every
    forward launch (``flash.py:64-66``).  The kernels are compiled ahead of time, so an override may
    only choose among ``FWD_TILES``; any other answer is reported once and the fallback is launched.
    The default takes the 256-row kernel where it applies and the launch has at least one workgroup
    per compute unit (its workgroups hold a compute unit alone)."""
    if wide_forward_applies(D) and -(-M // 256) * H * B >= _num_cus():
        return (256, 64, 5, 4)
    return (128, 64, 2, 4)


def wide_key_splits(B, H, M, N, D, num_cus):
    """Pieces of the key axis for a dense forward launch whose 256-row workgroups (one per compute unit at a
    time) would leave at least half of the compute units idle: Tq = 1024 against Tk = 8192 with 32 heads has
    128 of them on 256 units.  Each piece is a workgroup of its own and the pieces are merged like the split-KV
    path's (``split_kv.py:162-227`` of the reference); a piece keeps at least 1024 keys.  1 = do not split."""
    if not wide_forward_applies(D) or M < 256:
        return 1
    wgs = -(-M // 256) * H * B
    pieces = min(num_cus // wgs, N // 1024)
    if pieces < 2 or 4 * pieces * wgs < 3 * num_cus:
        return 1
    return pieces


_NUM_CUS = {}


def _num_cus():
    dev = torch.cuda.current_device() if torch.cuda.is_available() else -1
    if dev not in _NUM_CUS:
        _NUM_CUS[dev] = _lib.get().fa_num_cus() if dev >= 0 else 256
    return _NUM_CUS[dev]


_DEFAULT_FWD_CONFIG = get_fwd_config


def get_bwd_config(B, H, M, N, D, causal):
    """(BLOCK_M, BLOCK_N, num_stages, num_warps) of the dK/dV kernel: queries per pipeline step, keys
    per workgroup (``flash.py:493-519`` hook, called as in ``flash.py:185-186``; see ``BWD_TILES``)."""
    return (64, 128, 2, 4)


def _check_arguments(q, k, v, dropout_p):
    """The argument checks of ``flash.py:27-38`` of the reference."""
    Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Dq == Dk == Dv, "feature size of q, k, v should be equal"
    assert Dk in _HEAD_DIMS
    Hk, Hv = k.shape[1], v.shape[1]
    assert Hk == Hv, "num of heads in k and v should be equal"
    assert Hk > 0 and q.shape[1] % Hk == 0, "number of heads in q must be a multiple of that in k & v"
    assert 0.0 <= dropout_p < 1.0, "dropout_p must be in [0, 1)"


class NothingToAttend(torch.autograd.Function):
    """An empty batch, query or key axis: no kernel has anything to do.  A query row without keys gives
    O = 0 and L = -inf, as rows hidden entirely by the causal mask do (``flash.py:471-474``), and every
    gradient is zero.  (The reference divides by zero in its split rule for an empty batch or query axis
    and returns NaN for an empty key axis.)"""

    @staticmethod
    def forward(ctx, *inputs):
        ctx.like = [(t.shape, t.dtype, t.device) for t in inputs]
        return torch.zeros_like(inputs[0])

    @staticmethod
    def backward(ctx, do):
        return tuple(torch.zeros(shape, dtype=dtype, device=device) for shape, dtype, device in ctx.like)


class FlashAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, dropout_p, return_log_normalizer,
                return_total_attention, return_seed_offset):
        _check_arguments(q, k, v, dropout_p)
        B, H, M, D = q.shape
        N = k.shape[2]
        Hk = k.shape[1]
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(D)

        lib = _lib.get()
        q, k, v = _abi.kernel_ready(q), _abi.kernel_ready(k), _abi.kernel_ready(v)

        with torch.cuda.device(q.device):
            num_cus = _num_cus()
            is_dropout = dropout_p > 0
            if is_dropout:   # one Philox counter value per score element (flash.py:52-57)
                seed, offset = philox_cuda_seed_offset(B * H * M * N, q.device)
            else:
                seed, offset = 0, 0
            dropout = (dropout_p, seed, offset)
            split_block_m, split_block_n = split_units(B, H, M, N, D, causal)   # flash.py:59 of the reference
            splits = num_splits_heuristic(B, H, M, N, split_block_m, split_block_n, num_cus, 128)
            if splits > 1:
                assert not is_dropout, "Cannot apply dropout with splitkv."   # as flash.py:89
            if splits > 1 or (M <= DECODE_MAX_ROWS and N >= 1024 and not is_dropout):
                o, L = split_kv_forward(lib, q, k, v, causal, sm_scale, splits)
            else:
                # looked up by name at call time, so that an assignment to flash.get_fwd_config takes effect
                hook = get_fwd_config
                block_m, _ = _config.resolve(hook, FWD_TILES, "flash_attention forward", (B, H, M, N, D, causal))
                pieces = 1
                if hook is _DEFAULT_FWD_CONFIG:
                    # nobody overrode the hook: the library applies the same rule and also knows what the hook
                    # is not told (dropout, the sign of sm_scale, row strides the 256-row kernel cannot address)
                    block_m = 0
                    if not is_dropout and sm_scale > 0 and max(k.stride(2), v.stride(2)) * k.element_size() < 1 << 24:
                        pieces = wide_key_splits(B, H, M, N, D, num_cus)
                elif block_m == 256 and not wide_forward_applies(D, dropout_p):
                    _config.warn_once(("fwd-wide", D, is_dropout),
                                      "flash_attention forward: the 256-row kernel is built for head size 128 "
                                      "without dropout; launching the 128-row kernel")
                    block_m = 128
                elif block_m == 256 and not sm_scale > 0:
                    _config.warn_once(("fwd-wide-scale",),
                                      "flash_attention forward: the 256-row kernel needs sm_scale > 0; launching "
                                      "the 128-row kernel")
                    block_m = 128
                elif block_m == 256 and max(k.stride(2), v.stride(2)) * k.element_size() >= 1 << 24:
                    _config.warn_once(("fwd-wide-stride",),
                                      "flash_attention forward: the 256-row kernel addresses key/value rows less "
                                      "than 16 MiB apart; launching the 128-row kernel")
                    block_m = 128
                if pieces > 1:   # too few 256-row workgroups for the device: one per piece of the key axis, then the merge
                    o, L = split_kv_forward(lib, q, k, v, causal, sm_scale, pieces, exact=True)
                else:
                    o = torch.empty_like(q)
                    if not _abi.is_kernel_ready(o):
                        o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
                    L = torch.empty((B, H, M), device=q.device, dtype=torch.float32)
                    _abi.fa_fwd(lib, q, k, v, o, L, causal, sm_scale, dropout, block_m)
            tot_attn = None
            if return_total_attention:
                tot_attn = _total_attention(lib, q, k, L, causal, sm_scale)

        ctx.save_for_backward(q, k, v, o, L)
        ctx.sm_scale = sm_scale
        ctx.causal = causal
        ctx.dropout = dropout

        if return_log_normalizer or return_total_attention or return_seed_offset:
            return (o,
                    L if return_log_normalizer else None,
                    tot_attn if return_total_attention else None,
                    seed if is_dropout and return_seed_offset else None,
                    offset if is_dropout and return_seed_offset else None)
        return o

    @staticmethod
    def backward(ctx, do, *ignored):
        q, k, v, o, L = ctx.saved_tensors
        sm_scale, causal, dropout = ctx.sm_scale, ctx.causal, ctx.dropout
        B, H, M, D = q.shape
        N, Hk = k.shape[2], k.shape[1]
        group = H // Hk
        lib = _lib.get()
        do = _abi.kernel_ready(do)
        with torch.cuda.device(q.device):
            _config.resolve(get_bwd_config, BWD_TILES, "flash_attention backward", (B, H, M, N, D, causal))
            delta = torch.empty_like(L)
            _abi.fa_bwd_delta(lib, o, do, delta)
            # dK/dV come out summed over each kv head's group of query heads (flash.py:205-206,250-251
            # of the reference produce one slice per query head and reduce afterwards)
            # the kernels that sum query heads are built without dropout
            chunk = 1 if dropout[0] > 0 else dkdv_heads_per_slice(B, H, group, N, _num_cus())
            slices = H // chunk
            dk = torch.empty((B, slices, N, D), dtype=k.dtype, device=q.device)
            dv = torch.empty((B, slices, N, D), dtype=v.dtype, device=q.device)
            dq = torch.empty((B, H, M, D), dtype=q.dtype, device=q.device)
            heads = ds_heads_per_launch(lib, B, H, group, M, N, D)
            ds = None
            if heads >= B * H:
                ds = _ds_workspace(lib, q.device, B, H, M, N)
            elif heads > 0:
                heads = min(heads, H)
                ds = _ds_workspace(lib, q.device, 1, heads, M, N)
            if ds is None:   # dS not worth keeping for this shape, or no memory for it: recompute it
                _abi.fa_bwd_dkdv(lib, q, k, v, do, L, delta, dk, dv, causal, sm_scale, dropout)
                _abi.fa_bwd_dq(lib, q, k, v, do, L, delta, dq, causal, sm_scale, dropout)
            elif heads >= B * H:
                _abi.fa_bwd_dkdv_ds(lib, q, k, v, do, L, delta, dk, dv, ds, causal, sm_scale, dropout)
                _abi.fa_bwd_dq_from_ds(lib, k, ds, dq, causal, sm_scale)
            else:
                # bounded workspace: one batch entry and `heads` query heads at a time; the dropout
                # counter of a slice starts where the slice starts in the (B, H, M, N) score tensor
                for b in range(B):
                    for h0 in range(0, H, heads):
                        h1 = min(H, h0 + heads)
                        hs, ks = slice(h0, h1), slice(h0 // group, -(-h1 // group))
                        ss = slice(h0 // chunk, h1 // chunk)
                        bs = slice(b, b + 1)
                        drop = (dropout[0], dropout[1], dropout[2] + (b * H + h0) * M * N)
                        _abi.fa_bwd_dkdv_ds(lib, q[bs, hs], k[bs, ks], v[bs, ks], do[bs, hs], L[bs, hs],
                                            delta[bs, hs], dk[bs, ss], dv[bs, ss], ds, causal, sm_scale, drop)
                        _abi.fa_bwd_dq_from_ds(lib, k[bs, ks], ds, dq[bs, hs], causal, sm_scale)
            if slices > Hk:   # the kernel summed `chunk` heads of every group; add the chunks
                dk = dk.reshape(B, Hk, slices // Hk, N, D).sum(2)
                dv = dv.reshape(B, Hk, slices // Hk, N, D).sum(2)
        return dq, dk, dv, None, None, None, None, None, None


def dkdv_heads_per_slice(B, H, group, N, num_cus):
    """How many query heads of a kv head one dK/dV workgroup accumulates (``flash.py:205-206,250-251``
    of the reference write one slice per query head and reduce afterwards).  The whole group when
    the launch still has at least two workgroups per compute unit (with fewer, the unequal lengths of
    the workgroups under the causal mask cannot be balanced: 3.0 instead of 1.9 ms at 32 query / 4 kv
    heads, T = 8192), otherwise the largest divisor of the group that gets there; the remaining
    slices are added with one torch sum."""
    blocks = -(-N // 128)
    for chunk in range(group, 0, -1):
        if group % chunk == 0 and blocks * B * (H // chunk) >= 2 * num_cus:
            return chunk
    return 1


# Largest dS workspace the backward may take (MiB); 0 disables the dS path.  The workspace is
# M * N * 2 bytes per (batch, head) slice (128 MiB at 8192 x 8192); a backward whose slices do not
# all fit walks them in launches of as many heads as do.  Launches of fewer than about 32 heads of
# 8192 keys no longer fill the device: measured at B = 1, H = 32, T = 8192, D = 128 (needs 4096 MiB),
# a forward + backward step takes 2.16 ms with 4096 MiB or more, 2.20 with 2048, 2.33 with 1024,
# 3.11 with 512 and 5.51 with 256.  The default holds that workload whole.  A workspace that cannot be
# allocated is not an error: the backward then recomputes dS (the fa_bwd_dkdv + fa_bwd_dq pair).
DS_WORKSPACE_LIMIT_MIB = int(os.environ.get("FLAGATTN_DS_WORKSPACE_MIB", "4096"))


def ds_heads_per_launch(lib, B, H, group, M, N, D, grids=1):
    """How many (batch, head) slices one dK/dV + dQ-from-dS launch pair may cover, 0 = recompute dS
    in the dQ kernel instead.  Keeping dS costs M * N * 2 bytes per head (times ``grids``: piecewise
    attention keeps one grid per regime), written once and read once; it pays when the two recomputed
    products are expensive (head size 128) and the matrix is big enough for the launches to fill the
    device."""
    if D < 128 or M * N < 1024 * 1024 or DS_WORKSPACE_LIMIT_MIB <= 0:
        return 0
    per_head = grids * lib.fa_bwd_ds_workspace_mib(1, 1, M, N)
    fit = DS_WORKSPACE_LIMIT_MIB // per_head
    if fit >= B * H:
        return B * H
    fit = (fit // group) * group  # whole groups of query heads, so that k/v slices line up
    return fit


def _ds_workspace(lib, device, B, H, M, N, grids=1):
    """Device memory for dS, or None when the allocator has none left (the caller then recomputes)."""
    mib = lib.fa_bwd_ds_workspace_mib(B, H, M, N)
    assert mib > 0
    try:
        return torch.empty(grids * (mib << 20), dtype=torch.uint8, device=device)
    except torch.OutOfMemoryError:
        return None


def attention(q, k, v, causal=False, sm_scale=None, dropout_p=0.0,
              return_log_normalizer=False, return_total_attention=False, return_seed_offset=False):
    """FlashAttention-2.

    q (batch, heads_q, seqlen_q, headdim); k, v (batch, heads_k, seqlen_k, headdim); heads_q must be
    a multiple of heads_k.  ``causal`` masks with bottom-right alignment.  Returns ``out`` or, when
    any ``return_*`` flag is set, ``(out, log_normalizer|None, total_attention|None, seed|None,
    offset|None)`` -- exactly the reference's convention (``src/flag_attn/flash.py:150-160``).
    ``dropout_p > 0`` drops probabilities with the reference's Philox scheme (seed and offset taken from
    the device's default generator and returned when ``return_seed_offset`` is set); it cannot be
    combined with a shape that takes the split-KV path, as in the reference.  With an empty batch, query
    or key axis nothing is launched: out is zero, the log-normalizer -inf, the total attention zero.
    """
    if q.numel() == 0 or k.shape[2] == 0:
        _check_arguments(q, k, v, dropout_p)
        B, H, M, _ = q.shape
        o = NothingToAttend.apply(q, k, v)
        if not (return_log_normalizer or return_total_attention or return_seed_offset):
            return o
        seed = offset = None
        if dropout_p > 0 and return_seed_offset:
            seed, offset = philox_cuda_seed_offset(0, q.device)      # nothing is drawn
        return (o,
                torch.full((B, H, M), -math.inf, dtype=torch.float32, device=q.device) if return_log_normalizer else None,
                torch.zeros((B, H, k.shape[2]), dtype=torch.float32, device=q.device) if return_total_attention else None,
                seed, offset)
    return FlashAttention.apply(q, k, v, causal, sm_scale, dropout_p, return_log_normalizer,
                                return_total_attention, return_seed_offset)
