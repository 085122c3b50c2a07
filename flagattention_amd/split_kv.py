"""Split-KV forward (flash decoding): ``flash_attention_split_kv`` and the split-count rule.

Host-side counterpart of ``src/flag_attn/split_kv.py:229-330`` of the reference.  The split kernel
serves all query heads of a kv head from one workgroup, in steps of 32 keys per wavefront; the
reference's (BLOCK_M, BLOCK_N) = (16, 128) only survives as the unit in which the split rule counts
work, so that a given problem is split into the same number of pieces as in the reference.
"""
import math

import torch

from . import _abi, _config, _lib

__all__ = ["attention"]

SPLIT_BLOCK_M, SPLIT_BLOCK_N = 16, 128
FWD_TILES = ((SPLIT_BLOCK_M, SPLIT_BLOCK_N),)
# Up to this many query positions the decode-shaped kernel is used even where the reference's rule
# would not split: it multiplies 16-row tiles and reads K/V once per kv head, where the dense
# forward kernel would fill 128-row tiles per query head with a handful of rows.
DECODE_MAX_ROWS = 16


def get_fwd_config(B, H, M, N, D, causal):
    """(BLOCK_M, BLOCK_N, num_stages, num_warps): the overridable hook of ``split_kv.py:229-231``, called
    before the split rule is evaluated (``split_kv.py:288``, ``flash.py:59``).  The split kernel is
    compiled for one tile; any other answer is reported once and the compiled one is used."""
    return (SPLIT_BLOCK_M, SPLIT_BLOCK_N, 1, 4)


def split_units(B, H, M, N, D, causal):
    """(BLOCK_M, BLOCK_N) in which the split rule counts work: what the hook names, if compiled."""
    return _config.resolve(get_fwd_config, FWD_TILES, "flash_attention split-kv forward", (B, H, M, N, D, causal))


def num_splits_heuristic(B, H, M, N, block_m, block_n, num_cus, max_splits):
    """How many pieces to cut the key axis into (``split_kv.py:234-262``).

    No split when the un-split grid already fills 80 % of the compute units.  Otherwise every split
    count that does not leave a piece empty is scored by how full its last wave of workgroups is
    (waves / ceil(waves)), and the smallest count within 85 % of the best score wins.
    """
    base_blocks = B * H * -(-M // block_m)
    if base_blocks >= 0.8 * num_cus:
        return 1
    n_blocks = -(-N // block_n)
    limit = min(num_cus, n_blocks, max_splits)
    scored = []
    for s in range(1, limit + 1):
        per_split = -(-n_blocks // s)
        if s > 1 and per_split * s - n_blocks >= per_split:
            continue  # the last piece would be empty
        waves = base_blocks * s / num_cus
        scored.append((s, waves / math.ceil(waves)))
    best = max((eff for _, eff in scored), default=0.0)
    for s, eff in scored:
        if eff >= 0.85 * best:
            return s
    return 1


# spelling used by the reference, kept for callers that import it
num_splits_herustic = num_splits_heuristic


def _split_size(N, splits):
    return -(-(-(-N // SPLIT_BLOCK_N)) // splits) * SPLIT_BLOCK_N


def choose_num_splits(B, H, Hk, M, N, num_cus, reference_splits):
    """Number of pieces actually launched once the split path has been chosen.

    The split kernel serves a whole GQA group (up to 16 query rows) from one workgroup, so it starts
    ``B * Hk * ceil(G * M / 16)`` workgroups per split -- fewer than the per-query-head grid the
    reference's rule assumes.  Splits are added until the launch has about two workgroups per
    compute unit -- one resident wave, which measures 2-15 % faster than two shorter waves -- as long
    as every piece keeps at least 512 keys (four 32-key steps per wavefront).
    ``reference_splits`` (the count the reference's rule gives) is not used beyond having selected the
    split path.  The result of the operator does not depend on the count."""
    group = H // Hk
    base = B * Hk * -(-(group * M) // 16)
    n_units = -(-N // SPLIT_BLOCK_N)
    want = -(-2 * num_cus // base)
    cap = max(1, N // 512)
    splits = max(1, min(want, cap, 128))
    splits = min(splits, n_units)
    # drop counts that would leave the last piece empty
    while splits > 1 and (-(-n_units // splits)) * (splits - 1) >= n_units:
        splits -= 1
    return splits


def split_kv_forward(lib, q, k, v, causal, sm_scale, splits, single_direct=False, exact=False):
    """Runs the split kernel (+ merge) and returns (o, L).  ``splits`` is the count the reference's
    rule gave; the number of pieces launched is chosen by ``choose_num_splits`` unless ``exact`` asks for
    ``splits`` itself (the dense forward's own key pieces, ``flash.wide_key_splits``).  With
    ``single_direct`` a launch that ends up with one piece returns its fp16 partial output unmerged."""
    B, H, M, D = q.shape
    N = k.shape[2]
    if not exact and (splits != 1 or M <= DECODE_MAX_ROWS):
        splits = choose_num_splits(B, H, k.shape[1], M, N, lib.fa_num_cus(), splits)
    part_lse = torch.empty((B, H, splits, M), dtype=torch.float32, device=q.device)
    part_o = torch.empty((B, H, splits, M, D), dtype=torch.float16, device=q.device)
    _abi.fa_splitkv_fwd(lib, q, k, v, part_o, part_lse, causal, sm_scale, splits, _split_size(N, splits))
    if splits == 1:   # nothing to merge: the single piece is the result (a cast at most)
        o = part_o.squeeze(2)
        return (o if single_direct else o.to(q.dtype)), part_lse.squeeze(2)
    L = torch.empty((B, H, M), dtype=torch.float32, device=q.device)
    o = torch.empty_like(q)
    if not _abi.is_kernel_ready(o):
        o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    _abi.fa_splitkv_combine(lib, part_o, part_lse, o, L, splits)
    return o, L


def attention(q, k, v, causal=False, sm_scale=None):
    """Forward-only attention that always goes through the split-KV kernel (``split_kv.py:266-330``).

    With a single split the fp16 partial output is returned directly, as the reference does."""
    Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Dq == Dk == Dv
    assert Dk in (16, 32, 64, 128)
    B, H, M, D = q.shape
    N = k.shape[2]
    Hk, Hv = k.shape[1], v.shape[1]
    assert Hk == Hv, "num of heads in k and v should be equal"
    assert H % Hk == 0, "number of heads in q must be a multiple of that in k & v"
    if q.numel() == 0 or N == 0:      # nothing to launch; a row without keys is zero
        return torch.zeros(q.shape, dtype=q.dtype, device=q.device)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    lib = _lib.get()
    q, k, v = _abi.kernel_ready(q), _abi.kernel_ready(k), _abi.kernel_ready(v)
    with torch.cuda.device(q.device):
        block_m, block_n = split_units(B, H, M, N, D, causal)
        splits = num_splits_heuristic(B, H, M, N, block_m, block_n, lib.fa_num_cus(), 128)
        o, _ = split_kv_forward(lib, q, k, v, causal, sm_scale, splits, single_direct=True)
    return o
