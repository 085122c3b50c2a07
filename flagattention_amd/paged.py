"""``paged_attention``: single-token decode over a block-table-indexed key/value cache.

Host-side counterpart of ``src/flag_attn/paged.py:6-163`` of the reference: same signature, same
meaning of ``num_splits`` (0 = choose, 1 = one pass, > 1 = that many partitions of
``next_power_of_2(ceil(max_context_len / num_splits))`` tokens), partitions merged by a reduce kernel.
"""
import torch

from . import _abi, _lib

__all__ = ["attention"]

_HEAD_SIZES = (16, 32, 64, 128, 256, 512)


def _next_pow2(x):
    return 1 << max(0, (int(x) - 1).bit_length())


def choose_launch(num_seqs, num_kv_heads, group, head_size, max_context_len, num_cus):
    """Launch shape for ``num_splits == 0`` on a device with ``num_cus`` compute units.

    Returns ("balanced", num_workgroups) or ("single", 0).  The balanced launch divides the keys of
    all (sequence, kv head) pairs evenly over one resident wave of workgroups (two per compute unit
    fit up to head size 128, one above) and so does not depend on how the context lengths are
    spread; its fixed cost (a scan of the context lengths per workgroup, a merge kernel) only loses
    against one workgroup per pair when there are many more short pairs than workgroups, where the
    hardware's own dispatch already evens things out."""
    num_wgs = num_cus * (2 if head_size <= 128 else 1)
    pairs = num_seqs * num_kv_heads * (-(-group // 16))
    if pairs >= 8 * num_wgs and max_context_len <= 2048:
        return "single", 0
    return "balanced", num_wgs


_NUM_CUS = {}


def _num_cus(lib, device):
    """Compute units of ``device`` (asked once; the current device is ``device`` when this is called)."""
    key = (device.index if device.index is not None else torch.cuda.current_device()) if device.type == "cuda" else -1
    if key not in _NUM_CUS:
        _NUM_CUS[key] = lib.fa_num_cus()
    return _NUM_CUS[key]


def attention(query, key_cache, value_cache, context_lens, block_tables, attn_scale,
              max_context_len, num_splits=0):
    """query (num_seqs, heads_q, head_size); key_cache / value_cache (num_blocks, heads_kv, block_size,
    head_size) with identical strides; context_lens (num_seqs,) of any integer type; block_tables (num_seqs,
    max_blocks_per_seq) int32 or int64.  Returns out shaped like ``query``; a sequence of context length
    0 gets a zero row."""
    num_seqs, num_q_heads, head_size = query.shape
    num_kv_heads, block_size = key_cache.shape[1], key_cache.shape[2]
    assert key_cache.shape[3] == head_size and value_cache.shape == key_cache.shape
    assert head_size in _HEAD_SIZES, f"head_size={head_size}"
    assert num_q_heads % num_kv_heads == 0
    assert key_cache.stride() == value_cache.stride(), "key and value cache must share their strides"
    assert not context_lens.dtype.is_floating_point and context_lens.dtype != torch.bool, \
        f"context_lens must hold integers, got {context_lens.dtype}"

    if num_seqs == 0:      # nothing to launch
        return torch.empty_like(query)
    lib = _lib.get()
    if query.stride(-1) != 1 or query.data_ptr() % 16 or query.stride(0) % 8 or query.stride(1) % 8:
        query = query.contiguous()
    assert key_cache.stride(-1) == 1
    if context_lens.dtype != torch.int32:   # the kernels read 32-bit lengths (the reference takes any integer type)
        context_lens = context_lens.to(torch.int32)
    context_lens = context_lens.contiguous()
    if block_tables.stride(-1) != 1:
        block_tables = block_tables.contiguous()
    out = torch.empty_like(query)   # the caller's layout, as paged.py:16 of the reference, when the kernels can write it
    if out.stride(-1) != 1 or out.data_ptr() % 16 or out.stride(0) % 8 or out.stride(1) % 8:
        out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
    group = num_q_heads // num_kv_heads

    with torch.cuda.device(query.device):
        if num_splits == 0:
            kind, num_wgs = choose_launch(num_seqs, num_kv_heads, group, head_size, max_context_len,
                                          _num_cus(lib, query.device))
            if kind == "balanced":
                nbytes = lib.paged_attn_balanced_workspace(num_wgs, head_size)
                workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=query.device)
                _abi.paged_attn_balanced(lib, out, query, key_cache, value_cache, context_lens,
                                         block_tables, attn_scale, workspace, num_wgs)
                return out
            num_splits = 1
        if num_splits > 1:
            partition_size = _next_pow2(-(-max_context_len // num_splits))
            assert partition_size >= block_size and partition_size % block_size == 0, \
                f"partition_size={partition_size}, kv_block_size={block_size}"
        if num_splits == 1:
            _abi.paged_attn(lib, out, query, key_cache, value_cache, context_lens, block_tables,
                            attn_scale, 0, 1, None, None, None)
        else:
            shape = (num_seqs, num_kv_heads, num_splits, group)
            max_logits = torch.empty(shape, dtype=torch.float32, device=query.device)
            exp_sums = torch.empty(shape, dtype=torch.float32, device=query.device)
            tmp_out = torch.empty(shape + (head_size,), dtype=out.dtype, device=out.device)
            _abi.paged_attn(lib, out, query, key_cache, value_cache, context_lens, block_tables,
                            attn_scale, partition_size, num_splits, tmp_out, max_logits, exp_sums)
            _abi.paged_reduce(lib, out, tmp_out, max_logits, exp_sums, context_lens, num_kv_heads,
                              partition_size, num_splits)
    return out
