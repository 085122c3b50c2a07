"""Plain-torch statement of single-query attention over a paged key/value cache.

Test infrastructure only (see the package docstring).  Follows
``src/flag_attn/testing/paged.py:5-52`` of the reference: for each sequence the first
``context_len`` tokens are gathered through its row of the block table (token ``j`` lives in cache
block ``block_table[j // block_size]`` at slot ``j % block_size``, ``:31-37``), kv heads are
repeated over their query group (``:40-43``), and attention runs in fp32 with the result rounded to
the cache dtype (``:45-48``).  The gather here is one ``index_select`` per sequence instead of a
token loop; the arithmetic is the same.

``same_precision=True`` is an addition the reference does not have: both products run in the cache
dtype (scores rounded to 16 bits before the fp32 softmax, probabilities rounded before the second
product), which gives the same-precision comparator that the 2x acceptance rule needs.
"""
import torch


def paged_attention(query, key_cache, value_cache, block_tables, context_lens, scale,
                    same_precision=False):
    """query (S, Hq, D); caches (num_blocks, Hk, block, D); block_tables (S, max_blocks) int;
    context_lens (S,) int.  Returns (S, Hq, D) in the query dtype."""
    num_seqs, num_q_heads, head_size = query.shape
    _, num_kv_heads, block_size, _ = value_cache.shape
    group = num_q_heads // num_kv_heads
    out = torch.empty_like(query)
    tables = block_tables.to("cpu").tolist()
    lens = context_lens.to("cpu").tolist()
    for s in range(num_seqs):
        n = int(lens[s])
        used_blocks = (n + block_size - 1) // block_size
        ids = torch.tensor(tables[s][:used_blocks], dtype=torch.long, device=query.device)
        # (blocks, Hk, block, D) -> (Hk, tokens, D), cut to the context length
        keys = key_cache.index_select(0, ids).permute(1, 0, 2, 3).reshape(num_kv_heads, -1, head_size)[:, :n]
        vals = value_cache.index_select(0, ids).permute(1, 0, 2, 3).reshape(num_kv_heads, -1, head_size)[:, :n]
        if group > 1:
            keys = keys.repeat_interleave(group, dim=0)
            vals = vals.repeat_interleave(group, dim=0)
        q = query[s].unsqueeze(1)  # (Hq, 1, D)
        if same_precision:
            scores = (torch.bmm(q, keys.transpose(1, 2)) * scale).to(torch.float32)
            probs = torch.softmax(scores, dim=-1).to(vals.dtype)
            res = torch.bmm(probs, vals)
        else:
            scores = torch.bmm(q.to(torch.float32), keys.to(torch.float32).transpose(1, 2)) * scale
            probs = torch.softmax(scores, dim=-1)
            res = torch.bmm(probs, vals.to(torch.float32))
        out[s] = res.squeeze(1).to(out.dtype)
    return out
