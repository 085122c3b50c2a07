"""GPU parity tests of paged_attention.

Parametrisation and input distributions follow tests/flag_attn/test_paged_attention.py:9-143 of the
reference (uniform(-D^-0.5, D^-0.5) inputs, 1000 cache blocks, block tables drawn with repeats,
int64 tables, context_lens[0] = max).  Two acceptance checks:
  * the reference's own: allclose(out, fp32-math oracle rounded to fp16, atol=2e-3, rtol=1e-5);
  * the 2x rule against a same-precision (fp16 products) variant of the oracle.
"""
import pytest
import torch

import flagattention_amd as flag_attn
from oracle import paged_attention as oracle_paged, within_two_x

pytestmark = pytest.mark.gpu

NUM_BLOCKS = 1000


def run_case(num_seqs, num_query_heads, query_group_size, head_size, block_size, max_seq_len,
             num_splits=0, dtype=torch.float16, table_dtype=torch.int64, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    num_kv_heads = num_query_heads // query_group_size
    if max_seq_len > 1:
        context_lens = torch.randint(1, max_seq_len, [num_seqs], dtype=torch.int32, device="cuda", generator=g)
    else:
        context_lens = torch.ones([num_seqs], dtype=torch.int32, device="cuda")
    context_lens[0] = max_seq_len
    max_context_len = int(context_lens.max().item())
    max_blocks = (max_context_len + block_size - 1) // block_size
    scale = head_size ** -0.5
    q = torch.empty(num_seqs, num_query_heads, head_size, dtype=dtype, device="cuda").uniform_(-scale, scale, generator=g)
    k_cache = torch.empty(NUM_BLOCKS, num_kv_heads, block_size, head_size, dtype=dtype, device="cuda").uniform_(-scale, scale, generator=g)
    v_cache = torch.empty_like(k_cache).uniform_(-scale, scale, generator=g)
    block_tables = torch.randint(0, NUM_BLOCKS, (num_seqs, max_blocks), device="cuda", generator=g).to(table_dtype)

    out = flag_attn.paged_attention(q, k_cache, v_cache, context_lens, block_tables, scale, max_context_len, num_splits)
    ref = oracle_paged(q, k_cache, v_cache, block_tables, context_lens, scale)
    same = oracle_paged(q, k_cache, v_cache, block_tables, context_lens, scale, same_precision=True)
    assert out.shape == q.shape and out.dtype == dtype
    assert torch.allclose(out, ref, atol=2e-3, rtol=1e-5), f"max diff {(out - ref).abs().max().item():.3e}"
    ok, e_hyp, e_same = within_two_x(out, same, ref)
    assert ok, f"hip err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


@pytest.mark.parametrize("num_seqs", [1, 32])
@pytest.mark.parametrize("query_group_size", [1, 8])
@pytest.mark.parametrize("head_size", [64, 128])
@pytest.mark.parametrize("block_size", [16, 128, 256])
@pytest.mark.parametrize("max_seq_len", [512, 4096])
def test_paged_attention_default(num_seqs, query_group_size, head_size, block_size, max_seq_len):
    run_case(num_seqs, 64, query_group_size, head_size, block_size, max_seq_len)


@pytest.mark.parametrize("num_seqs", [1, 16])
@pytest.mark.parametrize("query_group_size", [1, 8])
@pytest.mark.parametrize("head_size", [32, 64])
@pytest.mark.parametrize("num_splits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_paged_attention_by_num_splits(num_seqs, query_group_size, head_size, num_splits):
    run_case(num_seqs, 64, query_group_size, head_size, 16, 2048, num_splits=num_splits)


@pytest.mark.parametrize("num_seqs,num_query_heads,query_group_size,head_size,block_size,max_seq_len,num_splits", [
    (1, 12, 1, 64, 16, 2, 0),
    (16, 64, 8, 32, 16, 2048, 2),
    (16, 64, 1, 64, 16, 2048, 6),
])
def test_paged_attention_by_case(num_seqs, num_query_heads, query_group_size, head_size, block_size,
                                 max_seq_len, num_splits):
    run_case(num_seqs, num_query_heads, query_group_size, head_size, block_size, max_seq_len, num_splits)


@pytest.mark.parametrize("head_size", [16, 256, 512])
@pytest.mark.parametrize("table_dtype", [torch.int32, torch.int64])
def test_other_head_sizes_and_table_types(head_size, table_dtype):
    run_case(4, 16, 4, head_size, 32, 700, table_dtype=table_dtype)


@pytest.mark.parametrize("num_splits", [0, 1, 3])
def test_head_size_512(num_splits):
    """The largest head size of the reference (paged.py:31): the kernel walks 16-key steps there."""
    run_case(6, 8, 2, 512, 16, 1500, num_splits=num_splits)
    run_case(3, 4, 1, 512, 16, 333, num_splits=num_splits, dtype=torch.bfloat16)


def test_bfloat16_and_large_group():
    run_case(3, 40, 40, 64, 16, 900, dtype=torch.bfloat16)


def test_baseline_decode_configuration_small_copy():
    """The benchmark's decode configuration (32 query heads over 8 kv heads, head 128, block 16) at a
    reduced number of sequences so that the token-gather oracle stays fast."""
    run_case(8, 32, 4, 128, 16, 8192)


def test_many_short_pairs_take_the_single_pass_launch():
    from flagattention_amd.paged import choose_launch
    assert choose_launch(700, 64, 1, 64, 300, 256)[0] == "single"
    run_case(700, 64, 1, 64, 16, 300)


def test_balanced_launch_skewed_contexts_with_an_empty_sequence():
    g = torch.Generator(device="cuda").manual_seed(3)
    num_seqs, Hq, Hkv, D, bs = 9, 16, 4, 128, 16
    context_lens = torch.tensor([5000, 1, 0, 129, 2047, 16, 0, 3001, 640], dtype=torch.int32, device="cuda")
    scale = D ** -0.5
    q = torch.empty(num_seqs, Hq, D, dtype=torch.float16, device="cuda").uniform_(-scale, scale, generator=g)
    k_cache = torch.empty(NUM_BLOCKS, Hkv, bs, D, dtype=torch.float16, device="cuda").uniform_(-scale, scale, generator=g)
    v_cache = torch.empty_like(k_cache).uniform_(-scale, scale, generator=g)
    block_tables = torch.randint(0, NUM_BLOCKS, (num_seqs, (5000 + bs - 1) // bs), device="cuda", generator=g)
    out = flag_attn.paged_attention(q, k_cache, v_cache, context_lens, block_tables, scale, 5000)
    live = context_lens > 0
    assert (out[~live] == 0).all()
    ref = oracle_paged(q[live], k_cache, v_cache, block_tables[live], context_lens[live], scale)
    same = oracle_paged(q[live], k_cache, v_cache, block_tables[live], context_lens[live], scale, same_precision=True)
    assert torch.allclose(out[live], ref, atol=2e-3, rtol=1e-5)
    ok, e_hyp, e_same = within_two_x(out[live], same, ref)
    assert ok, f"hip err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


def test_full_size_decode_launch_shapes_agree():
    """At the benchmark's size (64 sequences, contexts U[512, 8192], 32 query heads over 8 kv heads,
    head 128) the oracle's token gather is too slow, but how the keys are cut into pieces must not
    matter: the balanced launch, one pass and 4 or 16 partitions give the same output up to the fp16
    rounding of the partial results, and 8 sequences of it are checked against the oracle."""
    g = torch.Generator(device="cuda").manual_seed(10086)
    num_seqs, Hq, Hkv, D, bs = 64, 32, 8, 128, 16
    context_lens = torch.randint(512, 8193, (num_seqs,), dtype=torch.int32, device="cuda", generator=g)
    blocks_per_seq = (context_lens + bs - 1) // bs
    num_blocks = int(blocks_per_seq.sum())
    max_context_len = int(context_lens.max())
    scale = D ** -0.5
    q = torch.empty(num_seqs, Hq, D, dtype=torch.float16, device="cuda").uniform_(-scale, scale, generator=g)
    k_cache = torch.empty(num_blocks, Hkv, bs, D, dtype=torch.float16, device="cuda").uniform_(-scale, scale, generator=g)
    v_cache = torch.empty_like(k_cache).uniform_(-scale, scale, generator=g)
    block_tables = torch.randint(0, num_blocks, (num_seqs, (max_context_len + bs - 1) // bs), device="cuda", generator=g)
    outs = [flag_attn.paged_attention(q, k_cache, v_cache, context_lens, block_tables, scale, max_context_len, n)
            for n in (0, 1, 4, 16)]
    for o in outs[1:]:
        assert torch.allclose(outs[0].float(), o.float(), atol=1e-3, rtol=0)
    sub = slice(0, 8)
    ref = oracle_paged(q[sub], k_cache, v_cache, block_tables[sub], context_lens[sub], scale)
    assert torch.allclose(outs[0][sub], ref, atol=2e-3, rtol=1e-5)
