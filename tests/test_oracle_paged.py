"""Pins the paged-attention oracle: token-by-token fp64 gather, equivalence with dense single-query
attention, and invariance under a relabelling of the cache blocks."""
import math

import pytest
import torch

from oracle import flash_attention, paged_attention, max_abs_diff

torch.manual_seed(10086)


def make_case(num_seqs, Hq, Hk, D, block, max_len, num_blocks=64, dtype=torch.float32):
    lens = torch.randint(1, max_len + 1, (num_seqs,), dtype=torch.int32)
    lens[0] = max_len
    max_blocks = (max_len + block - 1) // block
    q = torch.randn(num_seqs, Hq, D, dtype=dtype)
    kc = torch.randn(num_blocks, Hk, block, D, dtype=dtype)
    vc = torch.randn(num_blocks, Hk, block, D, dtype=dtype)
    bt = torch.randint(0, num_blocks, (num_seqs, max_blocks))
    return q, kc, vc, bt, lens


def token_loop(q, kc, vc, bt, lens, scale):
    S, Hq, D = q.shape
    Hk, block = kc.shape[1], kc.shape[2]
    g = Hq // Hk
    out = torch.zeros(S, Hq, D, dtype=torch.float64)
    for s in range(S):
        for h in range(Hq):
            sc = []
            for j in range(int(lens[s])):
                blk = int(bt[s, j // block])
                sc.append(scale * float(torch.dot(q[s, h].double(), kc[blk, h // g, j % block].double())))
            top = max(sc)
            z = sum(math.exp(x - top) for x in sc)
            for j, x in enumerate(sc):
                blk = int(bt[s, j // block])
                out[s, h] += math.exp(x - top) / z * vc[blk, h // g, j % block].double()
    return out


@pytest.mark.parametrize("Hq,Hk", [(4, 4), (8, 2), (4, 1)])
@pytest.mark.parametrize("block,max_len", [(4, 13), (16, 16), (8, 1)])
def test_matches_token_loop(Hq, Hk, block, max_len):
    q, kc, vc, bt, lens = make_case(3, Hq, Hk, 8, block, max_len)
    o = paged_attention(q, kc, vc, bt, lens, 0.3)
    assert max_abs_diff(o, token_loop(q, kc, vc, bt, lens, 0.3).float()) < 2e-6


def test_equals_dense_single_query_attention():
    q, kc, vc, bt, lens = make_case(4, 8, 2, 16, 8, 37)
    o = paged_attention(q, kc, vc, bt, lens, 0.25)
    for s in range(4):
        n = int(lens[s])
        nb = (n + 7) // 8
        k = kc[bt[s, :nb]].permute(1, 0, 2, 3).reshape(1, 2, -1, 16)[:, :, :n]
        v = vc[bt[s, :nb]].permute(1, 0, 2, 3).reshape(1, 2, -1, 16)[:, :, :n]
        dense = flash_attention(q[s].reshape(1, 8, 1, 16), k, v, False, 0.25, upcast=True)
        assert max_abs_diff(o[s], dense.reshape(8, 16)) < 2e-6


def test_invariant_under_block_relabelling():
    q, kc, vc, bt, lens = make_case(3, 4, 2, 8, 4, 19, num_blocks=32)
    perm = torch.randperm(32)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(32)
    o1 = paged_attention(q, kc, vc, bt, lens, 0.5)
    o2 = paged_attention(q, kc[perm], vc[perm], inv[bt], lens, 0.5)
    assert max_abs_diff(o1, o2) == 0.0


def test_same_precision_variant_is_close_but_rounded():
    q, kc, vc, bt, lens = make_case(2, 4, 2, 16, 8, 40, dtype=torch.float16)
    ref = paged_attention(q, kc, vc, bt, lens, 0.25)
    sp = paged_attention(q, kc, vc, bt, lens, 0.25, same_precision=True)
    assert ref.dtype == sp.dtype == torch.float16
    assert max_abs_diff(ref, sp) < 2e-2
