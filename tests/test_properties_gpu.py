"""Size-independent properties of the kernels at the benchmark's full sizes, where the fp32 oracle is
too slow to cover every element: they hold exactly (bit for bit) by construction of the algorithm, so
any indexing, masking or tile-ordering mistake that depends on the position in a large tensor breaks
them.
"""
import pytest
import torch

import flagattention_amd as flag_attn

pytestmark = pytest.mark.gpu

B, H, T, D = 1, 32, 8192, 128


def randn(shape, dtype, seed, grad=False):
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = torch.empty(shape, dtype=dtype, device="cuda").normal_(0.0, 1.0, generator=g)
    return t.requires_grad_() if grad else t


@pytest.fixture(scope="module", autouse=True)
def one_forward_kernel():
    """The properties below compare launches of different sizes bit for bit, so every launch has to take the
    same forward kernel: the tile hook (flash.get_fwd_config) names the 256-row kernel for all of them, where
    the default would pick the 128-row kernel for the small launches."""
    from flagattention_amd import flash
    mp = pytest.MonkeyPatch()
    mp.setattr(flash, "get_fwd_config", lambda B, H, M, N, D, causal: (256, 64, 5, 4))
    yield
    mp.undo()


@pytest.fixture(scope="module")
def full(one_forward_kernel):
    q, k, v = (randn((B, H, T, D), torch.bfloat16, s, grad=True) for s in (1, 2, 3))
    do = randn((B, H, T, D), torch.bfloat16, 4)
    o, L, tot, _, _ = flag_attn.flash_attention(q, k, v, causal=True, return_log_normalizer=True,
                                                return_total_attention=True)
    grads = torch.autograd.grad(o, (q, k, v), do, retain_graph=True)
    return q, k, v, do, o, L, tot, grads


def test_backward_is_exactly_linear_under_a_power_of_two(full):
    """dO -> 2 dO doubles delta, dP and dS exactly and commutes with every rounding to bf16, so every
    gradient doubles bit for bit (the dS-kept route at this size)."""
    q, k, v, do, o, _, _, grads = full
    doubled = torch.autograd.grad(o, (q, k, v), 2 * do, retain_graph=True)
    for name, g, g2 in zip(("dq", "dk", "dv"), grads, doubled):
        assert torch.equal(2 * g, g2), name


def test_heads_are_independent(full):
    """A head computed alone, through strided views of the full tensors, equals the same head computed
    in the full launch: forward outputs and all gradients, bit for bit."""
    q, k, v, do, o, L, tot, grads = full
    for h in (0, 13, 31):
        hs = slice(h, h + 1)
        qs, ks, vs = (t.detach()[:, hs].requires_grad_() for t in (q, k, v))
        o1, L1, tot1, _, _ = flag_attn.flash_attention(qs, ks, vs, causal=True, return_log_normalizer=True,
                                                       return_total_attention=True)
        g1 = torch.autograd.grad(o1, (qs, ks, vs), do[:, hs])
        assert torch.equal(o1, o[:, hs]) and torch.equal(L1, L[:, hs]) and torch.equal(tot1, tot[:, hs])
        for name, a, b in zip(("dq", "dk", "dv"), g1, grads):
            assert torch.equal(a, b[:, hs]), (name, h)


def test_causal_prefix(full):
    """With the causal mask and equal lengths, the first T' rows of the output depend on the first T'
    keys only and walk the same tiles in the same order: truncating the sequence changes nothing."""
    q, k, v, _, o, L, _, _ = full
    for t in (128, 1000, 4097):
        o1, L1, _, _, _ = flag_attn.flash_attention(q.detach()[:, :, :t], k.detach()[:, :, :t], v.detach()[:, :, :t],
                                                    causal=True, return_log_normalizer=True)
        assert torch.equal(o1, o[:, :, :t]) and torch.equal(L1, L[:, :, :t]), t


def test_total_attention_sums_to_the_number_of_rows(full):
    """Every query row distributes a total probability of 1 over the keys."""
    _, _, _, _, _, _, tot, _ = full
    sums = tot.double().sum(-1)
    assert torch.allclose(sums, torch.full_like(sums, float(T)), rtol=2e-3)
    assert (tot >= 0).all()


def test_log_normalizer_bounds(full):
    """L = logsumexp of the visible scaled scores: at least the largest of them (row m's own key m is
    visible) and at most that maximum plus log(number of visible keys)."""
    q, k, _, _, _, L, _, _ = full
    m = torch.arange(T, device="cuda")
    own = (q.detach().float() * k.detach().float()).sum(-1) * D ** -0.5     # score of (m, m)
    assert (L >= own - 1e-2).all()
    assert (L[:, :, 0] - own[:, :, 0]).abs().max() < 2e-2                      # row 0 sees one key
    assert torch.isfinite(L).all() and m.numel() == L.shape[-1]


def test_offsets_beyond_two_to_the_31_elements():
    """Tensors with more than 2^31 elements (batch 66 of the benchmark shape; 4.4 GB each): the last
    (batch, head) slice, whose element offsets need 64 bits, equals the same slice computed alone --
    forward, log-normalizer and all gradients (the backward runs in bounded-workspace slices)."""
    Bb = 66
    assert Bb * H * T * D > 2 ** 31
    q, k, v = (randn((Bb, H, T, D), torch.bfloat16, s, grad=True) for s in (11, 12, 13))
    do = randn((Bb, H, T, D), torch.bfloat16, 14)
    o, L, _, _, _ = flag_attn.flash_attention(q, k, v, causal=True, return_log_normalizer=True)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), do)
    s = (slice(Bb - 1, Bb), slice(H - 1, H))
    qs, ks, vs = (t.detach()[s].requires_grad_() for t in (q, k, v))
    o1, L1, _, _, _ = flag_attn.flash_attention(qs, ks, vs, causal=True, return_log_normalizer=True)
    g1 = torch.autograd.grad(o1, (qs, ks, vs), do[s])
    assert torch.equal(o1, o[s]) and torch.equal(L1, L[s])
    for name, a, b in zip(("dq", "dk", "dv"), g1, (dq, dk, dv)):
        assert torch.equal(a, b[s]), name
    assert torch.isfinite(o.float()).all()


def test_paged_cache_beyond_two_to_the_31_elements():
    """A key/value cache of 2.3 G elements per tensor, the sequences' blocks taken from its top end:
    block offsets need 64 bits.  Compared with the same blocks copied into a small cache."""
    num_blocks, hkv, bs, Dh, hq, num_seqs, ctx = 140000, 8, 16, 128, 32, 8, 2000
    assert num_blocks * hkv * bs * Dh > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(5)
    kc = torch.empty((num_blocks, hkv, bs, Dh), dtype=torch.float16, device="cuda")
    vc = torch.empty_like(kc)
    per_seq = (ctx + bs - 1) // bs
    used = num_seqs * per_seq
    top = slice(num_blocks - used, num_blocks)
    kc[top].normal_(0.0, 1.0, generator=g)
    vc[top].normal_(0.0, 1.0, generator=g)
    q = randn((num_seqs, hq, Dh), torch.float16, 6)
    lens = torch.randint(1, ctx, (num_seqs,), dtype=torch.int32, device="cuda", generator=g)
    lens[0] = ctx
    perm = torch.randperm(used, device="cuda", generator=g)
    table_small = perm.reshape(num_seqs, per_seq).int()
    table_big = (table_small.long() + (num_blocks - used))
    for splits in (0, 1, 4):
        big = flag_attn.paged_attention(q, kc, vc, lens, table_big, Dh ** -0.5, ctx, num_splits=splits)
        small = flag_attn.paged_attention(q, kc[top].contiguous(), vc[top].contiguous(), lens, table_small,
                                          Dh ** -0.5, ctx, num_splits=splits)
        assert torch.equal(big, small), splits
