"""The kernels are launched on torch's current stream and contain no host synchronisation, so they can
run on side streams and be captured into HIP graphs.  A captured graph is replayed several times with
new inputs, with eager work and synchronisations between the replays, and every replay is compared
with the eager result.
"""
import pytest
import torch

import flagattention_amd as flag_attn

pytestmark = pytest.mark.gpu


def randn(shape, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.empty(shape, dtype=dtype, device="cuda").normal_(0.0, 1.0, generator=g)


def paged_inputs(seed, num_seqs=16, hq=32, hkv=8, D=128, bs=16, max_len=3000):
    g = torch.Generator(device="cuda").manual_seed(seed)
    lens = torch.randint(1, max_len, (num_seqs,), dtype=torch.int32, device="cuda", generator=g)
    lens[0] = max_len
    blocks = (max_len + bs - 1) // bs
    nb = num_seqs * blocks
    q = randn((num_seqs, hq, D), torch.float16, seed + 1)
    kc = randn((nb, hkv, bs, D), torch.float16, seed + 2)
    vc = randn((nb, hkv, bs, D), torch.float16, seed + 3)
    table = torch.randperm(nb, device="cuda", generator=g).reshape(num_seqs, blocks).int()
    return q, kc, vc, lens, table, D ** -0.5, max_len


def test_side_stream_gives_the_default_stream_results():
    q, k, v = (randn((2, 8, 1024, 128), torch.bfloat16, s).requires_grad_() for s in (1, 2, 3))
    do = randn((2, 8, 1024, 128), torch.bfloat16, 4)
    o0 = flag_attn.flash_attention(q, k, v, causal=True)
    g0 = torch.autograd.grad(o0, (q, k, v), do)
    p = paged_inputs(7)
    d0 = flag_attn.paged_attention(*p)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    busy = randn((4096, 4096), torch.float32, 9)
    with torch.cuda.stream(side):
        o1 = flag_attn.flash_attention(q, k, v, causal=True)
        g1 = torch.autograd.grad(o1, (q, k, v), do)
        d1 = flag_attn.paged_attention(*p)
    for _ in range(4):                      # unrelated work on the default stream at the same time
        busy = busy @ busy * 1e-4
    side.synchronize()
    torch.cuda.synchronize()
    assert torch.equal(o0, o1) and torch.equal(d0, d1)
    for a, b in zip(g0, g1):
        assert torch.equal(a, b)


def test_forward_and_paged_decode_replay_from_a_graph():
    q, k, v = (randn((1, 8, 2048, 128), torch.bfloat16, s) for s in (1, 2, 3))
    p = list(paged_inputs(11))
    # warm up on a side stream, as graph capture requires
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            flag_attn.flash_attention(q, k, v, causal=True)
            flag_attn.paged_attention(*p)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g = flag_attn.flash_attention(q, k, v, causal=True)
        d_g = flag_attn.paged_attention(*p)
    for seed in (21, 22, 23):
        q.copy_(randn(q.shape, q.dtype, seed))
        p[0].copy_(randn(p[0].shape, p[0].dtype, seed + 100))
        p[3][1:] = torch.randint(1, p[6], (p[3].numel() - 1,), dtype=torch.int32, device="cuda")
        graph.replay()
        torch.cuda.synchronize()
        o_e = flag_attn.flash_attention(q, k, v, causal=True)
        d_e = flag_attn.paged_attention(*p)
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e), seed
        assert torch.equal(d_g, d_e), seed
