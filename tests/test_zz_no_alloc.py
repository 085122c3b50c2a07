"""GPU test of ``paged_attn_balanced_static``: the paged decode entry point that allocates nothing (its
partial-result slots live in a static device array inside the library), against ``paged_attn_balanced``
with a caller-provided workspace.  The two share their kernels, so the outputs must be bit-equal; the
reference's ``atol=2e-3`` against the oracle (tests/flag_attn/test_paged_attention.py:53-62 of the
reference) is checked as well.  Two calls in a row, the second with a smaller input, so that the
second runs on a scratch that still holds the first call's partial results."""
import pytest
import torch

from flagattention_amd import _abi, _lib
from oracle import paged_attention as oracle_paged

pytestmark = pytest.mark.gpu


def make_case(seed, num_seqs, Hq, Hkv, D, bs, lo, hi):
    g = torch.Generator(device="cuda").manual_seed(seed)
    ctx = torch.randint(lo, hi + 1, (num_seqs,), device="cuda", generator=g, dtype=torch.int32)
    max_ctx = int(ctx.max().item())
    nblocks = 4096
    scale = D ** -0.5
    q = torch.empty(num_seqs, Hq, D, dtype=torch.float16, device="cuda").uniform_(-scale, scale, generator=g)
    kc = torch.empty(nblocks, Hkv, bs, D, dtype=torch.float16, device="cuda").uniform_(-scale, scale, generator=g)
    vc = torch.empty_like(kc).uniform_(-scale, scale, generator=g)
    bt = torch.randint(0, nblocks, (num_seqs, (max_ctx + bs - 1) // bs), device="cuda", generator=g)
    return q, kc, vc, ctx, bt, scale


def test_static_scratch_entry_point_matches_workspace_entry_point_twice():
    lib = _lib.get()
    with torch.cuda.device(0):   # what a caller does before it starts a stream capture: resolves the array's address
        assert lib.paged_attn_balanced_static_prepare() == 0
    num_wgs = 2 * lib.fa_num_cus()
    # first a launch whose pairs are cut over many workgroups, then a smaller one
    for seed, (num_seqs, Hq, Hkv, D, bs, lo, hi) in enumerate([(24, 32, 8, 128, 16, 512, 6000),
                                                               (5, 32, 8, 128, 16, 100, 900)]):
        q, kc, vc, ctx, bt, scale = make_case(seed, num_seqs, Hq, Hkv, D, bs, lo, hi)
        ws = torch.empty(lib.paged_attn_balanced_workspace(num_wgs, D) // 4, dtype=torch.float32, device="cuda")
        out_ws = torch.full_like(q, float("nan"))
        _abi.paged_attn_balanced(lib, out_ws, q, kc, vc, ctx, bt, scale, ws, num_wgs)
        out_static = torch.full_like(q, float("nan"))
        free_before = torch.cuda.mem_get_info()[0]
        _abi.paged_attn_balanced_static(lib, out_static, q, kc, vc, ctx, bt, scale, num_wgs)
        torch.cuda.synchronize()
        if seed > 0:   # the first call on a device looks up (and so loads) the static array: set-up
            assert torch.cuda.mem_get_info()[0] == free_before   # nothing allocated on the device
        assert torch.equal(out_static, out_ws), f"call {seed}: static-scratch output differs"
        ref = oracle_paged(q, kc, vc, bt, ctx, scale)
        assert torch.allclose(out_static, ref, atol=2e-3, rtol=1e-5)


def test_static_scratch_entry_point_rejects_oversized_launch():
    lib = _lib.get()
    q, kc, vc, ctx, bt, scale = make_case(9, 2, 8, 2, 128, 16, 20, 40)
    out = torch.empty_like(q)
    assert lib.paged_attn_balanced_workspace(4096, 128) > _lib.STATIC_SCRATCH_BYTES
    with pytest.raises(AssertionError, match="scratch"):
        _abi.paged_attn_balanced_static(lib, out, q, kc, vc, ctx, bt, scale, 4096)
