"""GPU parity tests of flash_attention (forward, split-KV path, backward, auxiliary outputs).

Shapes, scales and layouts follow the reference's own tests
(tests/flag_attn/test_flash_attention.py:20-222).  Acceptance rule, written out: for every output
x in {o, log-normalizer, total attention, dq, dk, dv}

    max|x_hip - x_fp32| <= 2 * max|x_torch_same_precision - x_fp32| + 1e-5

where both comparators come from the plain-torch oracle evaluated on the same device and inputs.
"""
import pytest
import torch

import flagattention_amd as flag_attn
from oracle import flash_attention as oracle_flash, within_two_x

pytestmark = pytest.mark.gpu

FWD_SHAPES = [
    (2, 4, 4, 512, 612, 128), (2, 4, 4, 1024, 1034, 64), (2, 4, 4, 2048, 2048, 32),
    (2, 4, 4, 4096, 4096, 16), (2, 4, 4, 4001, 4001, 32), (2, 4, 4, 4001, 4096, 64),
    (2, 4, 4, 4096, 4000, 128), (1, 2, 2, 8192, 8202, 16), (1, 2, 2, 8192, 8192, 32),
    # grouped / multi-query heads
    (2, 4, 2, 512, 612, 128), (2, 4, 1, 1024, 1034, 64), (2, 4, 2, 2048, 2048, 32),
    (2, 4, 1, 4096, 4096, 16), (2, 4, 2, 4001, 4001, 32), (2, 4, 1, 4001, 4096, 64),
    (2, 4, 2, 4096, 4000, 128), (1, 2, 1, 8192, 8202, 16), (1, 2, 1, 8192, 8192, 32),
]
SPLIT_SHAPES = [
    (2, 4, 4, 1, 612, 128), (2, 4, 4, 1, 1034, 64), (2, 4, 4, 1, 2048, 32), (2, 4, 4, 1, 4096, 16),
    (2, 4, 4, 1, 4001, 32), (2, 4, 4, 1, 4096, 64), (2, 4, 4, 2, 4000, 128), (1, 2, 2, 4, 8202, 16),
    (1, 2, 2, 1, 8192, 32),
    (2, 4, 2, 1, 612, 128), (2, 4, 1, 1, 1034, 64), (2, 4, 2, 1, 2048, 32), (2, 4, 1, 1, 4096, 16),
    (2, 4, 2, 1, 4001, 32), (2, 4, 1, 1, 4096, 64), (2, 4, 2, 2, 4000, 128), (1, 2, 1, 4, 8202, 16),
    (1, 2, 1, 1, 8192, 32),
]
BWD_SHAPES = [
    (2, 4, 4, 512, 612, 128), (2, 4, 4, 1024, 1034, 64), (2, 4, 4, 2048, 2048, 32),
    (2, 4, 4, 4096, 4096, 16), (2, 4, 4, 4001, 4001, 32), (2, 4, 4, 4001, 4096, 64),
    (2, 4, 4, 4096, 4001, 128), (1, 2, 2, 8192, 8202, 16), (1, 2, 2, 8192, 8192, 32),
    (2, 4, 4, 10006, 10, 128),
    (2, 4, 2, 512, 612, 128), (2, 4, 1, 1024, 1034, 64), (2, 4, 2, 2048, 2048, 32),
    (2, 4, 1, 4096, 4096, 16), (2, 4, 2, 4001, 4001, 32), (2, 4, 1, 4001, 4096, 64),
    (2, 4, 2, 4096, 4001, 128), (1, 2, 1, 8192, 8202, 16), (1, 2, 1, 8192, 8192, 32),
    (2, 4, 2, 10006, 10, 128),
]
AUX_SHAPES = [
    (2, 4, 512, 612, 128), (2, 4, 1024, 1034, 64), (2, 4, 2048, 2048, 32), (2, 4, 4096, 4096, 16),
    (2, 4, 4001, 4001, 32), (2, 4, 4001, 4096, 64), (2, 4, 4096, 4001, 128), (1, 2, 8192, 8202, 16),
    (1, 2, 8192, 8192, 32),
]


def make(shape, dtype, order, std, seed, grad=False):
    g = torch.Generator(device="cuda").manual_seed(seed)
    B, H, T, D = shape
    if order == "BHTD":
        t = torch.empty((B, H, T, D), dtype=dtype, device="cuda").normal_(0.0, std, generator=g)
    else:
        t = torch.empty((B, T, H, D), dtype=dtype, device="cuda").normal_(0.0, std, generator=g).transpose(1, 2)
    return t.requires_grad_() if grad else t


def check(name, hyp, same, ref, strict=False):
    ok, e_hyp, e_same = within_two_x(hyp, same, ref, strict=strict)
    assert ok, f"{name}: hip err {e_hyp:.3e} vs same-precision torch err {e_same:.3e}"


@pytest.mark.parametrize("scale", [1.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("B,Hq,Hk,M,N,D", FWD_SHAPES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
def test_attention_fwd(B, Hq, Hk, M, N, D, causal, order, dtype, scale):
    q = make((B, Hq, M, D), dtype, order, scale, 1)
    k = make((B, Hk, N, D), dtype, order, scale, 2)
    v = make((B, Hk, N, D), dtype, order, scale, 3)
    ref = oracle_flash(q, k, v, causal, upcast=True)
    same = oracle_flash(q, k, v, causal, upcast=False)
    hyp = flag_attn.flash_attention(q, k, v, causal)
    assert hyp.shape == q.shape and hyp.dtype == dtype
    check("o", hyp, same, ref)


@pytest.mark.parametrize("scale", [10.0])
@pytest.mark.parametrize("B,Hq,Hk,M,N,D", SPLIT_SHAPES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
def test_attention_splitkv(B, Hq, Hk, M, N, D, causal, order, dtype, scale):
    q = make((B, Hq, M, D), dtype, order, scale, 1)
    k = make((B, Hk, N, D), dtype, order, scale, 2)
    v = make((B, Hk, N, D), dtype, order, scale, 3)
    ref = oracle_flash(q, k, v, causal, upcast=True)
    same = oracle_flash(q, k, v, causal, upcast=False)
    hyp = flag_attn.flash_attention(q, k, v, causal)
    check("o", hyp, same, ref)


@pytest.mark.parametrize("scale", [1.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("B,Hq,Hk,M,N,D", BWD_SHAPES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
def test_attention_bwd(B, Hq, Hk, M, N, D, causal, order, dtype, scale):
    q = make((B, Hq, M, D), dtype, order, scale, 1, grad=True)
    k = make((B, Hk, N, D), dtype, order, scale, 2, grad=True)
    v = make((B, Hk, N, D), dtype, order, scale, 3, grad=True)
    do = make((B, Hq, M, D), dtype, order, 1.0, 4)
    o_ref = oracle_flash(q, k, v, causal, upcast=True)
    o_same = oracle_flash(q, k, v, causal, upcast=False)
    o_hyp = flag_attn.flash_attention(q, k, v, causal)
    g_ref = torch.autograd.grad(o_ref, (q, k, v), do)
    g_same = torch.autograd.grad(o_same, (q, k, v), do)
    g_hyp = torch.autograd.grad(o_hyp, (q, k, v), do)
    # strict "<", as the reference's backward tests compare (test_flash_attention.py:174-177, 317-320)
    check("o", o_hyp, o_same, o_ref, strict=True)
    for name, h, s, r in zip(("dq", "dk", "dv"), g_hyp, g_same, g_ref):
        assert h.shape == r.shape
        check(name, h, s, r, strict=True)


@pytest.mark.parametrize("scale", [1.0, 2.0, 3.0, 4.0])
@pytest.mark.parametrize("B,H,M,N,D", AUX_SHAPES)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
def test_attention_with_aux_outs(B, H, M, N, D, causal, order, dtype, scale):
    """The reference runs this test non-causal only; the causal half is added here."""
    q = make((B, H, M, D), dtype, order, scale, 1)
    k = make((B, H, N, D), dtype, order, scale, 2)
    v = make((B, H, N, D), dtype, order, scale, 3)
    ref = oracle_flash(q, k, v, causal, upcast=True, return_log_normalizer=True, return_total_attention=True)
    same = oracle_flash(q, k, v, causal, upcast=False, return_log_normalizer=True, return_total_attention=True)
    o, lse, tot, seed, offset = flag_attn.flash_attention(
        q, k, v, causal, return_log_normalizer=True, return_total_attention=True)
    assert seed is None and offset is None
    check("o", o, same[0], ref[0])
    check("log_normalizer", lse, same[1], ref[1])
    check("total_attention", tot, same[2], ref[2])


def test_return_convention_and_asserts():
    q = make((1, 2, 64, 32), torch.float16, "BHTD", 1.0, 1)
    k = make((1, 2, 64, 32), torch.float16, "BHTD", 1.0, 2)
    v = make((1, 2, 64, 32), torch.float16, "BHTD", 1.0, 3)
    assert isinstance(flag_attn.flash_attention(q, k, v), torch.Tensor)
    outs = flag_attn.flash_attention(q, k, v, return_log_normalizer=True)
    assert len(outs) == 5 and outs[2] is None and outs[1].shape == (1, 2, 64)
    with pytest.raises(AssertionError):
        flag_attn.flash_attention(q[..., :24], k[..., :24], v[..., :24])  # head dim not in {16,32,64,128}
    with pytest.raises(AssertionError):
        flag_attn.flash_attention(q, k[:, :1].expand(1, 3, 64, 32), v[:, :1].expand(1, 3, 64, 32))
    with pytest.raises(AssertionError):
        flag_attn.flash_attention(q, k, v, dropout_p=1.0)


@pytest.mark.parametrize("causal", [False, True])
def test_flash_attention_split_kv_entry(causal):
    q = make((2, 8, 1, 128), torch.float16, "BHTD", 1.0, 1)
    k = make((2, 2, 3000, 128), torch.float16, "BHTD", 1.0, 2)
    v = make((2, 2, 3000, 128), torch.float16, "BHTD", 1.0, 3)
    ref = oracle_flash(q, k, v, causal, upcast=True)
    same = oracle_flash(q, k, v, causal, upcast=False)
    hyp = flag_attn.flash_attention_split_kv(q, k, v, causal)
    check("o", hyp, same, ref)


def _grads(q, k, v, do, causal):
    o = flag_attn.flash_attention(q, k, v, causal)
    return (o,) + torch.autograd.grad(o, (q, k, v), do)


@pytest.mark.parametrize("Hk", [8, 2])
def test_backward_with_bounded_ds_workspace_matches_unbounded(Hk, monkeypatch):
    """Head size 128 keeps dS in a workspace for the dQ kernel; with a small limit the backward walks
    the batch and the heads in slices.  Both must give the very same bits; dK and dV also equal those
    of the route that recomputes dS (limit 0), whose dQ agrees to rounding."""
    from flagattention_amd import flash as flash_mod
    q = make((2, 8, 1024, 128), torch.bfloat16, "BTHD", 1.0, 1, grad=True)
    k = make((2, Hk, 1100, 128), torch.bfloat16, "BTHD", 1.0, 2, grad=True)
    v = make((2, Hk, 1100, 128), torch.bfloat16, "BTHD", 1.0, 3, grad=True)
    do = make((2, 8, 1024, 128), torch.bfloat16, "BHTD", 1.0, 4)
    lib = flash_mod._lib.get()
    per_head = lib.fa_bwd_ds_workspace_mib(1, 1, 1024, 1100)
    assert flash_mod.ds_heads_per_launch(lib, 2, 8, 8 // Hk, 1024, 1100, 128) == 16
    whole = _grads(q, k, v, do, True)
    monkeypatch.setattr(flash_mod, "DS_WORKSPACE_LIMIT_MIB", 5 * per_head)   # 4 (or 5) heads per launch
    assert 0 < flash_mod.ds_heads_per_launch(lib, 2, 8, 8 // Hk, 1024, 1100, 128) < 16
    sliced = _grads(q, k, v, do, True)
    monkeypatch.setattr(flash_mod, "DS_WORKSPACE_LIMIT_MIB", 0)
    assert flash_mod.ds_heads_per_launch(lib, 2, 8, 8 // Hk, 1024, 1100, 128) == 0
    recomputed = _grads(q, k, v, do, True)
    for name, a, b, c in zip(("o", "dq", "dk", "dv"), whole, sliced, recomputed):
        assert torch.equal(a, b), name
        if name == "dq":   # same products and the same rounding of dS to bf16, but P (dP - delta) is formed with
            # delta folded into the dP accumulator in one kernel and subtracted afterwards in the other
            assert (a.float() - c.float()).abs().max() <= 2e-2 * c.float().abs().max() + 1e-6
        else:
            assert torch.equal(a, c), name


def test_full_size_backward_paths_agree():
    """The benchmark's shape (1 x 32 heads x 8192 x 128, causal, bf16) is too large for the fp32
    oracle over all heads; what does not depend on size: dK and dV of the two backward routes are equal
    bit for bit and dQ from the stored dS agrees with dQ from the recomputed dS to rounding, gradients are
    linear in dO, and 2 heads are checked against the oracle."""
    from flagattention_amd import flash as flash_mod
    q = make((1, 32, 8192, 128), torch.bfloat16, "BHTD", 1.0, 1, grad=True)
    k = make((1, 32, 8192, 128), torch.bfloat16, "BHTD", 1.0, 2, grad=True)
    v = make((1, 32, 8192, 128), torch.bfloat16, "BHTD", 1.0, 3, grad=True)
    do = make((1, 32, 8192, 128), torch.bfloat16, "BHTD", 1.0, 4)
    stored = _grads(q, k, v, do, True)
    doubled = _grads(q, k, v, do * 2, True)   # exact in bf16: every product and sum scales by 2
    for a, b in zip(stored[1:], doubled[1:]):
        assert torch.equal(a * 2, b)
    saved = flash_mod.DS_WORKSPACE_LIMIT_MIB
    try:
        flash_mod.DS_WORKSPACE_LIMIT_MIB = 0
        recomputed = _grads(q, k, v, do, True)
    finally:
        flash_mod.DS_WORKSPACE_LIMIT_MIB = saved
    for name, a, b in zip(("o", "dq", "dk", "dv"), stored, recomputed):
        if name == "dq":
            assert (a.float() - b.float()).abs().max() <= 2e-2 * b.float().abs().max() + 1e-6
        else:
            assert torch.equal(a, b), name
    hs = slice(30, 32)
    qs, ks, vs = (t[:, hs].detach().requires_grad_() for t in (q, k, v))
    o_ref = oracle_flash(qs, ks, vs, True, upcast=True)
    g_ref = torch.autograd.grad(o_ref, (qs, ks, vs), do[:, hs])
    o_same = oracle_flash(qs, ks, vs, True, upcast=False)
    g_same = torch.autograd.grad(o_same, (qs, ks, vs), do[:, hs])
    check("o", stored[0][:, hs], o_same, o_ref)
    for name, h, s, r in zip(("dq", "dk", "dv"), stored[1:], g_same, g_ref):
        check(name, h[:, hs], s, r)


@pytest.mark.parametrize("B,Hq,Hk,M,N,D", [(2, 4, 4, 512, 612, 128), (2, 4, 2, 1024, 1034, 64), (1, 8, 2, 1300, 1300, 128),
                                            (2, 4, 4, 777, 300, 32)])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dropout_p", [0.2, 0.8])
def test_attention_dropout(B, Hq, Hk, M, N, D, causal, dtype, dropout_p):
    """Dropout through the public API: the returned (seed, offset) reproduce the mask in the oracle's
    restatement, and outputs and gradients then obey the 2x rule (covers the dS-kept backward at
    head size 128 with a large score matrix, and the recomputing one)."""
    from oracle import keep_mask
    q = make((B, Hq, M, D), dtype, "BHTD", 1.0, 1, grad=True)
    k = make((B, Hk, N, D), dtype, "BTHD", 1.0, 2, grad=True)
    v = make((B, Hk, N, D), dtype, "BTHD", 1.0, 3, grad=True)
    do = make((B, Hq, M, D), dtype, "BHTD", 1.0, 4)
    o, L, _, seed, offset = flag_attn.flash_attention(q, k, v, causal, dropout_p=dropout_p, return_log_normalizer=True,
                                                      return_seed_offset=True)
    grads = torch.autograd.grad(o, (q, k, v), do)
    assert isinstance(seed, int) and isinstance(offset, int)
    mask = keep_mask(B, Hq, M, N, dropout_p, seed, offset, device="cuda")
    assert abs((~mask).float().mean().item() - dropout_p) < 0.01
    ref = oracle_flash(q, k, v, causal, upcast=True, return_log_normalizer=True, dropout_p=dropout_p, dropout_mask=mask)
    same = oracle_flash(q, k, v, causal, upcast=False, return_log_normalizer=True, dropout_p=dropout_p, dropout_mask=mask)
    g_ref = torch.autograd.grad(ref[0], (q, k, v), do)
    g_same = torch.autograd.grad(same[0], (q, k, v), do)
    check("o", o, same[0], ref[0])
    check("L", L, same[1], ref[1])
    for name, h, s, r in zip(("dq", "dk", "dv"), grads, g_same, g_ref):
        check(name, h, s, r)


@pytest.mark.parametrize("B,H,M,N", [(2, 4, 512, 612), (2, 4, 1024, 1034), (2, 4, 4001, 4096), (1, 2, 8192, 8202)])
@pytest.mark.parametrize("p", [0.5, 0.8])
def test_recompute_mask(B, H, M, N, p):
    """flag_attn.testing.recompute_mask on the HIP kernel: drop rate within 1 % of p as the reference
    asserts (tests/flag_attn/test_dropout.py:18-30), and bit-exact with the oracle's Philox restatement
    on the first and the last rows of the tensor."""
    from oracle import keep_mask
    seed, offset = 123456789, 123456789123456789
    mask = flag_attn.testing.recompute_mask(B, H, M, N, p, seed, offset, torch.cuda.current_device())
    assert mask.dtype == torch.bool and mask.shape == (B, H, M, N)
    dropped = (~mask).float().mean().item()
    assert abs(dropped - p) < 0.01 * p
    rows = 3
    head = keep_mask(1, 1, rows, N, p, seed, offset, device="cuda")[0, 0]
    assert torch.equal(mask[0, 0, :rows], head)
    last = offset + ((B * H - 1) * M + (M - rows)) * N          # counter of element (B-1, H-1, M-rows, 0)
    tail = keep_mask(1, 1, rows, N, p, seed, last, device="cuda")[0, 0]
    assert torch.equal(mask[-1, -1, M - rows:], tail)
    assert flag_attn.testing.recompute_mask(1, 1, 4, 4, 0.0, seed, offset, "cuda").all()


def test_dropout_mask_matches_what_the_attention_kernels_drew():
    """The reference's own dropout test (tests/flag_attn/test_flash_attention.py:225-262): rebuild the
    mask from the returned (seed, offset) with recompute_mask and compare against the reference
    computation with that mask."""
    B, H, M, N, D, p = 2, 4, 512, 612, 64, 0.3
    q, k, v = (make((B, H, T, D), torch.float16, "BHTD", 1.0, s) for T, s in ((M, 1), (N, 2), (N, 3)))
    o, _, _, seed, offset = flag_attn.flash_attention(q, k, v, True, dropout_p=p, return_seed_offset=True)
    mask = flag_attn.testing.recompute_mask(B, H, M, N, p, seed, offset, q.device)
    ref = oracle_flash(q, k, v, True, upcast=True, dropout_p=p, dropout_mask=mask)
    same = oracle_flash(q, k, v, True, upcast=False, dropout_p=p, dropout_mask=mask)
    check("o", o, same, ref)


def test_dropout_advances_the_generator_and_is_reproducible():
    q, k, v = (make((2, 16, 256, 64), torch.float16, "BHTD", 1.0, s) for s in (1, 2, 3))
    torch.cuda.manual_seed(4321)
    o1, _, _, s1, off1 = flag_attn.flash_attention(q, k, v, dropout_p=0.5, return_seed_offset=True)
    o2, _, _, s2, off2 = flag_attn.flash_attention(q, k, v, dropout_p=0.5, return_seed_offset=True)
    assert s1 == s2 == 4321 and off2 == off1 + 2 * 16 * 256 * 256      # offset advanced by B * H * M * N
    assert not torch.equal(o1, o2)
    torch.cuda.manual_seed(4321)
    o3 = flag_attn.flash_attention(q, k, v, dropout_p=0.5)
    assert torch.equal(o1, o3)
    assert flag_attn.flash_attention(q, k, v, dropout_p=0.0, return_seed_offset=True)[3:] == (None, None)
    with pytest.raises(AssertionError):   # decode shapes take the split-KV path, which has no dropout
        flag_attn.flash_attention(q[:1, :2, :1], make((1, 2, 8192, 64), torch.float16, "BHTD", 1.0, 5),
                                  make((1, 2, 8192, 64), torch.float16, "BHTD", 1.0, 6), dropout_p=0.5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("M,N", [(1024, 1000), (2048, 1031), (1024, 2049)])
def test_ds_route_with_key_tail_and_very_negative_log_normalizer(M, N, causal, dtype):
    """Head size 128 at M * N >= 2^20 takes the route that keeps dS.  With a key count that is no
    multiple of 32 and log-normalizers below -11.5, exp(-L) of the lanes past the last key overflows
    fp16: those dS entries must be exact zeroes, or dQ becomes NaN.  dQ of the public backward is
    compared with the recomputing dQ kernel (same products, same rounding of dS) and with the oracle."""
    from flagattention_amd import _abi, _lib
    lib = _lib.get()
    g = torch.Generator(device="cuda").manual_seed(7)
    D = 128
    q = (torch.randn(1, 2, M, D, device="cuda", generator=g) * 0.1 + 1.0).to(dtype).requires_grad_()
    k = (torch.randn(1, 2, N, D, device="cuda", generator=g) * 0.1 - 2.0).to(dtype).requires_grad_()
    v = torch.randn(1, 2, N, D, device="cuda", generator=g).to(dtype).requires_grad_()
    do = torch.randn(1, 2, M, D, device="cuda", generator=g).to(dtype)
    o, lse, *_ = flag_attn.flash_attention(q, k, v, causal, return_log_normalizer=True)
    assert lse[torch.isfinite(lse)].max() < -11.5
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), do)
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all()
    delta = torch.empty_like(lse)
    _abi.fa_bwd_delta(lib, o.detach(), do, delta)
    dq_plain = torch.empty_like(dq)
    _abi.fa_bwd_dq(lib, q.detach(), k.detach(), v.detach(), do, lse, delta, dq_plain, causal, D ** -0.5)
    assert (dq.float() - dq_plain.float()).abs().max() <= 2e-2 * dq_plain.float().abs().max() + 1e-6
    ref = torch.autograd.grad(oracle_flash(q, k, v, causal, upcast=True), (q, k, v), do)
    same = torch.autograd.grad(oracle_flash(q, k, v, causal, upcast=False), (q, k, v), do)
    for name, h, s, r in zip(("dq", "dk", "dv"), (dq, dk, dv), same, ref):
        check(name, h, s, r)


WIDE_SHAPES = [
    # B, Hq, Hk, M, N  (head size 128)
    (2, 4, 4, 512, 612), (2, 4, 2, 512, 612), (2, 4, 4, 4096, 4000), (2, 4, 2, 4096, 4001), (1, 2, 1, 4001, 4096),
    (1, 8, 8, 2048, 2048), (1, 3, 1, 1000, 77), (2, 2, 2, 10006, 10), (1, 2, 2, 255, 8202), (1, 16, 4, 64, 64),
]


@pytest.mark.parametrize("scale", [1.0, 4.0])
@pytest.mark.parametrize("B,Hq,Hk,M,N", WIDE_SHAPES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
def test_attention_fwd_256_row_kernel(B, Hq, Hk, M, N, causal, order, dtype, scale):
    """The forward kernel with BLOCK_M = 256 (head size 128: 64 query rows per wavefront, slot-structured),
    called through the C entry point with the tile named explicitly, under the same 2x rule for o and the
    log-normalizer; rows without keys give o = 0 and -inf."""
    from flagattention_amd import _abi, _lib
    lib = _lib.get()
    D = 128
    q = make((B, Hq, M, D), dtype, order, scale, 1)
    k = make((B, Hk, N, D), dtype, order, scale, 2)
    v = make((B, Hk, N, D), dtype, order, scale, 3)
    o = torch.full_like(q, float("nan"))
    lse = torch.full((B, Hq, M), float("nan"), device="cuda")
    _abi.fa_fwd(lib, q, k, v, o, lse, causal, D ** -0.5, block_m=256)
    ref = oracle_flash(q, k, v, causal, upcast=True, return_log_normalizer=True)
    same = oracle_flash(q, k, v, causal, upcast=False, return_log_normalizer=True)
    check("o", o, same[0], ref[0])
    check("log_normalizer", lse, same[1], ref[1])
    if causal and M > N:
        assert torch.all(o[:, :, : M - N] == 0) and torch.all(torch.isinf(lse[:, :, : M - N]))


def test_forward_tile_hook_selects_the_kernel(monkeypatch):
    """``flash.get_fwd_config`` chooses between the two compiled forward kernels (examples/use_cutom_config_func.py
    of the reference): both answers give results within rounding of each other, and a tile that does not
    apply to the launch falls back with a warning."""
    import warnings
    from flag_attn import flash
    q, k, v = (make((1, 4, 1024, 128), torch.bfloat16, "BHTD", 1.0, s) for s in (1, 2, 3))
    outs = {}
    for bm in (128, 256):
        monkeypatch.setattr(flash, "get_fwd_config", lambda B, H, M, N, D, causal, bm=bm: (bm, 64, 2, 4))
        outs[bm] = flag_attn.flash_attention(q, k, v, causal=True, return_log_normalizer=True)
    assert (outs[128][0].float() - outs[256][0].float()).abs().max() < 2e-2
    assert (outs[128][1] - outs[256][1]).abs().max() < 1e-4
    assert not torch.equal(outs[128][0], outs[256][0])   # two different kernels ran (summation order differs)
    q64, k64, v64 = (make((1, 4, 1024, 64), torch.bfloat16, "BHTD", 1.0, s) for s in (1, 2, 3))
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        o = flag_attn.flash_attention(q64, k64, v64, causal=True)
    check("o", o, oracle_flash(q64, k64, v64, True, upcast=False), oracle_flash(q64, k64, v64, True, upcast=True))
    assert len(seen) <= 1
