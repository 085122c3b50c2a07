"""Host-side rules of the operator wrappers: split-count rule, paged partitioning, layout checks."""
import math

import pytest
import torch

from flagattention_amd import _abi
from flagattention_amd.paged import choose_launch, _next_pow2
from flagattention_amd.split_kv import choose_num_splits, num_splits_heuristic, _split_size


def brute_force_splits(B, H, M, N, bm, bn, cus, max_splits):
    """The split rule written as a direct search (follows src/flag_attn/split_kv.py:234-262)."""
    blocks = B * H * math.ceil(M / bm)
    if blocks >= 0.8 * cus:
        return 1
    nb = math.ceil(N / bn)
    cand = []
    for s in range(1, min(cus, nb, max_splits) + 1):
        per = math.ceil(nb / s)
        if s == 1 or per * s - nb < per:
            w = blocks * s / cus
            cand.append((s, w / math.ceil(w)))
    top = max(e for _, e in cand)
    return next(s for s, e in cand if e >= 0.85 * top)


@pytest.mark.parametrize("B,H,M,N", [(4, 32, 1, 32768), (2, 4, 1, 612), (1, 2, 4, 8202), (2, 4, 2, 4000),
                                     (1, 32, 1024, 8192), (1, 1, 1, 100), (8, 8, 1, 100000)])
@pytest.mark.parametrize("cus", [256, 108])
def test_split_rule(B, H, M, N, cus):
    assert num_splits_heuristic(B, H, M, N, 16, 128, cus, 128) == brute_force_splits(B, H, M, N, 16, 128, cus, 128)


def test_known_split_counts():
    # decode of 4 x 32 heads over 32768 keys on 256 compute units: 128 workgroups -> two splits
    assert num_splits_heuristic(4, 32, 1, 32768, 16, 128, 256, 128) == 2
    # a grid that already fills the device is never split
    assert num_splits_heuristic(1, 32, 1024, 8192, 16, 128, 256, 128) == 1


@pytest.mark.parametrize("N,S", [(32768, 2), (612, 3), (8202, 5), (100, 1)])
def test_split_size_covers_keys_in_128_key_units(N, S):
    size = _split_size(N, S)
    assert size % 128 == 0 and size * S >= N and size * (S - 1) < N + 128 * S


def test_split_count_actually_launched():
    # (B, H, Hk, M, N, compute units, reference count)
    assert choose_num_splits(1, 32, 8, 1, 32768, 256, 8) == 64       # 8 workgroups per split -> cap N / 512
    assert choose_num_splits(64, 32, 8, 1, 4096, 256, 1) == 1        # 512 workgroups: one resident wave already
    assert choose_num_splits(4, 32, 8, 1, 32768, 256, 2) == 16       # 32 workgroups per split -> 512
    assert choose_num_splits(256, 32, 8, 1, 4096, 256, 1) == 1       # the batch alone fills the device
    assert choose_num_splits(1, 8, 8, 4, 700, 256, 3) == 1           # pieces would be shorter than 512 keys
    for args in [(1, 32, 8, 1, 32768, 256, 8), (2, 4, 2, 2, 4000, 256, 5), (1, 2, 1, 4, 8202, 256, 7)]:
        s = choose_num_splits(*args)
        n_units = -(-args[4] // 128)
        assert 1 <= s <= 128 and (s == 1 or (-(-n_units // s)) * (s - 1) < n_units)   # no empty last piece


def test_dkdv_heads_per_slice():
    from flagattention_amd.flash import dkdv_heads_per_slice
    # (B, H, group, N, compute units)
    assert dkdv_heads_per_slice(1, 32, 1, 8192, 256) == 1
    assert dkdv_heads_per_slice(1, 32, 4, 8192, 256) == 4     # 64 key blocks x 8 kv heads = 512 workgroups
    assert dkdv_heads_per_slice(1, 32, 8, 8192, 256) == 4     # whole groups would leave 256 workgroups
    assert dkdv_heads_per_slice(1, 8, 8, 1024, 256) == 1      # tiny launch: one slice per query head
    for args in [(2, 40, 5, 3000, 256), (1, 6, 6, 70000, 304), (3, 16, 2, 100, 256)]:
        c = dkdv_heads_per_slice(*args)
        assert 1 <= c <= args[2] and args[2] % c == 0


def test_paged_launch_choice():
    # (num_seqs, kv heads, group, head size, max context, compute units)
    assert choose_launch(64, 8, 4, 128, 8192, 256) == ("balanced", 512)
    assert choose_launch(1, 8, 4, 128, 32768, 256) == ("balanced", 512)
    assert choose_launch(32, 16, 1, 256, 8192, 256) == ("balanced", 256)   # one workgroup per CU at 256
    assert choose_launch(2048, 8, 4, 128, 1024, 256) == ("single", 0)      # many short pairs
    assert choose_launch(2048, 8, 4, 128, 4096, 256) == ("balanced", 512)  # long contexts: keep balancing
    assert choose_launch(100, 1, 40, 64, 1024, 256) == ("balanced", 512)   # 3 row blocks per kv head
    assert _next_pow2(1) == 1 and _next_pow2(5) == 8 and _next_pow2(256) == 256


def test_kernel_ready_copies_only_when_needed():
    a = torch.zeros(2, 3, 8, 16, dtype=torch.float16)
    assert _abi.kernel_ready(a) is a
    t = torch.zeros(2, 8, 3, 16, dtype=torch.float16).transpose(1, 2)  # BTHD view: still fine
    assert _abi.kernel_ready(t) is t
    inner = torch.zeros(2, 3, 16, 8, dtype=torch.float16).transpose(2, 3)  # inner stride != 1
    assert _abi.kernel_ready(inner).stride(-1) == 1
    odd = torch.zeros(2, 3, 8, 20, dtype=torch.float16)[..., :16]  # row stride 20: not a multiple of 8
    assert _abi.kernel_ready(odd).stride(2) == 16
    shifted = torch.zeros(2 * 3 * 8 * 16 + 4, dtype=torch.float16)[4:].view(2, 3, 8, 16)  # 8-byte aligned only
    assert _abi.kernel_ready(shifted).data_ptr() % 16 == 0


def test_dtype_codes():
    assert _abi.dtype_code(torch.zeros(1, dtype=torch.float16)) == 0
    assert _abi.dtype_code(torch.zeros(1, dtype=torch.bfloat16)) == 1
    with pytest.raises(AssertionError):
        _abi.dtype_code(torch.zeros(1, dtype=torch.float32))


def test_reference_package_name_resolves_to_this_implementation():
    """``import flag_attn`` and its submodules (the names the reference's callers use,
    src/flag_attn/__init__.py:9-14) resolve to this package; nothing here needs a GPU."""
    import flag_attn
    import flag_attn.flash
    import flag_attn.testing
    from flag_attn.dropout import philox_cuda_seed_offset
    from flag_attn.testing import recompute_mask
    import flagattention_amd
    assert flag_attn.flash_attention is flagattention_amd.flash_attention
    assert flag_attn.piecewise_attention is flagattention_amd.piecewise_attention
    assert flag_attn.paged_attention is flagattention_amd.paged_attention
    assert flag_attn.flash_attention_split_kv is flagattention_amd.flash_attention_split_kv
    assert flag_attn.flash is flagattention_amd.flash and flag_attn.testing is flagattention_amd.testing
    assert callable(philox_cuda_seed_offset) and callable(recompute_mask)
    assert callable(flag_attn.flash.get_fwd_config) and callable(flag_attn.flash.get_bwd_config)


def test_config_hook_resolution():
    """The tile hooks (flash.py:290,493 of the reference) are called with the launch's shape; a compiled
    tile is taken, anything else falls back to the default with one warning per distinct answer, and a
    malformed answer is an assertion like the reference's shape checks."""
    import warnings
    from flagattention_amd import _config
    compiled = ((128, 64), (256, 64))
    seen_args = []

    def hook(*a):
        seen_args.append(a)
        return (256, 64, 1, 4)
    assert _config.resolve(hook, compiled, "t1", (1, 2, 3, 4, 128, True)) == (256, 64)
    assert seen_args == [(1, 2, 3, 4, 128, True)]
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        assert _config.resolve(lambda *a: (32, 32, 1, 4), compiled, "t2", (1,) * 6) == (128, 64)
        assert _config.resolve(lambda *a: (32, 32, 1, 4), compiled, "t2", (1,) * 6) == (128, 64)
        assert _config.resolve(lambda *a: (16, 32, 1, 4), compiled, "t2", (1,) * 6) == (128, 64)
    assert len(w) == 2 and all(issubclass(x.category, RuntimeWarning) for x in w)
    with pytest.raises(AssertionError):
        _config.resolve(lambda *a: (128, 64), compiled, "t3", (1,) * 6)
    with pytest.raises(AssertionError):
        _config.resolve(lambda *a: (0, 64, 1, 4), compiled, "t3", (1,) * 6)


def test_default_hooks_name_compiled_tiles():
    from flagattention_amd import flash, piecewise
    for mod in (flash, piecewise):
        assert mod.get_fwd_config(1, 1, 4096, 4096, 128, True)[:2] in mod.FWD_TILES
        assert mod.get_bwd_config(1, 1, 4096, 4096, 128, True)[:2] in mod.BWD_TILES


class _SizesOnly:
    """Stands in for the kernel library where only the workspace size is asked for."""

    @staticmethod
    def fa_bwd_ds_workspace_mib(B, H, M, N):
        return (B * H * -(-M // 128) * -(-N // 128) * 32768 + (1 << 20) - 1) >> 20


def test_ds_workspace_policy(monkeypatch):
    from flagattention_amd import flash
    lib = _SizesOnly()
    monkeypatch.setattr(flash, "DS_WORKSPACE_LIMIT_MIB", 4096)
    # the headline shape needs 32 x 128 MiB and is held whole; twice the batch goes in slices
    assert flash.ds_heads_per_launch(lib, 1, 32, 1, 8192, 8192, 128) == 32
    assert flash.ds_heads_per_launch(lib, 2, 32, 1, 8192, 8192, 128) == 32
    # slices are whole groups of query heads
    monkeypatch.setattr(flash, "DS_WORKSPACE_LIMIT_MIB", 128 * 7)
    assert flash.ds_heads_per_launch(lib, 1, 32, 4, 8192, 8192, 128) == 4
    # small matrices, small heads and a zero limit recompute dS
    assert flash.ds_heads_per_launch(lib, 1, 32, 1, 512, 512, 128) == 0
    assert flash.ds_heads_per_launch(lib, 1, 32, 1, 8192, 8192, 64) == 0
    monkeypatch.setattr(flash, "DS_WORKSPACE_LIMIT_MIB", 0)
    assert flash.ds_heads_per_launch(lib, 1, 32, 1, 8192, 8192, 128) == 0


def test_ds_workspace_allocation_failure_is_reported_as_none(monkeypatch):
    from flagattention_amd import flash

    def no_memory(*args, **kwargs):
        raise torch.OutOfMemoryError("out of memory")

    monkeypatch.setattr(flash.torch, "empty", no_memory)
    assert flash._ds_workspace(_SizesOnly(), "cpu", 1, 32, 8192, 8192) is None


def test_split_and_total_hooks_are_live(monkeypatch):
    """Replacing ``split_kv.get_fwd_config`` / ``total.get_fwd_config`` takes effect at the next call
    (the reference reads them at ``split_kv.py:288``, ``flash.py:59`` and ``total.py:29``)."""
    import warnings
    from flagattention_amd import _config, split_kv, total
    assert split_kv.split_units(1, 8, 1, 4096, 128, False) == (16, 128)
    calls = []

    def mine(B, H, M, N, D, causal):
        calls.append((B, H, M, N, D, causal))
        return (32, 64, 2, 8)

    monkeypatch.setattr(split_kv, "get_fwd_config", mine)
    monkeypatch.setattr(_config, "_warned", set())
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        assert split_kv.split_units(1, 8, 1, 4096, 128, False) == (16, 128)   # not compiled: said once, default used
        assert split_kv.split_units(1, 8, 1, 4096, 128, False) == (16, 128)
    assert calls == [(1, 8, 1, 4096, 128, False)] * 2
    assert len([w for w in caught if "BLOCK_M=32" in str(w.message)]) == 1
    # the default hooks name the compiled tiles
    assert tuple(total.get_fwd_config(1, 8, 128, 128, 64, True)[:2]) in total.FWD_TILES


def test_bench_counts_the_flops_of_the_quoted_workloads():
    """bench.py's FLOP counts against the figures of the workload list: forward 2 products, backward 5,
    each 2 * B * H * pairs * D with `pairs` the unmasked (query, key) pairs of the bottom-right aligned mask."""
    import bench
    assert bench.causal_pairs(8192, 8192) == 8192 * 8193 // 2
    assert bench.causal_pairs(4, 6) == 3 + 4 + 5 + 6            # every query sees the 2 extra keys
    assert bench.causal_pairs(6, 4) == 0 + 0 + 1 + 2 + 3 + 4    # the first rows see nothing
    assert bench.causal_pairs(1024, 8192) == 1024 * 7168 + 1024 * 1025 // 2
    c3 = bench.WORKLOADS["c3"]
    x = 2.0 * c3["B"] * c3["H"] * bench.causal_pairs(c3["T"], c3["T"]) * c3["D"]
    assert abs(7 * x / 1e9 - 1924.4) < 0.3          # 549.8 forward + 1374.5 backward
    c2 = bench.WORKLOADS["c2"]
    x2 = 2.0 * c2["B"] * c2["H"] * bench.causal_pairs(c2["T"], c2["T"]) * c2["D"]
    assert abs(7 * x2 / 1e9 - 240.6) < 0.2
    assert bench.PEAK_BF16_TFLOPS == 2500.0 and bench.PEAK_HBM_GBS == 8000.0


@pytest.mark.parametrize("B,H,M,N", [(0, 2, 5, 7), (1, 2, 0, 7), (1, 2, 5, 0), (0, 2, 0, 0)])
def test_empty_axes_launch_nothing(monkeypatch, B, H, M, N):
    """An empty batch, query or key axis: zero output, -inf log-normalizer, zero total attention and zero
    gradients of the inputs' shapes, without touching the kernel library.  (The reference's split rule divides
    by zero for an empty batch or query axis, and its kernels return NaN for an empty key axis.)"""
    import flag_attn
    from flagattention_amd import _lib

    def no_library():
        raise AssertionError("the kernel library must not be needed")

    monkeypatch.setattr(_lib, "get", no_library)
    D = 32
    q = torch.randn(B, H, M, D, dtype=torch.float16, requires_grad=True)
    k = torch.randn(B, 1, N, D, dtype=torch.float16, requires_grad=True)
    v = torch.randn(B, 1, N, D, dtype=torch.float16, requires_grad=True)
    o, L, tot, seed, offset = flag_attn.flash_attention(q, k, v, causal=True, return_log_normalizer=True,
                                                        return_total_attention=True)
    assert o.shape == q.shape and o.dtype == q.dtype and not o.any()
    assert L.shape == (B, H, M) and bool((L == -math.inf).all()) and tot.shape == (B, H, N) and not tot.any()
    assert seed is None and offset is None
    grads = torch.autograd.grad(o, (q, k, v), torch.ones_like(o))
    assert [g.shape for g in grads] == [q.shape, k.shape, v.shape] and not any(g.any() for g in grads)
    assert flag_attn.flash_attention(q, k, v).shape == q.shape
    assert flag_attn.flash_attention_split_kv(q.detach(), k.detach(), v.detach()).shape == q.shape

    k1 = torch.randn(B, H, N, D, dtype=torch.float16, requires_grad=True)
    ins = [q, k1, q.detach().clone().requires_grad_(), k1.detach().clone().requires_grad_(), k1.detach().clone().requires_grad_()]
    o = flag_attn.piecewise_attention(*ins, 3, causal=True)
    assert o.shape == q.shape and not o.any()
    grads = torch.autograd.grad(o, ins, torch.ones_like(o))
    assert [g.shape for g in grads] == [t.shape for t in ins] and not any(g.any() for g in grads)

    with pytest.raises(AssertionError):       # the argument checks still apply
        flag_attn.flash_attention(q, k, torch.randn(B, 1, N, 2 * D, dtype=torch.float16))


def test_paged_attention_without_sequences_launches_nothing(monkeypatch):
    import flag_attn
    from flagattention_amd import _lib
    monkeypatch.setattr(_lib, "get", lambda: (_ for _ in ()).throw(AssertionError("the kernel library must not be needed")))
    q = torch.empty(0, 8, 64, dtype=torch.float16)
    cache = torch.empty(4, 2, 16, 64, dtype=torch.float16)
    out = flag_attn.paged_attention(q, cache, cache, torch.empty(0, dtype=torch.int32),
                                    torch.empty(0, 4, dtype=torch.int32), 0.125, 0)
    assert out.shape == q.shape and out.dtype == q.dtype


def test_total_attention_with_empty_axes_launches_nothing(monkeypatch):
    """The standalone total_attention treats an empty batch, query or key axis like flash_attention does."""
    import flag_attn
    from flagattention_amd import _lib
    monkeypatch.setattr(_lib, "get", lambda: (_ for _ in ()).throw(AssertionError("the kernel library must not be needed")))
    for B, H, M, N in [(0, 2, 5, 7), (1, 2, 0, 7), (1, 2, 5, 0)]:
        q = torch.randn(B, H, M, 32, dtype=torch.float16)
        k = torch.randn(B, 1, N, 32, dtype=torch.float16)
        tot = flag_attn.total_attention(q, k, torch.zeros(B, H, M), causal=True)
        assert tot.shape == (B, H, N) and tot.dtype == torch.float32 and not tot.any()


class _RecordingLibrary:
    """Stands in for the kernel library: every entry point returns 0 and is recorded with its arguments."""

    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        if name == "fa_num_cus":
            return lambda: 256
        if name == "paged_attn_balanced_workspace":
            return lambda wgs, d: 1024

        def call(*args):
            self.calls.append((name, args))
            return 0
        return call


def _with_recording_library(monkeypatch):
    import contextlib
    from flagattention_amd import _lib, flash, paged
    lib = _RecordingLibrary()
    monkeypatch.setattr(_lib, "get", lambda: lib)
    monkeypatch.setattr(torch.cuda, "device", lambda device: contextlib.nullcontext())
    monkeypatch.setattr(flash, "_NUM_CUS", {})
    monkeypatch.setattr(paged, "_NUM_CUS", {})
    return lib


def test_default_forward_hook_leaves_the_tile_to_the_library(monkeypatch, recwarn):
    """With the module's own get_fwd_config nobody chose a tile: fa_fwd gets block_m = 0, so that a large head-128
    launch with dropout (which the hook is not told about) warns about nothing, and so does a stride the
    256-row kernel cannot address; an override that asks for 256 rows where they do not apply is told once."""
    import flag_attn
    from flagattention_amd import flash, _config
    lib = _with_recording_library(monkeypatch)
    monkeypatch.setattr(flash, "philox_cuda_seed_offset", lambda n, device: (1, 2))
    monkeypatch.setattr(_config, "_warned", set())
    q = torch.empty(1, 32, 8192, 128, dtype=torch.bfloat16)
    assert flash.get_fwd_config(1, 32, 8192, 8192, 128, True)[0] == 256        # the default's answer for this launch
    flag_attn.flash_attention(q, q, q, causal=True, dropout_p=0.1)
    name, args = lib.calls[-1]
    assert name == "fa_fwd" and args[-2] == 0
    assert not [w for w in recwarn.list if issubclass(w.category, RuntimeWarning)]
    monkeypatch.setattr(flash, "get_fwd_config", lambda *a: (256, 64, 5, 4))
    with pytest.warns(RuntimeWarning, match="without dropout"):
        flag_attn.flash_attention(q, q, q, causal=True, dropout_p=0.1)
    assert lib.calls[-1][1][-2] == 128
    with pytest.warns(RuntimeWarning, match="sm_scale > 0"):
        flag_attn.flash_attention(q, q, q, causal=True, sm_scale=-1.0)
    assert lib.calls[-1][1][-2] == 128
    flag_attn.flash_attention(q, q, q, causal=True)
    assert lib.calls[-1][1][-2] == 256


def test_paged_attention_accepts_any_integer_context_lens_and_keeps_the_query_layout(monkeypatch):
    """paged.py:16 of the reference returns empty_like(query) and takes context_lens of any integer type."""
    import flag_attn
    lib = _with_recording_library(monkeypatch)
    q = torch.empty(8, 4, 64, dtype=torch.float16).transpose(0, 1)          # (4, 8, 64) view with strides (64, 256, 1)
    cache = torch.empty(6, 2, 16, 64, dtype=torch.float16)
    table = torch.zeros(4, 3, dtype=torch.int32)
    out = flag_attn.paged_attention(q, cache, cache, torch.tensor([3, 40, 0, 17], dtype=torch.int64), table, 0.125, 40)
    assert out.shape == q.shape and out.stride() == q.stride()
    name, args = lib.calls[0]
    assert name == "paged_attn_balanced" and (args[2], args[3]) == (q.stride(0), q.stride(1))
    with pytest.raises(AssertionError, match="integers"):
        flag_attn.paged_attention(q, cache, cache, torch.tensor([3., 40., 0., 17.]), table, 0.125, 40)


def test_key_pieces_of_a_dense_forward_that_would_leave_compute_units_idle():
    from flagattention_amd.flash import wide_key_splits
    # (B, H, M, N, D, compute units)
    assert wide_key_splits(1, 32, 1024, 8192, 128, 256) == 2     # 128 workgroups of 256 rows on 256 units
    assert wide_key_splits(1, 32, 8192, 8192, 128, 256) == 1     # 1024 workgroups: nothing to gain
    assert wide_key_splits(1, 32, 1024, 8192, 64, 256) == 1      # the 256-row kernel is built for head size 128
    assert wide_key_splits(1, 8, 1024, 8192, 128, 256) == 8      # 32 workgroups -> 8 pieces of 1024 keys
    assert wide_key_splits(1, 8, 1024, 4096, 128, 256) == 1      # pieces of 1024 keys would fill half the device only
    assert wide_key_splits(1, 48, 1024, 8192, 128, 256) == 1     # 192 workgroups: a second piece would start a second round
    assert wide_key_splits(4, 32, 100, 8192, 128, 256) == 1      # fewer rows than one 256-row tile
