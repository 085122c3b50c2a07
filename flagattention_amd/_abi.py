"""Marshalling between torch tensors and the C entry points of ``include/flagattn.h``.

Every function takes the bound library as its first argument and only uses ``data_ptr()``,
``stride()`` and ``dtype`` of the tensors it is given; outputs and workspaces are allocated by the
callers (torch's caching allocator owns all device memory, as in the reference).
"""
import ctypes

import torch

from ._lib import View4

F16, BF16 = 0, 1


class KernelError(RuntimeError):
    pass


def dtype_code(t):
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.bfloat16:
        return BF16
    raise AssertionError(f"only float16 and bfloat16 are supported, got {t.dtype}")


def stream_of(t):
    if t.is_cuda:
        return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)
    return ctypes.c_void_p(0)


def view4(t):
    (n0, n1, n2, _), (s0, s1, s2, s3) = t.shape, t.stride()      # raises unless t has four dimensions
    assert s3 == 1
    # the stride of a dimension of extent 1 is never used; torch leaves arbitrary values there
    return ctypes.byref(View4(t.data_ptr(), s0 if n0 > 1 else 0, s1 if n1 > 1 else 0, s2 if n2 > 1 else 0))


def ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def check(code, what):
    if code == 0:
        return
    if code == -1:
        raise AssertionError(f"{what}: argument rejected by the kernel library")
    if code == -2:
        raise AssertionError(f"{what}: configuration not supported by the kernel library")
    if code == -3:
        raise AssertionError(f"{what}: the launch needs more scratch memory than the library's static device "
                             "array holds (FA_STATIC_SCRATCH_BYTES); use the entry point that takes a workspace")
    raise KernelError(f"{what}: HIP error {code}")


def is_kernel_ready(t):
    strides = t.stride()
    if strides[-1] != 1 or t.data_ptr() % 16:
        return False
    for extent, stride in zip(t.shape[:-1], strides[:-1]):
        if extent > 1 and stride % 8:
            return False
    return True


def kernel_ready(t):
    """The kernels move 16 bytes at a time: unit inner stride, 16-byte aligned base, strides that are
    multiples of 8 elements.  Anything else is copied (the reference copies when the inner stride is
    not 1, src/flag_attn/flash.py:14-17)."""
    return t if is_kernel_ready(t) else t.clone(memory_format=torch.contiguous_format)


NO_DROPOUT = (0.0, 0, 0)  # (dropout_p, seed, offset)


def _u64(x):
    return int(x) & 0xFFFFFFFFFFFFFFFF


def fa_fwd(lib, q, k, v, o, lse, causal, sm_scale, dropout=NO_DROPOUT, block_m=0):
    """block_m: query rows per workgroup (128 or 256), 0 = the library's choice."""
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_fwd(dtype_code(q), view4(q), view4(k), view4(v), view4(o), ptr(lse),
                     B, H, Hk, M, N, D, int(causal), float(sm_scale), float(dropout[0]), _u64(dropout[1]),
                     _u64(dropout[2]), int(block_m), stream_of(q)), "fa_fwd")


def pw_fwd(lib, q1, k1, q2, k2, v, o, lse, w, causal, sm_scale):
    B, H, M, D = q1.shape
    N = k1.shape[2]
    check(lib.pw_fwd(dtype_code(q1), view4(q1), view4(k1), view4(q2), view4(k2), view4(v), view4(o),
                     ptr(lse), B, H, M, N, D, int(w), int(causal), float(sm_scale), stream_of(q1)),
          "pw_fwd")


def fa_bwd_delta(lib, o, do, delta):
    B, H, M, D = o.shape
    check(lib.fa_bwd_delta(dtype_code(o), view4(o), view4(do), ptr(delta), B, H, M, D, stream_of(o)),
          "fa_bwd_delta")


def _heads_per_slice(q, dk):
    """dk / dv hold one slice per this many query heads (summed by the kernel)."""
    H, slices = q.shape[1], dk.shape[1]
    assert H % slices == 0
    return H // slices


def fa_bwd_dkdv(lib, q, k, v, do, lse, delta, dk, dv, causal, sm_scale, dropout=NO_DROPOUT):
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_bwd_dkdv(dtype_code(q), view4(q), view4(k), view4(v), view4(do), ptr(lse), ptr(delta),
                          view4(dk), view4(dv), _heads_per_slice(q, dk), B, H, Hk, M, N, D, int(causal),
                          float(sm_scale), float(dropout[0]), _u64(dropout[1]), _u64(dropout[2]),
                          stream_of(q)), "fa_bwd_dkdv")


def fa_bwd_dq(lib, q, k, v, do, lse, delta, dq, causal, sm_scale, dropout=NO_DROPOUT):
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_bwd_dq(dtype_code(q), view4(q), view4(k), view4(v), view4(do), ptr(lse), ptr(delta),
                        view4(dq), B, H, Hk, M, N, D, int(causal), float(sm_scale), float(dropout[0]),
                        _u64(dropout[1]), _u64(dropout[2]), stream_of(q)), "fa_bwd_dq")


def fa_bwd_dkdv_ds(lib, q, k, v, do, lse, delta, dk, dv, ds, causal, sm_scale, dropout=NO_DROPOUT):
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_bwd_dkdv_ds(dtype_code(q), view4(q), view4(k), view4(v), view4(do), ptr(lse), ptr(delta),
                             view4(dk), view4(dv), _heads_per_slice(q, dk), ptr(ds),
                             ds.numel() * ds.element_size(), B, H, Hk, M, N, D, int(causal),
                             float(sm_scale), float(dropout[0]), _u64(dropout[1]), _u64(dropout[2]),
                             stream_of(q)), "fa_bwd_dkdv_ds")


def fa_bwd_dq_from_ds(lib, k, ds, dq, causal, sm_scale):
    B, H, M, D = dq.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_bwd_dq_from_ds(dtype_code(dq), view4(k), ptr(ds), ds.numel() * ds.element_size(),
                                view4(dq), B, H, Hk, M, N, D, int(causal), float(sm_scale),
                                stream_of(dq)), "fa_bwd_dq_from_ds")


def pw_bwd_dkdv(lib, q1, k1, q2, k2, v, do, lse, delta, dk1, dk2, dv, w, causal, sm_scale):
    B, H, M, D = q1.shape
    N = k1.shape[2]
    check(lib.pw_bwd_dkdv(dtype_code(q1), view4(q1), view4(k1), view4(q2), view4(k2), view4(v), view4(do),
                          ptr(lse), ptr(delta), view4(dk1), view4(dk2), view4(dv), B, H, M, N, D,
                          int(w), int(causal), float(sm_scale), stream_of(q1)), "pw_bwd_dkdv")


def pw_bwd_dq(lib, q1, k1, q2, k2, v, do, lse, delta, dq1, dq2, w, causal, sm_scale):
    B, H, M, D = q1.shape
    N = k1.shape[2]
    check(lib.pw_bwd_dq(dtype_code(q1), view4(q1), view4(k1), view4(q2), view4(k2), view4(v), view4(do),
                        ptr(lse), ptr(delta), view4(dq1), view4(dq2), B, H, M, N, D, int(w),
                        int(causal), float(sm_scale), stream_of(q1)), "pw_bwd_dq")


def pw_bwd_dkdv_ds(lib, q1, k1, q2, k2, v, do, lse, delta, dk1, dk2, dv, ds, w, causal, sm_scale):
    B, H, M, D = q1.shape
    N = k1.shape[2]
    check(lib.pw_bwd_dkdv_ds(dtype_code(q1), view4(q1), view4(k1), view4(q2), view4(k2), view4(v), view4(do),
                             ptr(lse), ptr(delta), view4(dk1), view4(dk2), view4(dv), ptr(ds),
                             ds.numel() * ds.element_size(), B, H, M, N, D, int(w), int(causal),
                             float(sm_scale), stream_of(q1)), "pw_bwd_dkdv_ds")


def pw_bwd_dq_from_ds(lib, k1, k2, ds, dq1, dq2, w, causal, sm_scale):
    B, H, M, D = dq1.shape
    N = k1.shape[2]
    check(lib.pw_bwd_dq_from_ds(dtype_code(dq1), view4(k1), view4(k2), ptr(ds), ds.numel() * ds.element_size(),
                                view4(dq1), view4(dq2), B, H, M, N, D, int(w), int(causal),
                                float(sm_scale), stream_of(dq1)), "pw_bwd_dq_from_ds")


def fa_dropout_mask(lib, mask, dropout_p, seed, offset):
    B, H, M, N = mask.shape
    assert mask.is_contiguous() and mask.element_size() == 1
    check(lib.fa_dropout_mask(ptr(mask), B, H, M, N, float(dropout_p), _u64(seed), _u64(offset),
                              stream_of(mask)), "fa_dropout_mask")


def fa_total_attn(lib, q, k, lse, total, causal, sm_scale):
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_total_attn(dtype_code(q), view4(q), view4(k), ptr(lse), ptr(total), B, H, Hk, M, N, D,
                            int(causal), float(sm_scale), stream_of(q)), "fa_total_attn")


def fa_splitkv_fwd(lib, q, k, v, part_o, part_lse, causal, sm_scale, num_splits, split_size):
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_splitkv_fwd(dtype_code(q), view4(q), view4(k), view4(v), ptr(part_o), ptr(part_lse),
                             B, H, Hk, M, N, D, int(causal), float(sm_scale), int(num_splits),
                             int(split_size), stream_of(q)), "fa_splitkv_fwd")


def fa_splitkv_combine(lib, part_o, part_lse, o, lse, num_splits):
    B, H, M, D = o.shape
    check(lib.fa_splitkv_combine(dtype_code(o), ptr(part_o), ptr(part_lse), view4(o), ptr(lse),
                                 B, H, M, D, int(num_splits), stream_of(o)), "fa_splitkv_combine")


def paged_attn(lib, out, query, key_cache, value_cache, context_lens, block_tables, scale,
               partition_size, num_parts, tmp_out, max_logits, exp_sums):
    num_seqs, Hq, D = query.shape
    _, Hkv, block_size, _ = key_cache.shape
    assert block_tables.dtype in (torch.int32, torch.int64)
    check(lib.paged_attn(dtype_code(query), ptr(out), out.stride(0), out.stride(1),
                         ptr(query), query.stride(0), query.stride(1),
                         ptr(key_cache), ptr(value_cache),
                         key_cache.stride(0), key_cache.stride(1), key_cache.stride(2),
                         ptr(context_lens), ptr(block_tables), int(block_tables.dtype == torch.int64),
                         block_tables.stride(0), float(scale), num_seqs, Hq, Hkv, D, block_size,
                         int(partition_size), int(num_parts), ptr(tmp_out), ptr(max_logits),
                         ptr(exp_sums), stream_of(query)), "paged_attn")


def paged_attn_balanced(lib, out, query, key_cache, value_cache, context_lens, block_tables, scale,
                        workspace, num_workgroups):
    num_seqs, Hq, D = query.shape
    _, Hkv, block_size, _ = key_cache.shape
    assert block_tables.dtype in (torch.int32, torch.int64)
    check(lib.paged_attn_balanced(dtype_code(query), ptr(out), out.stride(0), out.stride(1),
                                  ptr(query), query.stride(0), query.stride(1),
                                  ptr(key_cache), ptr(value_cache),
                                  key_cache.stride(0), key_cache.stride(1), key_cache.stride(2),
                                  ptr(context_lens), ptr(block_tables),
                                  int(block_tables.dtype == torch.int64), block_tables.stride(0),
                                  float(scale), num_seqs, Hq, Hkv, D, block_size, ptr(workspace),
                                  workspace.numel() * workspace.element_size(), int(num_workgroups),
                                  stream_of(query)), "paged_attn_balanced")


def paged_attn_balanced_static(lib, out, query, key_cache, value_cache, context_lens, block_tables, scale,
                               num_workgroups):
    """paged_attn_balanced on the library's static device scratch: allocates nothing."""
    num_seqs, Hq, D = query.shape
    _, Hkv, block_size, _ = key_cache.shape
    assert block_tables.dtype in (torch.int32, torch.int64)
    check(lib.paged_attn_balanced_static(dtype_code(query), ptr(out), out.stride(0), out.stride(1),
                                         ptr(query), query.stride(0), query.stride(1),
                                         ptr(key_cache), ptr(value_cache),
                                         key_cache.stride(0), key_cache.stride(1), key_cache.stride(2),
                                         ptr(context_lens), ptr(block_tables),
                                         int(block_tables.dtype == torch.int64), block_tables.stride(0),
                                         float(scale), num_seqs, Hq, Hkv, D, block_size, int(num_workgroups),
                                         stream_of(query)), "paged_attn_balanced_static")


def paged_reduce(lib, out, tmp_out, max_logits, exp_sums, context_lens, Hkv, partition_size, num_parts):
    num_seqs, Hq, D = out.shape
    check(lib.paged_reduce(dtype_code(out), ptr(out), out.stride(0), out.stride(1), ptr(tmp_out),
                           ptr(max_logits), ptr(exp_sums), ptr(context_lens), num_seqs, Hq, Hkv, D,
                           int(partition_size), int(num_parts), stream_of(out)), "paged_reduce")


def fa_probe_mfma(lib, sink, iters, random_operands=True, dtype=torch.bfloat16):
    """Enqueues the matrix-pipe rate probe on ``sink``'s device; returns the FLOP the launch executes."""
    code = F16 if dtype == torch.float16 else BF16
    check(lib.fa_probe_mfma(code, int(bool(random_operands)), int(iters), ptr(sink), sink.numel(), stream_of(sink)),
          "fa_probe_mfma")
    return lib.fa_num_cus() * 4 * int(iters) * 16 * 32768
