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


def _stride(t, dim):
    # the stride of a dimension of extent 1 is never used; torch leaves arbitrary values there
    return t.stride(dim) if t.shape[dim] > 1 else 0


def view4(t):
    assert t.dim() == 4 and t.stride(-1) == 1
    return ctypes.byref(View4(t.data_ptr(), _stride(t, 0), _stride(t, 1), _stride(t, 2)))


def ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def check(code, what):
    if code == 0:
        return
    if code == -1:
        raise AssertionError(f"{what}: argument rejected by the kernel library")
    if code == -2:
        raise AssertionError(f"{what}: configuration not supported by the kernel library")
    raise KernelError(f"{what}: HIP error {code}")


def kernel_ready(t):
    """The kernels move 16 bytes at a time: unit inner stride, 16-byte aligned base, strides that are
    multiples of 8 elements.  Anything else is copied (the reference copies when the inner stride is
    not 1, src/flag_attn/flash.py:14-17)."""
    ok = (t.stride(-1) == 1 and t.data_ptr() % 16 == 0
          and all(_stride(t, d) % 8 == 0 for d in range(t.dim() - 1)))
    return t if ok else t.clone(memory_format=torch.contiguous_format)


def fa_fwd(lib, q, k, v, o, lse, causal, sm_scale):
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    check(lib.fa_fwd(dtype_code(q), view4(q), view4(k), view4(v), view4(o), ptr(lse),
                     B, H, Hk, M, N, D, int(causal), float(sm_scale), stream_of(q)), "fa_fwd")


def pw_fwd(lib, q1, k1, q2, k2, v, o, lse, w, causal, sm_scale):
    B, H, M, D = q1.shape
    N = k1.shape[2]
    check(lib.pw_fwd(dtype_code(q1), view4(q1), view4(k1), view4(q2), view4(k2), view4(v), view4(o),
                     ptr(lse), B, H, M, N, D, int(w), int(causal), float(sm_scale), stream_of(q1)),
          "pw_fwd")
