"""Dropout mask of flash_attention, restated on the CPU (test infrastructure only).

The reference draws one Philox-4x32 number per score element (``src/flag_attn/flash.py:367-371,
454-457``; mask recomputation for its tests in ``src/flag_attn/testing/dropout.py:5-27``):

    counter = offset + ((b * H + h) * M + m) * N + n       (low word c0, high word c1, c2 = c3 = 0)
    key     = seed                                          (low word k0, high word k1)
    x       = first output word of 6 Philox rounds
    keep    = uniform(x) > dropout_p

with Triton's ``tl.rand(seed, offs, n_rounds=6)`` (dependency ``triton>=2.2.0``, installed copy 3.6.0,
``triton/language/random.py``: ``philox_impl``, ``randint4x``, ``uint_to_uniform_float``) whose published
algorithm is restated here: Philox-4x32 with multipliers 0xD2511F53 / 0xCD9E8D57 and key increments
0x9E3779B9 / 0xBB67AE85, and uniform(x) = (x as int32, negative values mapped to -x - 1) * 4.6566127342e-10.

Pinned by (tests/test_oracle_dropout.py): the Random123 known-answer vectors of philox4x32 with 10 rounds
(the round function does not depend on the round count), the drop rate, the bounds of the uniform map --
and, bit for bit, by what Triton 3.6.0's ``tl.rand`` returns for seeds and counters on both sides of 2^31
and 2^32 and by the masks the reference's ``recompute_mask_kernel`` draws, both produced with Triton's CPU
interpreter (tests/golden/make_dropout_vectors.py -> tests/golden/dropout_vectors.npz).

One difference is known and lies outside what the reference can do: its kernels form the counter in 32-bit
arithmetic whenever seed offset and tensor extents fit 32 bits (Triton types integer arguments by value),
so it wraps for score tensors of 2^31 elements and more; the counter here is 64 bits wide throughout.
"""
import numpy as np
import torch

_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = np.uint32(0x9E3779B9), np.uint32(0xBB67AE85)
_LO = np.uint64(0xFFFFFFFF)


def philox4x32(c0, c1, c2, c3, k0, k1, rounds):
    """Philox-4x32 on uint32 arrays (broadcast); returns the four output words."""
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint32) for c in (c0, c1, c2, c3))
    k0, k1 = np.uint32(k0), np.uint32(k1)
    with np.errstate(over="ignore"):
        for _ in range(rounds):
            p0 = _M0 * c0.astype(np.uint64)   # 64-bit products
            p1 = _M1 * c2.astype(np.uint64)
            hi0, lo0 = (p0 >> np.uint64(32)).astype(np.uint32), (p0 & _LO).astype(np.uint32)
            hi1, lo1 = (p1 >> np.uint64(32)).astype(np.uint32), (p1 & _LO).astype(np.uint32)
            c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
            k0, k1 = np.uint32(k0 + _W0), np.uint32(k1 + _W1)
    return c0, c1, c2, c3


def uniform_from_bits(x):
    """uint32 -> float32 in [0, 1): reinterpret as int32, fold negatives, scale by just under 2^-31."""
    v = np.asarray(x, dtype=np.uint32).view(np.int32).astype(np.int64)
    v = np.where(v < 0, -v - 1, v)
    return (v.astype(np.float32) * np.float32(4.6566127342e-10)).astype(np.float32)


def keep_mask(B, H, M, N, dropout_p, seed, offset, device="cpu"):
    """Boolean (B, H, M, N) tensor: True where the probability is kept."""
    if dropout_p == 0:
        return torch.ones(B, H, M, N, dtype=torch.bool, device=device)
    ctr = np.uint64(offset) + np.arange(B * H * M * N, dtype=np.uint64)
    zeros = np.zeros(ctr.shape, dtype=np.uint32)
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    x, _, _, _ = philox4x32((ctr & _LO).astype(np.uint32), (ctr >> np.uint64(32)).astype(np.uint32), zeros, zeros,
                            seed & 0xFFFFFFFF, seed >> 32, 6)
    keep = uniform_from_bits(x) > np.float32(dropout_p)
    return torch.from_numpy(keep.reshape(B, H, M, N)).to(device)
