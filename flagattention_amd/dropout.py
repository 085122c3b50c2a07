"""Dropout bookkeeping of ``flash_attention``: the generator state the mask is drawn from, and the mask
itself as a tensor.

Counterparts of ``src/flag_attn/dropout.py:5-16`` (``philox_cuda_seed_offset``) and of
``src/flag_attn/testing/dropout.py:19-25`` (``recompute_mask``) of the reference.
"""
import torch

from . import _abi, _lib

__all__ = ["philox_cuda_seed_offset", "recompute_mask"]


def philox_cuda_seed_offset(increment, device=None):
    """(seed, offset) of the device's default random generator, whose offset is then advanced by
    ``increment`` rounded up to a multiple of 4 -- the generator state is two int64 words, seed and
    offset, exactly as the reference reads and advances it."""
    if device is None:
        index = torch.cuda.current_device()
    else:
        device = torch.device(device)
        index = device.index if device.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[index]
    state = gen.get_state()
    words = state.view(torch.int64)
    seed, offset = int(words[0]), int(words[1])
    words[1] += (increment + 3) // 4 * 4
    gen.set_state(state)
    return seed, offset


def recompute_mask(B, H, M, N, dropout_p, seed, offset, device):
    """The (B, H, M, N) bool mask (True = kept) that ``flash_attention`` applied for
    ``(dropout_p, seed, offset)``, written by a HIP kernel that draws the same Philox numbers."""
    mask = torch.full((B, H, M, N), True, dtype=torch.bool, device=device)
    if dropout_p == 0:
        return mask
    lib = _lib.get()
    with torch.cuda.device(mask.device):
        _abi.fa_dropout_mask(lib, mask, dropout_p, seed, offset)
    return mask
