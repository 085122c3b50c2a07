"""Alias package: ``import flag_attn`` resolves to the gfx950 implementation in ``flagattention_amd``
so that callers of the reference need no source change."""
import sys

import flagattention_amd as _impl
from flagattention_amd import (flash_attention, piecewise_attention, flash_attention_split_kv,  # noqa: F401
                               paged_attention, total_attention)
from flagattention_amd import flash, piecewise, paged, split_kv, total, dropout, testing  # noqa: F401

for _name in ("flash", "piecewise", "paged", "split_kv", "total", "dropout", "testing"):
    sys.modules[__name__ + "." + _name] = getattr(_impl, _name)
__version__ = _impl.__version__
