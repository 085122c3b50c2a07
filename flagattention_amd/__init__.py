"""flag_attn operators on hand-written gfx950 (MI355X) HIP kernels.

Same names as the reference package facade (``src/flag_attn/__init__.py:9-14``).
"""
from .piecewise import attention as piecewise_attention  # noqa: F401
from .flash import attention as flash_attention  # noqa: F401
from .split_kv import attention as flash_attention_split_kv  # noqa: F401
from .paged import attention as paged_attention  # noqa: F401
from .total import total_attention  # noqa: F401
from . import testing  # noqa: F401

__version__ = "0.1.0"
