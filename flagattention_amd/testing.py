"""``flag_attn.testing`` namespace of the reference (``src/flag_attn/testing/__init__.py``), as far as it
is device code: ``recompute_mask``.  The plain-torch reference implementations of the operators are
not part of this package."""
from .dropout import recompute_mask  # noqa: F401

__all__ = ["recompute_mask"]
