"""Tile-configuration hooks.

The reference lets callers replace the module-level ``get_fwd_config`` / ``get_bwd_config`` functions
(``src/flag_attn/flash.py:290,493``, ``examples/use_cutom_config_func.py:6-9``) and calls them before
every launch (``flash.py:64-66, 185-186``); Triton then compiles a kernel for whatever tile comes
back.  Here the kernels are compiled ahead of time for a fixed set of tiles, so the wrappers still
call the hook on every launch, use its answer when it names a compiled tile, and otherwise say so --
once per distinct answer -- and launch the default.
"""
import warnings

_warned = set()


def warn_once(key, message):
    if key not in _warned:
        _warned.add(key)
        warnings.warn(message, RuntimeWarning, stacklevel=3)


def resolve(hook, compiled, what, args):
    """Calls ``hook(*args)`` -> (BLOCK_M, BLOCK_N, num_stages, num_warps) and returns the
    (BLOCK_M, BLOCK_N) to launch: the hook's if it is in ``compiled`` (a sequence whose first entry is
    the default), else the default after a one-time warning."""
    cfg = hook(*args)
    try:
        block_m, block_n, num_stages, num_warps = (int(x) for x in cfg)
    except (TypeError, ValueError):
        raise AssertionError(f"{what}: the config hook must return (BLOCK_M, BLOCK_N, num_stages, num_warps), "
                             f"got {cfg!r}")
    assert block_m > 0 and block_n > 0 and num_stages > 0 and num_warps > 0, \
        f"{what}: config values must be positive, got {cfg!r}"
    if (block_m, block_n) in compiled:
        return block_m, block_n
    key = (what, block_m, block_n)
    if key not in _warned:
        _warned.add(key)
        warnings.warn(f"{what}: tile (BLOCK_M={block_m}, BLOCK_N={block_n}) is not among the tiles the gfx950 "
                      f"kernels are compiled for {list(compiled)}; launching {compiled[0]}. num_stages and "
                      "num_warps are fixed by the kernels.", RuntimeWarning, stacklevel=3)
    return compiled[0]
