"""The C-ABI library loads without a GPU and exports exactly what include/flagattn.h declares;
the ctypes signature table matches the header's argument counts.  No compute calls."""
import os
import re

import pytest

from flagattention_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flagattn.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\bint\s+(\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        name, args = m.group(1), m.group(2).strip()
        decls[name] = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
    return decls


def test_header_declares_the_expected_entry_points():
    decls = declared_functions()
    for name in ("fa_fwd", "fa_bwd_delta", "fa_bwd_dkdv", "fa_bwd_dq", "fa_total_attn", "fa_splitkv_fwd",
                 "fa_splitkv_combine", "pw_fwd", "pw_bwd_dkdv", "pw_bwd_dq", "paged_attn", "paged_reduce",
                 "fa_num_cus", "fa_version"):
        assert name in decls


def test_signature_table_matches_header():
    decls = declared_functions()
    assert set(decls) == set(_lib.SIGNATURES)
    for name, nargs in decls.items():
        assert len(_lib.SIGNATURES[name]) == nargs, name


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} has not been built (run `python -c 'import __graft_entry__ as g; g.build()'`)")
    lib = _lib.bind(_lib.LIB_PATH)  # getattr on every declared name; raises if one is missing
    assert lib.fa_version() >= 1


def test_missing_library_raises(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.get()
