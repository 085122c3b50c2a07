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
    assert lib.fa_version() == _lib.ABI_VERSION
    text = open(HEADER).read()
    assert int(re.search(r"#define\s+FA_ABI_VERSION\s+(\d+)", text).group(1)) == _lib.ABI_VERSION


def test_loader_refuses_a_library_of_another_interface_revision(monkeypatch):
    """A caller built against another argument list must not call the library: bind() compares revisions."""
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} has not been built")
    monkeypatch.setattr(_lib, "ABI_VERSION", _lib.ABI_VERSION + 1)
    with pytest.raises(RuntimeError, match="revision"):
        _lib.bind(_lib.LIB_PATH)


def test_missing_library_raises(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.get()


def test_integration_doc_binding_matches_signature_table():
    """The worked ctypes binding in the integration document is evaluated as written (with a stand-in
    for the loaded library) and its argument types must equal the loader's table for fa_fwd."""
    import ctypes
    import types
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    block = next(b for b in blocks if "fa_fwd.argtypes" in b)
    # everything up to the helper that touches tensors: struct, library handle, argtypes, restype
    setup = block.split("def _view")[0]
    setup = setup.replace("import ctypes, torch", "import ctypes")
    fake_lib = types.SimpleNamespace(fa_fwd=types.SimpleNamespace())
    setup = setup.replace('ctypes.CDLL("libflagattn_hip.so")', "_fake_lib")
    env = {"_fake_lib": fake_lib}
    exec(setup, env)
    doc_types = fake_lib.fa_fwd.argtypes
    table = _lib.SIGNATURES["fa_fwd"]
    assert len(doc_types) == len(table) == declared_functions()["fa_fwd"]
    for i, (d, t) in enumerate(zip(doc_types, table)):
        if t is _lib._v:   # pointer to the view struct: the document declares its own mirror of it
            assert issubclass(d, ctypes._Pointer) and \
                [f[0] for f in d._type_._fields_] == [f[0] for f in _lib.View4._fields_], i
        else:
            assert d is t, (i, d, t)
    assert fake_lib.fa_fwd.restype is ctypes.c_int
    # the call in the document passes as many arguments as the binding declares
    call = re.search(r"_lib\.fa_fwd\((.*?)\)\nassert rc == 0", block, flags=re.S).group(1)
    call = re.sub(r"#.*", "", call)
    depth, nargs = 0, 1
    for ch in call:
        depth += ch in "([" 
        depth -= ch in ")]"
        nargs += (ch == "," and depth == 0)
    assert nargs == len(table)
