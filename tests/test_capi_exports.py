"""The C-ABI library loads and exports every symbol the headers under include/ declare (no GPU work)."""
import ctypes
import os
import re

from cudf_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = set()
    for header in sorted(os.listdir(os.path.join(ROOT, "include"))):
        if not header.endswith(".h"):
            continue
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(nvtext_amd_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_header_and_binding_agree():
    assert declared_functions() == sorted(_capi.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name


def test_version_and_error_text_without_gpu():
    lib = _capi.load()
    assert lib.nvtext_amd_version() >= 100
    assert isinstance(lib.nvtext_amd_last_error(), bytes)


def test_argument_checks_need_no_gpu():
    """Argument validation happens before any device work, as in the reference
    (cpp/src/text/minhash.cu:435-446, cpp/src/text/wordpiece_tokenize.cu:217-218)."""
    lib = _capi.load()
    col = _capi.StringsColumn(None, None, 0, None, 1, 0, 0)
    out = _capi.ListColumn()
    st = lib.nvtext_amd_minhash(ctypes.byref(col), 0, None, None, 0, 0, 1, None, None, ctypes.byref(out))
    assert st == _capi.INVALID_ARGUMENT
    assert b"width" in lib.nvtext_amd_last_error()
    st = lib.nvtext_amd_minhash(ctypes.byref(col), 0, None, None, 0, 0, 4, None, None, ctypes.byref(out))
    assert st == _capi.INVALID_ARGUMENT and b"cannot be empty" in lib.nvtext_amd_last_error()
    st = lib.nvtext_amd_minhash64(ctypes.byref(col), 0, None, None, 3, 2, 4, None, None, ctypes.byref(out))
    assert st == _capi.INVALID_ARGUMENT
    big = _capi.StringsColumn(None, None, 0, None, 50000, 0, 0)
    st = lib.nvtext_amd_minhash(ctypes.byref(big), 0, None, None, 50000, 50000, 4, None, None, ctypes.byref(out))
    assert st == _capi.OVERFLOW
    empty = _capi.StringsColumn(None, None, 0, None, 0, 0, 0)
    h = ctypes.c_void_p()
    st = lib.nvtext_amd_wordpiece_vocabulary_create(ctypes.byref(empty), None, None, ctypes.byref(h))
    assert st == _capi.INVALID_ARGUMENT and b"must not be empty" in lib.nvtext_amd_last_error()
    nulls = _capi.StringsColumn(None, None, 0, None, 3, 0, 3)
    st = lib.nvtext_amd_wordpiece_vocabulary_create(ctypes.byref(nulls), None, None, ctypes.byref(h))
    assert st == _capi.INVALID_ARGUMENT and b"nulls" in lib.nvtext_amd_last_error()
