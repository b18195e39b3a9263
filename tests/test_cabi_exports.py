"""CPU checks of the C-ABI boundary: the library loads, exports every symbol the header
declares, and the ctypes signature table covers exactly that set. No compute calls."""

import ctypes
import os
import re

from moespresso_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "moespresso_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mspr_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert _lib.library_available(), "build the library first: python -m moespresso_amd.build"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 10
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in the header but not exported"


def test_ctypes_table_matches_header():
    assert sorted(_lib.SIGNATURES) == _declared_symbols()


def test_abi_version_and_error_text():
    lib = _lib.lib()
    assert lib.mspr_abi_version() >= 1
    # a rejected call reports through the return code and mspr_last_error, without touching a GPU
    rc = lib.mspr_topk_select(None, 0, 1, 10, 5, None, None)
    assert rc == _lib.MSPR_ERR_ARG
    assert b"null pointer" in lib.mspr_last_error()
