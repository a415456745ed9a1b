"""The C-ABI library must load and export every symbol include/mi355x_search.h declares (no GPU calls)."""
import ctypes
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import pytest  # noqa: E402

import __graft_entry__ as ge  # noqa: E402


@pytest.fixture(scope="module", autouse=True)
def built():
    ge.ensure_built()  # compiles only where no library has been built yet


def test_every_declared_symbol_is_exported():
    hdr = open(os.path.join(ROOT, "include", "mi355x_search.h")).read()
    names = set(re.findall(r"\b(mi355x_[a-z0-9_]+)\s*\(", hdr))
    assert len(names) >= 20
    so = os.path.join(ROOT, "onnxruntime-genai_amd", "libmi355x_search.so")
    assert os.path.exists(so), "build the library first: python __graft_entry__.py"
    lib = ctypes.CDLL(so)
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, f"declared but not exported: {missing}"


def test_error_paths_without_gpu():
    lib = ctypes.CDLL(os.path.join(ROOT, "onnxruntime-genai_amd", "libmi355x_search.so"))
    lib.mi355x_search_last_error.restype = ctypes.c_char_p
    h = ctypes.c_void_p()
    assert lib.mi355x_search_create(0, 0, 100, ctypes.byref(h)) == -1  # MI355X_E_INVALID before any HIP call
    assert b"positive" in lib.mi355x_search_last_error()
    assert lib.mi355x_argmax(None, None, None, 1, 0, 1, 1, None, None) == -1
    assert b"null context" in lib.mi355x_search_last_error()
