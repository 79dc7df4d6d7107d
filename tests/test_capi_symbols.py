"""The C-ABI library loads on a machine without a GPU and exports exactly what
include/torpor_amd.h declares; the ctypes table binds every one of them."""
import ctypes
import os
import re

from torpor_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "torpor_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(tp_[a-z0-9_]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert len(names) >= 45
    l = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in sorted(names) if not hasattr(l, n)]
    assert not missing, missing


def test_ctypes_table_matches_header():
    assert set(_lib.SYMBOLS) == _declared()
    _lib.lib()   # sets restype/argtypes for all of them


def test_version_and_strerror():
    l = _lib.lib()
    assert b"gfx950" in l.tp_version()
    assert l.tp_strerror(0) == b"ok"
    assert b"address" in l.tp_strerror(-14)


def test_struct_sizes_match_the_header_layout():
    # natural alignment of the fields as declared in include/torpor_amd.h
    assert ctypes.sizeof(_lib.Config) == 64
    assert ctypes.sizeof(_lib.Epilogue) == 72
    assert ctypes.sizeof(_lib.GemmDesc) == 3 * 8 + 8 * 8 + 8 + 6 * 8 + 72
    assert ctypes.sizeof(_lib.ConvDesc) == 3 * 8 + 14 * 4 + 2 * 8 + 72
    assert ctypes.sizeof(_lib.KernelStat) == 64 + 8 + 3 * 8
