"""The C-ABI library loads without a GPU and exports every symbol include/sptmm.h declares."""
import ctypes
import os
import re

import pytest

import sptmm_amd as sp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sptmm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sptmm_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(sp.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(sp.lib_path())
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_errors_are_reported_not_fatal():
    with pytest.raises(sp.SptmmError) as e:
        sp.generate_ternary(6912, 2560, 4097)
    assert "S mod 2" in str(e.value)
    assert sp.lib().sptmm_version().startswith(b"sptmm")


def test_no_cpu_fallback_in_product():
    # the package must not reach for the oracle
    for root, _, files in os.walk(os.path.join(ROOT, "sptmm_amd")):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".hpp", ".h")):
                src = open(os.path.join(root, f)).read()
                assert "oracle" not in src.lower(), f
