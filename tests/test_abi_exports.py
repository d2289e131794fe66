"""The built library exports every symbol the public header declares, and the ctypes table
covers the same set (no compute is invoked: this runs without a GPU)."""
import ctypes
import os
import re

import pytest

from catccos_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "catccos_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cch_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_something():
    syms = declared_symbols()
    assert "cch_mx_quant_rows" in syms and "cch_init" in syms


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_abi.LIB_PATH):
        pytest.fail("libcatccos_hip.so not built; run python -m catccos_amd.build")
    L = ctypes.CDLL(_abi.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(L, s)]
    assert not missing, missing


def test_ctypes_table_matches_header():
    assert sorted(_abi.PROTOTYPES) == declared_symbols()


def test_missing_device_is_reported_not_hidden():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    L = _abi.lib()
    assert L.cch_init(0) == _abi.ENODEV
    assert b"no HIP device" in L.cch_last_error()
