"""The C-ABI library loads without a GPU and exports every symbol that
include/moonep_hip.h declares; host-side argument validation returns error
codes without touching a device."""

import ctypes
import os
import re

from moonep_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "moonep_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mep_[a-z_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert _declared() == sorted(_lib.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name


def test_version_and_error_strings():
    lib = _lib.lib()
    assert lib.mep_version() >= 100
    assert lib.mep_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4):
        assert len(lib.mep_strerror(code)) > 3


def test_argument_validation_needs_no_device():
    lib = _lib.lib()
    # null pointers / bad sizes are rejected before any launch
    assert lib.mep_plan(None, None, 0, 4, 2, 8, 2, 8, 64, None, None, None, None, None, None, 0, None) == -1
    assert lib.mep_dispatch(None, None, None, None, None, 0, None, 0, 0, 4, 64, 2, 2, 4, 64, 8, 0, None) == -1
    assert lib.mep_combine(None, 0, None, 0, None, None, None, 4, 64, 2, 2, 64, 0, None) == -1
    assert lib.mep_grad_reduce(None, None, 0, None, 0, 4, 2, 16, None) == -1
    assert lib.mep_plan_scratch_bytes(4096, 8, 256, 8, 1) == 0          # tables fit in LDS
    assert lib.mep_plan_scratch_bytes(256, 1, 2050, 2, 2) > 0           # they do not
    assert lib.mep_dedup_scratch_bytes(4096, 8) >= 4096 * 8 * 4


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    try:
        _lib.lib()
    except RuntimeError as e:
        assert "no CPU or eager fallback" in str(e)
    else:
        raise AssertionError("expected RuntimeError")
