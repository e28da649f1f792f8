"""The shared library loads without a GPU and exports every symbol include/metis_hip.h declares."""
import os
import re

from metis_hip import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "metis_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(metis_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in metis_hip.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_host_only_calls():
    lib = _lib.load()
    assert lib.metis_version() >= 0x100
    assert b"16" in lib.metis_error_string(_lib.E_SHAPE)
    assert lib.metis_nvfp4_workspace_bytes(8192, 4096) >= 8192 * 4096 // 16 * 2
    assert lib.metis_nvfp4_workspace_bytes(0, 0) > 0
