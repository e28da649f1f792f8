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


def test_size_helpers_of_the_one_pass_entry_points_need_no_device():
    """The workspace and buffer sizes a caller asks for before it allocates: pure host arithmetic (a 256-CU device is
    assumed when none is present).  K slices only while the row tiles alone leave compute units idle, never more than 16,
    never fewer than four 256-element steps each; the deferred buffer holds 2048 partial maxima and one bf16 per block."""
    from metis_hip import _lib
    L = _lib.load()
    ws = L.metis_lowrank_project_rows_workspace_bytes
    assert ws(8192, 64, 4096) == 0 and ws(16384, 64, 18944) == 0          # 256 row tiles or more: one slice
    assert ws(1024, 64, 18944) == 16 * 1024 * 64 * 4                       # 32 row tiles, 74 steps: 16 slices
    assert ws(4096, 32, 8960) == 4 * 4096 * 32 * 4                         # 128 row tiles: 4 slices
    assert ws(4096, 32, 1536) == 0                                          # 6 steps: fewer than four per slice
    assert ws(0, 64, 4096) == 0 and ws(1024, 0, 4096) == 0
    for rows, cols in ((256, 64), (8192, 4096), (300, 192)):
        nb = rows * cols // 16
        assert L.metis_nvfp4_deferred_bytes(rows, cols) == 2048 * 4 + (nb * 2 + 255) // 256 * 256
        assert L.metis_nvfp4_workspace_bytes(rows, cols) >= 16384 + nb * 4
    assert L.metis_nvfp4_deferred_bytes(0, 64) == 0
