"""The C-ABI library loads (no GPU needed) and exports every symbol the header declares."""

import ctypes
import re
from pathlib import Path

from steptronoss_amd import _lib

ROOT = Path(__file__).resolve().parents[1]


def _declared_symbols():
    text = (ROOT / "include" / "steptron_moe.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(stm_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared_symbols()
    assert len(names) >= 10
    lib = ctypes.CDLL(str(_lib.library_path()))
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"


def test_version_and_status_strings():
    lib = _lib.load()
    assert lib.stm_abi_version() >= 1
    assert _lib.status_string(0) == "ok"
    assert "workspace" in _lib.status_string(-3)


def test_workspace_query_is_host_only():
    lib = _lib.load()
    assert lib.stm_route_workspace_bytes(131072, 128) >= 512 * 128 * 4
    assert lib.stm_route_workspace_bytes(0, 128) > 0
