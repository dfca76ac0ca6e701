"""The C-ABI library loads and exports every symbol the header declares (CPU)."""

import ctypes
import re
from pathlib import Path

import pytest

import jigsaw_amd
from jigsaw_amd import _lib

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "jigsaw_hip.h"


def declared_symbols() -> list[str]:
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jg_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    syms = declared_symbols()
    assert "jg_last_error" in syms and "jg_halo_assemble_3d" in syms
    assert len(syms) >= 10


def test_library_is_built_in_tree():
    assert jigsaw_amd.lib_path().exists(), "run `python -m jigsaw_amd.build` first"
    assert ROOT in jigsaw_amd.lib_path().parents


def test_every_declared_symbol_is_exported():
    lib = ctypes.CDLL(str(jigsaw_amd.lib_path()))
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_table_matches_header():
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_abi_version_and_error_string():
    assert jigsaw_amd.abi_version() >= 1
    assert isinstance(jigsaw_amd.load().jg_last_error(), bytes)


def test_bad_arguments_are_rejected_without_a_gpu():
    """Argument validation happens on the host before any launch."""
    lib = jigsaw_amd.load()
    g = _lib.HaloGeom()
    g.planes = 1
    for a in range(3):
        g.size[a], g.lo[a], g.hi[a] = 4, 0, 0
    g.lo[2] = 9  # wider than the tile
    tab = _lib.VoidP27()
    rc = lib.jg_halo_assemble_3d(ctypes.c_void_p(16), tab, g, 2, None)
    assert rc == -1
    assert b"wider than the tile" in lib.jg_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc, "jg_halo_assemble_3d")
