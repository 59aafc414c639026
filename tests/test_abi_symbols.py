"""The C-ABI library loads and exports everything the header declares (no GPU)."""
import ctypes
import os

from conftest import load_scn


def test_library_exports_every_declared_symbol():
    scn = load_scn()
    assert os.path.exists(scn.LIB_PATH), "build the library first: __graft_entry__.build()"
    declared = scn.declared_symbols()
    assert len(declared) >= 25
    L = ctypes.CDLL(scn.LIB_PATH)
    missing = [s for s in declared if not hasattr(L, s)]
    assert not missing, missing


def test_binding_covers_the_header():
    scn = load_scn()
    bound = set(scn.lib()._signatures)
    assert bound == set(scn.declared_symbols())


def test_version_and_error_string_without_gpu():
    scn = load_scn()
    assert b"gfx950" in scn.lib().scn_version()
    assert isinstance(scn.lib().scn_last_error(), bytes)
