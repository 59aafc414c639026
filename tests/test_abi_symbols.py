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


def test_host_library_exports_the_c_facade():
    scn = load_scn()
    from sparseconvnet_archived_amd import hostapi
    assert os.path.exists(hostapi.LIB_PATH)
    L = hostapi.lib()
    import re
    hdr = open(os.path.join(os.path.dirname(hostapi.LIB_PATH), "host", "scn_host_c.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    for name in sorted(set(re.findall(r"\b(scnh_[a-z0-9_]+)\s*\(", hdr))):
        assert hasattr(L, name), name
