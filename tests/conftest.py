import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # the no-allocation entry point's test must be collected last
    items.sort(key=lambda it: 1 if "test_zz_" in it.nodeid else 0)


def load_scn():
    """Import the package (its folder name is not a Python identifier)."""
    import importlib.util

    name = "sparseconvnet_archived_amd"
    if name in sys.modules:
        return sys.modules[name]
    path = os.path.join(ROOT, "sparseconvnet-archived_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=[os.path.dirname(path)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def scn():
    return load_scn()


@pytest.fixture(scope="session")
def ctx(scn):
    c = scn.Context(0)
    yield c
    c.close()
