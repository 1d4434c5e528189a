"""Shared test plumbing: the `gpu` marker, import paths for the package (its directory name
has a hyphen, so it is loaded by path under the module name `project_aeon_amd`) and for the
CPU oracle's ctypes front end."""
import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _load_package():
    if "project_aeon_amd" in sys.modules:
        return sys.modules["project_aeon_amd"]
    pkg_dir = os.path.join(ROOT, "project-aeon_amd")
    spec = importlib.util.spec_from_file_location(
        "project_aeon_amd", os.path.join(pkg_dir, "__init__.py"),
        submodule_search_locations=[pkg_dir])
    module = importlib.util.module_from_spec(spec)
    sys.modules["project_aeon_amd"] = module
    spec.loader.exec_module(module)
    return module


_load_package()
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.join(ROOT, "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    import orc as _orc
    _orc.lib()
    return _orc


@pytest.fixture(scope="session")
def ref(orc):
    r = orc.ref()
    if r is None:
        pytest.skip("oracle/_ref was not built (the reference tree is absent)")
    return r
