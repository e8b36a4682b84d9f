import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def load_package():
    """The package directory name has a hyphen, so it is imported by path."""
    import importlib.util

    name = "jpdc23_artifact_amd"
    if name in sys.modules:
        return sys.modules[name]
    path = os.path.join(ROOT, "jpdc23-artifact_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=[os.path.dirname(path)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import xcorr_oracle

    xcorr_oracle.lib()
    return xcorr_oracle


@pytest.fixture(scope="session")
def xc():
    return load_package()
