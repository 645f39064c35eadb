import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_package():
    """The package directory is called `sd3.c_amd`, which is not an importable name: load it as `sd3_c_amd`."""
    if "sd3_c_amd" in sys.modules:
        return sys.modules["sd3_c_amd"]
    d = os.path.join(ROOT, "sd3.c_amd")
    spec = importlib.util.spec_from_file_location("sd3_c_amd", os.path.join(d, "__init__.py"), submodule_search_locations=[d])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["sd3_c_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pkg():
    return load_package()
