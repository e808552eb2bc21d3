"""pytest configuration: registers the `gpu` marker and makes the package (whose directory
name `lux.jl_amd` is not a valid Python identifier) importable as `lux_jl_amd`."""
import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def load_package():
    """Import <repo>/lux.jl_amd as module `lux_jl_amd` (idempotent)."""
    if "lux_jl_amd" in sys.modules:
        return sys.modules["lux_jl_amd"]
    pkg_dir = os.path.join(ROOT, "lux.jl_amd")
    spec = importlib.util.spec_from_file_location(
        "lux_jl_amd", os.path.join(pkg_dir, "__init__.py"), submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["lux_jl_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lux():
    return load_package()


@pytest.fixture(scope="session")
def gpu(lux):
    """The package with the HIP library initialised on device 0.  Fails loudly (never
    falls back) when the library or the device is missing."""
    lux.init(0)
    return lux
