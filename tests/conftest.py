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


def pytest_sessionfinish(session, exitstatus):
    """LUX_PARITY_REPORT=<path>: write every comparison of this run (name, storage type, allowed and achieved worst
    error in units of |want| + rms, the float32 oracle's own worst error where the test supplied it) as JSON."""
    path = os.environ.get("LUX_PARITY_REPORT")
    if not path:
        return
    import json
    from tests.util import ERROR_LOG
    rows = [dict(what=w, dtype=t, allowed=r, worst=e, oracle_f32=e32, elements=n) for w, t, r, e, e32, n in ERROR_LOG]
    with open(path, "w") as f:
        json.dump(rows, f, indent=0)


@pytest.fixture(scope="session")
def lux():
    return load_package()


@pytest.fixture(scope="session")
def gpu(lux):
    """The package with the HIP library initialised on device 0.  Fails loudly (never
    falls back) when the library or the device is missing."""
    lux.init(0)
    return lux


@pytest.fixture(params=["resident", "streaming", "no_wait"])
def bn_path(gpu, request):
    """The three ways the library can run a training-mode batchnorm: single-pass kernels that keep
    the tensor in registers (default where it fits), the two-kernel streaming path, and the
    single-pass kernels with the wait for peer workgroups cut to zero polls, which makes every
    workgroup recompute its peers' partial results itself (the bounded-wait exit)."""
    gpu.set_option("bn_resident", 0 if request.param == "streaming" else 1)
    gpu.set_option("bn_spin_limit", 0 if request.param == "no_wait" else 1 << 22)
    yield request.param
    gpu.set_option("bn_resident", 1)
    gpu.set_option("bn_spin_limit", 1 << 22)
