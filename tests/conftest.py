import importlib.util
import os
import sys

import pytest

# PyTorch ships its own copy of the HIP runtime under the same soname as the
# system one the C-ABI libraries are linked against; whichever is loaded first
# serves the whole process.  Tests use torch for device memory, so its copy has
# to be the one: import it before any test loads a library.
try:
    import torch  # noqa: F401
except ImportError:      # the CPU-only checks do not need it
    torch = None

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_package():
    """The package directory is named `ascend-mlir_amd`; a hyphen cannot be
    imported by name, so register it under `ascend_mlir_amd`."""
    name = "ascend_mlir_amd"
    if name in sys.modules:
        return sys.modules[name]
    pkg_dir = os.path.join(ROOT, "ascend-mlir_amd")
    spec = importlib.util.spec_from_file_location(
        name, os.path.join(pkg_dir, "__init__.py"),
        submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pkg():
    return load_package()
