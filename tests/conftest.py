import importlib.util
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def load_package():
    """The package directory is named paralia-framework_amd (not an identifier): import it by path."""
    name = "paralia_framework_amd"
    if name in sys.modules:
        return sys.modules[name]
    init = os.path.join(ROOT, "paralia-framework_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location(name, init, submodule_search_locations=[os.path.dirname(init)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pkg():
    mod = load_package()
    if not os.path.exists(mod.LIB_PATH):  # tests load what is built and build only if nothing is
        mod.build_library()
    return mod


@pytest.fixture(scope="session")
def L(pkg):
    return pkg.load()


@pytest.fixture(scope="session")
def orc():
    import oracle_binding
    return oracle_binding.load()


@pytest.fixture(scope="session")
def openblas(orc):
    if orc.orc_openblas_open(None) != 0:
        pytest.skip("no OpenBLAS found on this machine: OpenBLAS parity checks skipped (brute-force oracle still runs)")
    return orc
