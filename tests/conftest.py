import importlib.util
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


# The driver executables are started by a small launcher process that is itself started before any test has touched
# the GPU (a process that has initialised the GPU must not start other programs on these machines).
_LAUNCHER_CODE = r"""
import json, subprocess, sys
for line in sys.stdin:
    req = json.loads(line)
    try:
        r = subprocess.run(req["argv"], env=req["env"], capture_output=True, text=True, timeout=req["timeout"])
        out = {"rc": r.returncode, "stdout": r.stdout, "stderr": r.stderr}
    except subprocess.TimeoutExpired as e:
        out = {"rc": 124, "stdout": "", "stderr": "timeout after %s s" % req["timeout"]}
    except OSError as e:
        out = {"rc": 127, "stdout": "", "stderr": str(e)}
    sys.stdout.write(json.dumps(out) + "\n")
    sys.stdout.flush()
"""
_launcher = None


def pytest_collection_finish(session):
    global _launcher
    if _launcher is None and any("test_gpu_drivers" in item.nodeid for item in session.items):
        _launcher = subprocess.Popen([sys.executable, "-u", "-c", _LAUNCHER_CODE], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)


def pytest_sessionfinish(session, exitstatus):
    global _launcher
    if _launcher is not None:
        _launcher.stdin.close()
        _launcher.wait(timeout=30)
        _launcher = None


@pytest.fixture(scope="session")
def run_program():
    """run_program(argv, env, timeout) -> dict(rc, stdout, stderr), executed by the launcher process."""
    import json
    if _launcher is None:
        pytest.skip("launcher process not started")

    def run(argv, env=None, timeout=300):
        _launcher.stdin.write(json.dumps({"argv": [str(a) for a in argv], "env": dict(env or os.environ), "timeout": timeout}) + "\n")
        _launcher.stdin.flush()
        return json.loads(_launcher.stdout.readline())
    return run


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


class _HostReferenceBlas:
    """Stands where OpenBLAS stands when none is found on the machine: the same five entry points, computed by the
    oracle's long double brute force (GEMM, GEMV, dot) and its fused daxpy.  Slower, but a parity test then still
    compares the device result with an independent host result instead of being skipped."""

    def __init__(self, orc):
        self._orc = orc

    def __getattr__(self, name):
        return getattr(self._orc, name)

    def orc_openblas_dgemm(self, ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc):
        self._orc.orc_dgemm_bruteforce(ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc)
        return 0

    def orc_openblas_sgemm(self, ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc):
        self._orc.orc_sgemm_bruteforce(ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc)
        return 0

    def orc_openblas_dgemv(self, ta, M, N, alpha, A, lda, x, incx, beta, y, incy):
        self._orc.orc_dgemv_bruteforce(ta, M, N, alpha, A, lda, x, incx, beta, y, incy)
        return 0

    def orc_openblas_daxpy(self, n, alpha, x, incx, y, incy):
        self._orc.orc_daxpy(n, alpha, x, incx, y, incy)
        return 0

    def orc_openblas_ddot(self, n, x, incx, y, incy, out):
        out._obj.value = float(self._orc.orc_ddot_longdouble(n, x, incx, y, incy))
        return 0

    def orc_openblas_path(self):
        return b"(none: host reference = the oracle's long double brute force)"


@pytest.fixture(scope="session")
def openblas(orc):
    if orc.orc_openblas_open(None) != 0:
        print("\nno OpenBLAS found on this machine: parity checks run against the oracle's brute-force host reference", flush=True)
        return _HostReferenceBlas(orc)
    return orc
