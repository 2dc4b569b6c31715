"""ctypes face of libparalia.so, the MI355X-native PARALiA runtime.

The product is the shared library (HIP kernels, C ABI, C++ scheduler and autotuner); this module only declares
its C signatures for Python callers such as the tests and the benchmark.  There is no Python or CPU fallback:
loading fails loudly when the library has not been built.
"""
from .binding import (LIB_PATH, PKG_DIR, ParaliaError, atc_info, build_library, check, lib, load, plan_rows,
                      PL_PLAN_ROW, PL_PLAN_MAX_WAITS)

__all__ = ["LIB_PATH", "PKG_DIR", "ParaliaError", "atc_info", "build_library", "check", "lib", "load", "plan_rows",
           "PL_PLAN_ROW", "PL_PLAN_MAX_WAITS"]
