"""ctypes face of oracle/liboracle.so -- the CPU restatement used as the checker (test infrastructure only)."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "liboracle.so")


class orc_link(C.Structure):
    _fields_ = [("ti", C.c_double), ("tb", C.c_double), ("sl", C.c_double)]


class orc_exec_table(C.Structure):
    _fields_ = [("lines", C.c_int), ("T", C.POINTER(C.c_long)), ("t", C.POINTER(C.c_double)), ("ta", C.c_char_p),
                ("tb", C.c_char_p)]


class orc_problem(C.Structure):
    _fields_ = [("D1", C.c_long), ("D2", C.c_long), ("D3", C.c_long), ("dtype_sz", C.c_int), ("ta", C.c_char),
                ("tb", C.c_char), ("remote", C.c_int * 3), ("out_remote", C.c_int * 3), ("h2d", orc_link),
                ("d2h", orc_link), ("exec", C.POINTER(orc_exec_table))]


_vp, _l, _ll, _i, _d, _f, _c = C.c_void_p, C.c_long, C.c_longlong, C.c_int, C.c_double, C.c_float, C.c_char
_pd = C.POINTER(C.c_double)

_SIGS = {
    "orc_splitmix64": (C.c_uint64, [C.POINTER(C.c_uint64)]),
    "orc_rand_fill_f64": (None, [_vp, _ll, C.c_uint64]),
    "orc_rand_fill_f32": (None, [_vp, _ll, C.c_uint64]),
    "orc_normwise_err_f64": (_d, [_vp, _vp, _l, _l, _l, _l, _d]),
    "orc_normwise_err_f32": (_d, [_vp, _vp, _l, _l, _l, _l, _d]),
    "orc_fro_norm_f64": (_d, [_vp, _l, _l, _l]),
    "orc_fro_norm_f32": (_d, [_vp, _l, _l, _l]),
    "orc_max_ulp_f64": (_ll, [_vp, _vp, _ll]),
    "orc_digits_equal": (_i, [_vp, _vp, _ll]),
    "orc_dgemm_bruteforce": (None, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l]),
    "orc_sgemm_bruteforce": (None, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l]),
    "orc_dgemm_tiled": (_l, [_l, _i, _c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l]),
    "orc_sgemm_tiled": (_l, [_l, _i, _c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l]),
    "orc_dgemv_bruteforce": (None, [_c, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l]),
    "orc_dgemv_tiled": (_l, [_l, _c, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l]),
    "orc_daxpy": (None, [_l, _d, _vp, _l, _vp, _l]),
    "orc_daxpy_mul_add": (None, [_l, _d, _vp, _l, _vp, _l]),
    "orc_daxpy_tiled": (_l, [_l, _l, _d, _vp, _l, _vp, _l]),
    "orc_ddot_tiled": (_l, [_l, _l, _vp, _l, _vp, _l, _pd]),
    "orc_ddot_longdouble": (C.c_longdouble, [_l, _vp, _l, _vp, _l]),
    "orc_sk_num_blas3": (_l, [_l, _l, _l, _l]),
    "orc_get_T_slowdowns": (None, [_l, _l, _l, _i, _l, _pd]),
    "orc_optimize_tile": (_l, [_l, _l, _l, _i, _pd]),
    "orc_gemm_block_num": (_l, [_l, _l, _l, _l, _i]),
    "orc_t_com_predict": (_d, [C.POINTER(orc_link), _d]),
    "orc_t_com_sl": (_d, [C.POINTER(orc_link), _d]),
    "orc_t_com_bid_predict": (_d, [C.POINTER(orc_link), C.POINTER(orc_link), _d, _d]),
    "orc_clamp_slowdown": (_d, [_d]),
    "orc_exec_nearest_T": (_l, [C.POINTER(orc_exec_table), _l]),
    "orc_exec_predict": (_d, [C.POINTER(orc_exec_table), _l, _c, _c]),
    "orc_predict_blas3": (_d, [_i, C.POINTER(orc_problem), _l]),
    "orc_predict_blas1_bidirectional": (_d, [C.POINTER(orc_problem), _i, C.POINTER(_i), C.POINTER(_i), _l]),
    "orc_predict_blas2": (_d, [_i, C.POINTER(orc_problem), _l]),
    "orc_optimize_tile_model": (_l, [_i, C.POINTER(orc_problem), _pd]),
    "orc_openblas_open": (_i, [C.c_char_p]),
    "orc_openblas_path": (C.c_char_p, []),
    "orc_openblas_config": (C.c_char_p, []),
    "orc_openblas_threads": (_i, [_i]),
    "orc_openblas_dgemm": (_i, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l]),
    "orc_openblas_sgemm": (_i, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l]),
    "orc_openblas_dgemv": (_i, [_c, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l]),
    "orc_openblas_daxpy": (_i, [_l, _d, _vp, _l, _vp, _l]),
    "orc_openblas_ddot": (_i, [_l, _vp, _l, _vp, _l, _pd]),
}

_lib = None


def build():
    subprocess.run(["make", "-C", ORACLE_DIR], check=True)


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(ORACLE_LIB):
        build()
    L = C.CDLL(ORACLE_LIB)
    for name, (res, args) in _SIGS.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def rand_f64(n, seed):
    a = np.empty(n, dtype=np.float64)
    load().orc_rand_fill_f64(ptr(a), n, seed)
    return a


def rand_f32(n, seed):
    a = np.empty(n, dtype=np.float32)
    load().orc_rand_fill_f32(ptr(a), n, seed)
    return a


def make_table(Ts, ts, ta=None, tb=None):
    """Build an orc_exec_table; the returned tuple keeps the backing arrays alive."""
    n = len(Ts)
    Tarr = (C.c_long * n)(*Ts)
    tarr = (C.c_double * n)(*ts)
    tab = orc_exec_table(n, Tarr, tarr, ta.encode() if ta else None, tb.encode() if tb else None)
    return tab, (Tarr, tarr)
