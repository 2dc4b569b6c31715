"""C signatures of libparalia.so (see include/paralia_hip.h) for ctypes."""
import ctypes as C
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "lib", "libparalia.so")
PL_PLAN_MAX_WAITS = 12
PL_PLAN_ROW = 14 + PL_PLAN_MAX_WAITS


class ParaliaError(RuntimeError):
    pass


class atc_info(C.Structure):
    _fields_ = [("T", C.c_long), ("pred_t", C.c_double), ("subkernel_num", C.c_long), ("order_id", C.c_int),
                ("exec_queues", C.c_int), ("cache_limit", C.c_longlong), ("has_db", C.c_int),
                ("selected_by", C.c_char * 32), ("slowdowns", C.c_double * 6), ("pipe_total", C.c_double),
                ("pipe_h2d", C.c_double), ("pipe_exec", C.c_double), ("pipe_d2h", C.c_double)]


class gemm_fit(C.Structure):
    """pl_gemm_fit of include/paralia_hip.h."""
    _fields_ = [("lone_us_per_k", C.c_double * 2), ("lone_fixed_k", C.c_double), ("splitk_launch_us", C.c_double),
                ("pass_bytes_per_us", C.c_double), ("f32_small_us_per_k", C.c_double), ("f32_small_fixed_us", C.c_double),
                ("f32_wide_gain", C.c_double), ("f32_wide_fixed_us", C.c_double * 2), ("f32_large_gain", C.c_double * 4),
                ("f32_large_fixed_us", (C.c_double * 2) * 4), ("edge_rounds", C.c_double * 2)]


def build_library(jobs=8):
    """Compile every HIP and C++ source for gfx950 (hipcc cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", PKG_DIR, "-j%d" % jobs], check=True)


_lib = None

_vp, _l, _ll, _i, _d, _f, _c = C.c_void_p, C.c_long, C.c_longlong, C.c_int, C.c_double, C.c_float, C.c_char
_pi = C.POINTER(C.c_int)

_SIGS = {
    "pl_last_error": (C.c_char_p, []),
    "pl_device_count": (_i, [_pi]),
    "pl_set_device": (_i, [_i]),
    "pl_get_device": (_i, [_pi]),
    "pl_device_sync": (_i, []),
    "pl_device_name": (_i, [_i, C.c_char_p, _i]),
    "pl_mem_info": (_i, [C.POINTER(_ll), C.POINTER(_ll)]),
    "pl_malloc_device": (_i, [C.POINTER(_vp), _ll]),
    "pl_free_device": (_i, [_vp]),
    "pl_malloc_pinned": (_i, [C.POINTER(_vp), _ll]),
    "pl_free_pinned": (_i, [_vp]),
    "pl_ptr_location": (_i, [_vp, _pi]),
    "pl_stream_create": (_i, [C.POINTER(_vp)]),
    "pl_stream_destroy": (_i, [_vp]),
    "pl_stream_sync": (_i, [_vp]),
    "pl_stream_query": (_i, [_vp, _pi]),
    "pl_event_create": (_i, [C.POINTER(_vp), _i]),
    "pl_event_destroy": (_i, [_vp]),
    "pl_event_record": (_i, [_vp, _vp]),
    "pl_stream_wait_event": (_i, [_vp, _vp]),
    "pl_event_sync": (_i, [_vp]),
    "pl_event_query": (_i, [_vp, _pi]),
    "pl_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(_f)]),
    "pl_copy2d_async": (_i, [_vp, _l, _vp, _l, _l, _l, _i, _vp]),
    "pl_copy_async": (_i, [_vp, _vp, _ll, _vp]),
    "pl_copy": (_i, [_vp, _vp, _ll]),
    "pl_stream_shares_queue": (_i, [_vp, C.POINTER(_vp), _i, _pi]),
    "pl_memset_async": (_i, [_vp, _i, _ll, _vp]),
    "pl_sync_check": (_i, []),
    "pl_dgemm_tile": (_i, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _vp]),
    "pl_sgemm_tile": (_i, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l, _vp]),
    "pl_gemm_tile_workspace_bytes": (_l, [_l, _l, _l, _i]),
    "pl_gemm_fit_defaults": (None, [C.POINTER(gemm_fit)]),
    "pl_gemm_set_fit": (_i, [C.POINTER(gemm_fit)]),
    "pl_gemm_get_fit": (_i, [C.POINTER(gemm_fit)]),
    "pl_gemm_tile_choice": (_i, [_i, _c, _c, _l, _l, _l, _i, _l, _pi, _pi, _pi]),
    "pl_dgemm_tile_ws": (_i, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _vp, _l, _vp]),
    "pl_sgemm_tile_ws": (_i, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l, _vp, _l, _vp]),
    "pl_gemm_tile_alone_workspace_bytes": (_l, [_c, _c, _l, _l, _l, _i, _i]),
    "pl_dgemm_tile_alone": (_i, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _vp, _l, _vp]),
    "pl_sgemm_tile_alone": (_i, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l, _vp, _l, _vp]),
    "pl_gemm_tile_choice_alone": (_i, [_i, _c, _c, _l, _l, _l, _i, _l, _pi, _pi, _pi]),
    "pl_gemm_tile_cut_alone": (_i, [_i, _c, _c, _l, _l, _l, _i, _l, C.POINTER(_l), _pi]),
    "pl_gemm_tile_alone_us": (_d, [_i, _c, _c, _l, _l, _l, _i, _l]),
    "pl_dgemm_tile_padded": (_i, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _vp, _l, _i, _l, _l, _vp]),
    "pl_sgemm_tile_padded": (_i, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l, _vp, _l, _i, _l, _l, _vp]),
    "pl_dgemm_tile_split": (_i, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _vp, _l, _i, _vp]),
    "pl_sgemm_tile_split": (_i, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l, _vp, _l, _i, _vp]),
    "pl_dgeadd_tile": (_i, [_l, _l, _d, _vp, _l, _vp, _l, _vp, _l, _vp]),
    "pl_sgeadd_tile": (_i, [_l, _l, _f, _vp, _l, _vp, _l, _vp, _l, _vp]),
    "pl_daxpy": (_i, [_l, _d, _vp, _l, _vp, _l, _vp]),
    "pl_ddot_workspace_doubles": (_l, []),
    "pl_ddot": (_i, [_l, _vp, _l, _vp, _l, _vp, _i, _vp, _vp]),
    "pl_dgemv_workspace_doubles": (_ll, [_c, _l, _l]),
    "pl_dgemv": (_i, [_c, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _vp, _vp]),
    "pl_dgemv_noalloc_max_doubles": (_ll, []),
    "pl_dgemv_noalloc": (_i, [_c, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _vp]),
    "PARALiA_last_error": (C.c_char_p, []),
    "PARALiA_dgemm": (_i, [_c, _c, _l, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _l, _ll, C.POINTER(atc_info)]),
    "PARALiA_sgemm": (_i, [_c, _c, _l, _l, _l, _f, _vp, _l, _vp, _l, _f, _vp, _l, _l, _ll, C.POINTER(atc_info)]),
    "PARALiA_dgemv": (_i, [_c, _l, _l, _d, _vp, _l, _vp, _l, _d, _vp, _l, _l, _ll, C.POINTER(atc_info)]),
    "PARALiA_daxpy": (_i, [_l, _d, _vp, _l, _vp, _l, _l, C.POINTER(atc_info)]),
    "PARALiA_ddot": (_i, [_l, _vp, _l, _vp, _l, C.POINTER(_d), _l, C.POINTER(atc_info)]),
    "PARALiA_host_copy2d": (_i, [_vp, _l, _vp, _l, _l, _l, _i]),
    "PARALiA_dev_cache_free": (_i, [_i]),
    "PARALiA_runtime_stats": (_i, [C.POINTER(_l), C.POINTER(_l), C.POINTER(_ll), C.POINTER(_l)]),
    "PARALiA_runtime_reset": (_i, []),
    "PARALiA_stream_queues": (_i, [_pi, _pi]),
    "PARALiA_last_call_phases": (_i, [C.POINTER(_d)]),
    "PARALiA_runtime_shutdown": (_i, []),
    "PARALiA_trace_enable": (_i, [_i]),
    "PARALiA_trace_read": (_l, [C.POINTER(_d), _l]),
    "PARALiA_set_db_dir": (_i, [C.c_char_p]),
    "PARALiA_malloc": (_i, [C.POINTER(_vp), _ll, _i]),
    "PARALiA_free": (_i, [_vp, _i]),
    "PARALiA_vec_init_f64": (_i, [_vp, _ll, _i, _i]),
    "PARALiA_vec_init_f32": (_i, [_vp, _ll, _i, _i]),
    "PARALiA_test_equality_f64": (_i, [_vp, _vp, _ll]),
    "PARALiA_test_equality_f32": (_i, [_vp, _vp, _ll]),
    "PARALiA_heuristic_tile": (_l, [_l, _l, _l, C.POINTER(_d)]),
    "PARALiA_T_slowdowns": (_i, [_l, _l, _l, _l, C.POINTER(_d)]),
    "PARALiA_model_predict": (_d, [C.c_char_p, C.c_char_p, _i, _l, _l, _l, _c, _c, _pi, _l]),
    "PARALiA_autotune": (_i, [C.c_char_p, C.c_char_p, _l, _l, _l, _c, _c, _pi, _i, _l, _ll, C.POINTER(atc_info)]),
    "PARALiA_gemm_plan": (_l, [_l, _l, _l, _l, _i, _i, _i, _i, _i, _i, _l, _i, _pi, _l, C.POINTER(_l)]),
    "PARALiA_gemm_plan_simulate": (_d, [_l, _l, _l, _l, _i, _i, _i, _i, _i, _i, _l, _i, _d, _d, _d, _d, _d, _d, _d, _d, _pi,
                                        C.POINTER(_d)]),
}


def load(path=None):
    """Load libparalia.so and attach argument types.  Raises ParaliaError when it is not built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise ParaliaError("%s is missing: build it first (make -C %s, or __graft_entry__.build())" % (p, PKG_DIR))
    L = C.CDLL(p)
    for name, (res, args) in _SIGS.items():
        fn = getattr(L, name)  # AttributeError here means the library is stale
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = L
    return L


def lib():
    return load()


def check(rc, what="call"):
    if rc != 0:
        L = lib()
        msg = L.PARALiA_last_error().decode(errors="replace")
        hip = L.pl_last_error().decode(errors="replace")
        raise ParaliaError("%s failed with code %d: %s [hip: %s]" % (what, rc, msg, hip))


def plan_rows(M, N, K, T, a_remote=1, b_remote=1, c_remote=1, beta_zero=0, elem=8, exec_queues=2, pool_blocks=0,
              order_id=10000):
    """Static GEMM plan as a list of dicts plus the stats tuple."""
    L = lib()
    stats = (C.c_long * 6)()
    n = L.PARALiA_gemm_plan(M, N, K, T, a_remote, b_remote, c_remote, beta_zero, elem, exec_queues, pool_blocks, order_id,
                            None, 0, stats)
    if n < 0:
        raise ParaliaError(L.PARALiA_last_error().decode())
    buf = (C.c_int * (n * PL_PLAN_ROW))()
    L.PARALiA_gemm_plan(M, N, K, T, a_remote, b_remote, c_remote, beta_zero, elem, exec_queues, pool_blocks, order_id,
                        buf, n, stats)
    rows = []
    for i in range(n):
        r = buf[i * PL_PLAN_ROW:(i + 1) * PL_PLAN_ROW]
        rows.append(dict(kind=r[0], mi=r[1], ni=r[2], ki=r[3], stream=r[4], block=r[5], a_block=r[6], b_block=r[7],
                         beta_mode=r[8], waits=[w for w in r[10:10 + r[9]]], kn=r[10 + PL_PLAN_MAX_WAITS],
                         row0=r[11 + PL_PLAN_MAX_WAITS], rows=r[12 + PL_PLAN_MAX_WAITS], splits=r[13 + PL_PLAN_MAX_WAITS]))
    return rows, tuple(stats)
