"""The C ABI: the library loads, exports every symbol include/paralia_hip.h declares, and its argument checks
answer with status codes before anything touches a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "paralia_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:pl_|PARALiA_)[A-Za-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(pkg, L):
    names = declared_symbols()
    assert len(names) >= 55
    raw = C.CDLL(pkg.LIB_PATH)
    missing = [n for n in names if not hasattr(raw, n)]
    assert not missing, missing
    # and the Python face declares a signature for each of them
    from_binding = set(pkg.binding._SIGS)
    assert set(names) <= from_binding, sorted(set(names) - from_binding)


def test_cxx_api_is_exported(pkg):
    import subprocess
    out = subprocess.run(["nm", "-DC", pkg.LIB_PATH], capture_output=True, text=True, check=True).stdout
    for sym in ("PARALiADgemm(", "PARALiADgemmControled(", "PARALiASgemm(", "PARALiASgemmControled(", "PARALiADaxpy(",
                "PARALiADaxpyControled(", "PARALiADdot(", "PARALiADdotControled(", "PARALiADevCacheFree(", "CoCoMalloc(",
                "CoCoFree(", "CoCoMemcpy(", "CoCoSyncCheckErr(", "Dtest_equality(", "Stest_equality(", "csecond(",
                "ATC::print_csv(", "ATC::autotune_problem("):
        assert sym in out, sym


def test_kernel_launchers_validate_before_launching(L):
    # invalid arguments are refused on the host: no device is needed to see the status code
    assert L.pl_dgemm_tile(b"X", b"N", 4, 4, 4, 1.0, None, 4, None, 4, 0.0, None, 4, None) == 1
    assert L.pl_dgemm_tile(b"N", b"N", -1, 4, 4, 1.0, None, 4, None, 4, 0.0, None, 4, None) == 2
    assert L.pl_dgemm_tile(b"N", b"N", 8, 4, 4, 1.0, None, 4, None, 4, 0.0, None, 8, None) == 3   # lda < M
    assert L.pl_dgemm_tile(b"T", b"N", 8, 4, 16, 1.0, None, 8, None, 16, 0.0, None, 8, None) == 3  # lda < K when transposed
    assert L.pl_sgemm_tile(b"N", b"T", 8, 4, 4, 1.0, None, 8, None, 2, 0.0, None, 8, None) == 3    # ldb < N when transposed
    assert L.pl_dgemm_tile(b"N", b"N", 0, 4, 4, 1.0, None, 1, None, 4, 0.0, None, 1, None) == 0    # empty: nothing to do
    assert L.pl_dgemm_tile(b"N", b"N", 4, 4, 4, 1.0, None, 4, None, 4, 0.0, None, 4, None) == 5    # null operands
    assert L.pl_daxpy(0, 1.0, None, 1, None, 1, None) == 0
    assert L.pl_daxpy(10, 0.0, None, 1, None, 1, None) == 0    # alpha == 0: quick return, y untouched
    assert L.pl_daxpy(10, 1.0, None, 1, None, 1, None) == 5
    assert L.pl_dgeadd_tile(8, 8, 1.0, None, 4, None, 8, None, 8, None) == 5
    assert L.pl_ddot_workspace_doubles() >= 1024


def test_csv_row_round_trip(pkg, L, tmp_path):
    """The runner log row (reference testing.cpp:420-428): 'T,units,dev_token,cache, TransA,TransB,alpha,beta,M,N,K,
    Aloc,Bloc,Cloc,Coutloc, t,pred_t,pred_J'."""
    row = "%s, %c,%c,%.5lf,%.5lf,%zu,%zu,%zu,%d,%d,%d,%d, %e,%e,%e\n"
    line = "2048,1,1,0, N,N,1.00000,0.00000,16384,16384,16384,-1,-1,-1,-1, 1.300000e-01,1.250000e-01,-1.000000e+00\n"
    parts = [p.strip() for p in line.split(",")]
    assert len(parts) == 18 and parts[0] == "2048" and parts[4] == "N" and float(parts[15]) == 0.13


def test_predictor_driver_emits_a_runner_row(pkg, tmp_path):
    """dgemm_predictor needs no GPU: it parses the reference's 15 driver arguments (testing.cpp:273-329), autotunes and
    appends one row in the runner log format (testing.cpp:424) whose first four columns are T, unit count, unit token
    and cache limit (ATC::print_csv)."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(pkg.LIB_PATH), "..", "bin", "dgemm_predictor")
    if not os.path.exists(exe):
        pytest.skip("driver executables not built")
    env = dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path))
    args = "-1 -1 -1 -1 N N 1.0 0.0 16384 16384 16384 -1 -1 -1 -1".split()
    run = subprocess.run([exe] + args, env=env, capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
    logs = list(tmp_path.glob("CoCoPeLiaDgemmPredictor_MI355X_*.log"))
    assert len(logs) == 1
    parts = [p.strip() for p in logs[0].read_text().strip().split(",")]
    assert len(parts) == 18
    assert parts[:4] == ["2048", "1", "1", "0"] and parts[4:6] == ["N", "N"]
    assert [int(p) for p in parts[8:15]] == [16384, 16384, 16384, -1, -1, -1, -1]
    assert 0.1 < float(parts[16]) < 0.15            # predicted seconds for 16384^3 streamed from the host
    assert "T =  2048" in run.stderr and "pipeline-model" in run.stderr
    # a preset tile goes to the other log and is kept
    run = subprocess.run([exe] + "1 1 4096 -1 N N 1.0 0.0 16384 16384 16384 -1 -1 -1 -1".split(), env=env, capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
    row = next(tmp_path.glob("CoCoPeLiaDgemmPredictor_predefined_vals_MI355X_*.log")).read_text()
    assert row.startswith("4096,1,1,")
    # wrong argument count is the reference's usage error
    run = subprocess.run([exe, "1", "2"], env=env, capture_output=True, text=True, timeout=60)
    assert run.returncode != 0 and "Incorrect input arguments" in run.stderr


def test_split_k_workspace_sizing(L):
    """Host-side decision only: products whose 128 x 128 tiles cover the chip are not split; small or skinny ones ask
    for whole M x N slices, at least two, with chunks of at least 128 in k."""
    assert L.pl_gemm_tile_workspace_bytes(16384, 16384, 16384, 8) == 0
    assert L.pl_gemm_tile_workspace_bytes(2048, 2048, 2048, 8) == 0      # 256 tiles: one per compute unit
    assert L.pl_gemm_tile_workspace_bytes(1024, 1024, 128, 8) == 0       # K too short to split
    assert L.pl_gemm_tile_workspace_bytes(0, 10, 10, 8) == 0 and L.pl_gemm_tile_workspace_bytes(10, 10, 10, 3) == 0
    for M, N, K, esz in ((1024, 1024, 1024, 8), (1024, 1024, 1024, 4), (128, 128, 65536, 8), (300, 200, 777, 8)):
        b = L.pl_gemm_tile_workspace_bytes(M, N, K, esz)
        assert b > 0 and b % (M * N * esz) == 0
        s = b // (M * N * esz)
        assert 2 <= s <= 64 and K / s >= 112 and b <= 256 << 20
    assert L.pl_gemm_tile_workspace_bytes(1024, 1024, 1024, 8) == 4 * 1024 * 1024 * 8


def test_runner_row_is_readable_by_the_reference_plotters(pkg, tmp_path):
    """The reference's plotting scripts read runner logs with pandas: no header, skipinitialspace, 18 columns of which
    0-5, 8-13 and 15-17 are used (T, units, unit token, cache / ratio, TransA, TransB, M, N, K, the three locations and
    three timings: Benchmarking/Python_Scripts/CoCoPeLiA_plotters/input_parsing.py:41-47).  A row written by the
    predictor driver must come through that call with the right types."""
    import os
    import subprocess
    pd = pytest.importorskip("pandas")
    exe = os.path.join(os.path.dirname(pkg.LIB_PATH), "..", "bin", "dgemm_predictor")
    if not os.path.exists(exe):
        pytest.skip("driver executables not built")
    env = dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path))
    for args in ("1 1 2048 -1 N T 1.0 0.5 8192 4096 2048 -1 0 -1 -1", "1 1 1024 -1 T N 1.0 0.5 4096 4096 4096 -1 -1 -1 -1"):
        run = subprocess.run([exe] + args.split(), env=env, capture_output=True, text=True, timeout=120)
        assert run.returncode == 0, run.stderr
    log = next(tmp_path.glob("CoCoPeLiaDgemmPredictor_predefined_vals_MI355X_*.log"))
    names = ["T", "dev_num", "dev_ids_token", "cpu_ratio", "TransA", "TransB", "M", "N", "K", "Aloc", "Bloc", "Cloc", "t0", "t1", "t2"]
    df = pd.read_csv(log, header=None, skipinitialspace=True, names=names, usecols=[0, 1, 2, 3, 4, 5, 8, 9, 10, 11, 12, 13, 15, 16, 17],
                     dtype={"T": int, "dev_num": int, "dev_ids_token": int, "TransA": str, "TransB": str, "M": int, "N": int, "K": int,
                            "Aloc": int, "Bloc": int, "Cloc": int, "t0": float, "t1": float, "t2": float})
    assert len(df) == 2
    assert list(df["T"]) == [2048, 1024] and list(df["TransA"]) == ["N", "T"] and list(df["TransB"]) == ["T", "N"]
    assert list(df["M"]) == [8192, 4096] and list(df["N"]) == [4096, 4096] and list(df["K"]) == [2048, 4096]
    assert list(df["Bloc"]) == [0, -1] and (df["t1"] > 0).all()


def test_driver_written_against_the_reference_call_shapes_compiles_and_links(pkg, tmp_path):
    """tests/golden/reference_call_shapes.cpp uses the helper surface the way the reference's drivers do (six-argument
    TransposeTranslate with the caller's own operation enums, CoCoMalloc / CoCoVecInit / CoCoMemcpy, PARALiADgemm and its
    Controled twin, CheckLogLvl3 / StoreLogLvl3 with TESTLIBDIR, CoCoImplementationPrint() and VERSION).  It must compile
    against include/ alone and link libparalia.so; its host mode (no GPU call) must run and leave one 18-column row."""
    import subprocess
    src = os.path.join(ROOT, "tests", "golden", "reference_call_shapes.cpp")
    exe = str(tmp_path / "reference_call_shapes")
    libdir = os.path.dirname(pkg.LIB_PATH)
    cmd = ["g++", "-O1", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "include"), src, "-o", exe, "-L", libdir, "-lparalia",
           "-Wl,-rpath," + libdir, "-ldl", "-lpthread"]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-3000:]
    env = dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path))
    run = subprocess.run([exe, "host"], env=env, capture_output=True, text=True, timeout=60)
    assert run.returncode == 0, (run.returncode, run.stderr[-2000:])
    log = next(tmp_path.glob("CoCoPeLiaDgemmRunner_MI355X_*.log"))
    parts = [p.strip() for p in log.read_text().strip().split(",")]
    assert len(parts) == 18 and parts[:6] == ["128", "1", "1", "0", "N", "T"] and [int(p) for p in parts[8:11]] == [300, 200, 100]
    # the row is in the log now: the CHECKLOG helper refuses to repeat the configuration once it is given the
    # returned controller (exit status 1, as in the reference)
    probe = tmp_path / "probe.cpp"
    probe.write_text('#include "Testing.hpp"\nint main() { ATC c; c.T = 128; c.active_unit_num = 1; c.active_unit_id_list[0] = 0;\n'
                     ' CheckLogLvl3("%s", &c, \'N\', \'T\', 1.2, 1.1, 300, 200, 100, -1, -1, -1, -1); return 0; }\n' % log)
    exe2 = str(tmp_path / "probe")
    run = subprocess.run(["g++", "-std=c++17", "-I", os.path.join(ROOT, "include"), str(probe), "-o", exe2, "-L", libdir, "-lparalia",
                          "-Wl,-rpath," + libdir, "-ldl", "-lpthread"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-3000:]
    run = subprocess.run([exe2], capture_output=True, text=True, timeout=60)
    assert run.returncode == 1 and "found. Quiting" in run.stderr
