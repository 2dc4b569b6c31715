"""The benchmark drivers on the GPU (the counterpart of the reference's Benchmarking/CuCuBLAS/src/PARALia programs):
argv order of testing.cpp:215-329, validation against OpenBLAS, the timing protocol of dgemm_runner.cpp:121-151 and
the CSV rows of testing.cpp:420-428.  Sizes are small: this checks the programs, the full sizes are timed elsewhere."""
import os
import re

import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def bindir(pkg):
    d = os.path.join(os.path.dirname(pkg.LIB_PATH), "..", "bin")
    if not os.path.exists(os.path.join(d, "dgemm_runner")):
        pytest.skip("driver executables not built")
    return d


def run_driver(run_program, bindir, tmp_path, name, args, timeout=300, **extra_env):
    env = dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path), **extra_env)
    print("driver", name, args, flush=True)
    r = run_program([os.path.join(bindir, name)] + args.split(), env, timeout)
    assert r["rc"] == 0, r["stderr"][-2000:]
    return r["stderr"]


def rows_of(tmp_path, pattern):
    logs = list(tmp_path.glob(pattern))
    assert len(logs) == 1, [p.name for p in tmp_path.iterdir()]
    return [[c.strip() for c in line.split(",")] for line in logs[0].read_text().strip().splitlines()]


def digits_of(err):
    m = re.search(r"Matching digits vs OpenBLAS: (\d+)", err)
    if m is None:
        assert "OpenBLAS absent" in err
        return None
    return int(m.group(1))


def test_dgemm_runner_validates_times_and_logs(run_program, bindir, tmp_path):
    err = run_driver(run_program, bindir, tmp_path, "dgemm_runner", "-1 -1 -1 -1 N T 1.2 1.1 1024 768 512 -1 -1 -1 -1")
    d = digits_of(err)
    assert d is None or d >= 9
    for key in ("first_it_t", "avg_t", "min_t", "max_t", "predicted_t"):
        assert key in err
    rows = rows_of(tmp_path, "CoCoPeLiaDgemmRunner_MI355X_*.log")
    assert len(rows) == 10 and all(len(r) == 18 for r in rows)          # ten timed iterations, one row each
    r = rows[0]
    assert int(r[0]) > 0 and r[1:4] == ["1", "1", "0"] and r[4:6] == ["N", "T"]
    assert float(r[6]) == 1.2 and float(r[7]) == 1.1 and [int(x) for x in r[8:15]] == [1024, 768, 512, -1, -1, -1, -1]
    assert 0 < float(r[15]) < 1.0 and float(r[16]) > 0


def test_dgemm_runner_controlled_tile_and_pool_limit(run_program, bindir, tmp_path):
    """Preset T = 256 and a block pool of 8 tiles (the ...Controled entry point): the other log file, first columns
    as given."""
    limit = 8 * 256 * 256 * 8
    err = run_driver(run_program, bindir, tmp_path, "dgemm_runner", f"1 1 256 {limit} N N 1.0 0.5 1024 1024 1024 -1 -1 -1 -1")
    d = digits_of(err)
    assert d is None or d >= 9
    rows = rows_of(tmp_path, "CoCoPeLiaDgemmRunner_predefined_vals_MI355X_*.log")
    assert len(rows) == 10 and rows[0][:4] == ["256", "1", "1", str(limit)]
    assert "selected by user" in err


def test_dgemm_runner_rejects_bad_arguments(run_program, bindir, tmp_path):
    env = dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path))
    r = run_program([os.path.join(bindir, "dgemm_runner"), "1", "2"], env, 60)
    assert r["rc"] != 0 and "Incorrect input arguments" in r["stderr"]
    r = run_program([os.path.join(bindir, "dgemm_runner")] + "1 1 4096 -1 N N 1.0 0.5 1024 1024 1024 -1 -1 -1 -1".split(), env, 60)
    assert r["rc"] != 0 and "bigger than problem dim" in r["stderr"]


@pytest.mark.parametrize("loc", ["0 0 0 0", "-1 -1 -1 -1", "-2 -2 -2 -2"])
def test_blas1_runners(run_program, bindir, tmp_path, loc):
    n = 1 << 22
    err = run_driver(run_program, bindir, tmp_path, "daxpy_runner", f"-1 -1 -1 -1 0.7 {n} 1 1 {loc}")
    d = digits_of(err)
    assert (d is None or d >= 9) and "avg_t" in err
    err = run_driver(run_program, bindir, tmp_path, "ddot_runner", f"-1 -1 -1 -1 0.7 {n} 1 1 {loc}")
    m = re.search(r"OpenBLAS cblas_ddot: .* -> (\S+), PARALiA -> (\S+)", err)
    if m is None:
        assert "OpenBLAS absent" in err
    else:   # uniform [-1, 1) vectors: |x||y| is about n / 3, the runner's own bound is 1e-13 of that
        assert abs(float(m.group(1)) - float(m.group(2))) <= 1e-13 * n
    assert "avg_t" in err
    assert len(list(tmp_path.glob("CoCoPeLiaDaxpyRunner*.log"))) == 1 and len(list(tmp_path.glob("CoCoPeLiaDdotRunner*.log"))) == 1


@pytest.mark.parametrize("ta", ["N", "T"])
def test_dgemv_runner(run_program, bindir, tmp_path, ta):
    err = run_driver(run_program, bindir, tmp_path, "dgemv_runner", f"-1 -1 -1 -1 {ta} 1.2 1.1 3000 2000 1 1 -1 -1 -1 -1")
    d = digits_of(err)
    assert d is None or d >= 9
    rows = rows_of(tmp_path, "CoCoPeLiaDgemvRunner_MI355X_*.log")
    assert len(rows) == 100 and rows[0][4] == ta      # 100 timed iterations below 20000 x 20000 (dgemv_runner.cpp:159-160)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("name", ["dgemm_tester", "sgemm_tester"])
def test_gemm_testers_full_sweep(run_program, bindir, tmp_path, name):
    """The reference testers' grid (squares, non-squares, 289 / 353 / 307, transposes, every residency mix) on views
    of 8192 x 8192 buffers, squares up to 8192 (69 cases, about 10 s); the program itself fails on any result with too few digits matching OpenBLAS."""
    r = run_program([os.path.join(bindir, name)], dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path)), 800)
    if r["rc"] == 2 and "OpenBLAS not found" in r["stderr"]:
        pytest.skip("no OpenBLAS on this machine")
    assert r["rc"] == 0, r["stderr"][-3000:]
    m = re.search(r"(\d+) cases, (\d+) failures", r["stderr"])
    assert m and int(m.group(1)) >= 60 and int(m.group(2)) == 0
