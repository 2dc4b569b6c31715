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
    """Digits the driver's validation reported: against OpenBLAS, or, on a machine without it, against the reference
    the driver computes itself (never "compared with nothing")."""
    m = re.search(r"Matching digits vs (OpenBLAS|long double samples|host reference): (\d+)", err)
    assert m is not None, err[-1500:]
    if m.group(1) != "OpenBLAS":
        assert "OpenBLAS absent" in err
    return int(m.group(2))


def test_dgemm_runner_validates_times_and_logs(run_program, bindir, tmp_path):
    err = run_driver(run_program, bindir, tmp_path, "dgemm_runner", "-1 -1 -1 -1 N T 1.2 1.1 1024 768 512 -1 -1 -1 -1")
    assert digits_of(err) >= 9
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
    assert digits_of(err) >= 9
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
    assert digits_of(err) >= 9 and "avg_t" in err
    err = run_driver(run_program, bindir, tmp_path, "ddot_runner", f"-1 -1 -1 -1 0.7 {n} 1 1 {loc}")
    m = re.search(r"(?:OpenBLAS cblas_ddot: .*|long double sum on the host) -> (\S+), PARALiA -> (\S+)", err)
    assert m is not None, err[-1500:]
    # uniform [-1, 1) vectors: |x||y| is about n / 3, the runner's own bound is 1e-13 of that
    assert abs(float(m.group(1).rstrip(",")) - float(m.group(2))) <= 1e-13 * n
    assert "avg_t" in err
    assert len(list(tmp_path.glob("CoCoPeLiaDaxpyRunner*.log"))) == 1 and len(list(tmp_path.glob("CoCoPeLiaDdotRunner*.log"))) == 1


def test_runners_validate_without_openblas(run_program, bindir, tmp_path):
    """PARALIA_OPENBLAS_LIB=none makes the drivers behave as on a machine without OpenBLAS: they must still validate,
    against references they compute themselves (sampled long double dot products for GEMM, full host references for
    the vector routines), and the CHECKLOG switch must refuse to repeat a configuration that is already in the log."""
    err = run_driver(run_program, bindir, tmp_path, "dgemm_runner", "-1 -1 -1 -1 T N 1.2 1.1 700 900 1100 -1 -1 -1 -1", PARALIA_OPENBLAS_LIB="none")
    assert "Matching digits vs long double samples" in err and digits_of(err) >= 9
    err = run_driver(run_program, bindir, tmp_path, "sgemm_runner", "-1 -1 -1 -1 N T 1.0 1.0 512 768 640 -1 -1 0 0", PARALIA_OPENBLAS_LIB="none")
    assert digits_of(err) >= 4
    err = run_driver(run_program, bindir, tmp_path, "daxpy_runner", "-1 -1 -1 -1 0.7 300000 2 -3 -1 -1 -1 -1", PARALIA_OPENBLAS_LIB="none")
    assert "Matching digits vs host reference" in err and digits_of(err) >= 9
    err = run_driver(run_program, bindir, tmp_path, "ddot_runner", "-1 -1 -1 -1 0.7 300000 1 1 -1 0 -1 0", PARALIA_OPENBLAS_LIB="none")
    assert "long double sum on the host" in err
    err = run_driver(run_program, bindir, tmp_path, "dgemv_runner", "-1 -1 -1 -1 T 1.2 1.1 1500 1000 1 1 -1 -1 -1 -1", PARALIA_OPENBLAS_LIB="none")
    assert "Matching digits vs host reference" in err and digits_of(err) >= 9
    # CHECKLOG: the dgemm configuration above is in the log now, a second run with the switch on stops before running
    env = dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path), PARALIA_CHECKLOG="1", PARALIA_SKIP_VALIDATION="1")
    r = run_program([os.path.join(bindir, "dgemm_runner")] + "-1 -1 -1 -1 T N 1.2 1.1 700 900 1100 -1 -1 -1 -1".split(), env, 120)
    assert r["rc"] == 1 and "found. Quiting" in r["stderr"]
    r = run_program([os.path.join(bindir, "dgemm_runner")] + "-1 -1 -1 -1 T N 1.2 1.1 700 900 1101 -1 -1 -1 -1".split(), env, 120)
    assert r["rc"] == 0, r["stderr"][-1500:]


@pytest.mark.parametrize("ta", ["N", "T"])
def test_dgemv_runner(run_program, bindir, tmp_path, ta):
    err = run_driver(run_program, bindir, tmp_path, "dgemv_runner", f"-1 -1 -1 -1 {ta} 1.2 1.1 3000 2000 1 1 -1 -1 -1 -1")
    assert digits_of(err) >= 9
    rows = rows_of(tmp_path, "CoCoPeLiaDgemvRunner_MI355X_*.log")
    assert len(rows) == 100 and rows[0][4] == ta      # 100 timed iterations below 20000 x 20000 (dgemv_runner.cpp:159-160)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("name", ["dgemm_tester", "sgemm_tester"])
def test_gemm_testers_full_sweep(run_program, bindir, tmp_path, name):
    """The reference testers' grid (squares, non-squares, 289 / 353 / 307, transposes, every residency mix) on views
    of 8192 x 8192 buffers, squares up to 8192 (69 cases, about 10 s); the program itself fails on any result with too few digits matching OpenBLAS."""
    r = run_program([os.path.join(bindir, name)], dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path)), 800)
    assert r["rc"] == 0, r["stderr"][-3000:]
    m = re.search(r"(\d+) cases, (\d+) failures", r["stderr"])
    assert m and int(m.group(1)) >= 60 and int(m.group(2)) == 0


def test_reference_call_shape_driver_runs_on_the_gpu(run_program, pkg, tmp_path):
    """The driver of tests/golden/reference_call_shapes.cpp (written with the reference drivers' call shapes, compiled
    against include/ only) makes its PARALiADgemm / PARALiA_dgemm calls on the GPU and logs one row."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.path.dirname(pkg.LIB_PATH)
    exe = str(tmp_path / "reference_call_shapes")
    r = run_program(["g++", "-O1", "-std=c++17", "-I", os.path.join(root, "include"), os.path.join(root, "tests", "golden", "reference_call_shapes.cpp"),
                     "-o", exe, "-L", libdir, "-lparalia", "-Wl,-rpath," + libdir, "-ldl", "-lpthread"], dict(os.environ), 300)
    assert r["rc"] == 0, r["stderr"][-2000:]
    r = run_program([exe, "gpu"], dict(os.environ, PARALIA_TESTLIBDIR=str(tmp_path)), 120)
    assert r["rc"] == 0, r["stderr"][-2000:]
    rows = rows_of(tmp_path, "CoCoPeLiaDgemmRunner_MI355X_*.log")
    assert len(rows) == 1 and len(rows[0]) == 18 and rows[0][4:6] == ["N", "T"]


def _table(path, key_cols):
    """Processed lookup table -> {key tuple: seconds}; the time is the column after the keys."""
    out = {}
    for line in open(path):
        parts = [p.strip() for p in line.strip().split(",")]
        if len(parts) > key_cols:
            out[tuple(parts[:key_cols])] = float(parts[key_cols])
    return out


def _link(path):
    vals = {}
    for line in open(path):
        k, _, v = line.partition(":")
        vals[k.strip().split("(")[0]] = float(v)
    return vals


@pytest.mark.timeout(900)
def test_deploy_tool_rebuilds_the_shipped_database(run_program, pkg, L, bindir, tmp_path):
    """The deploy-time pipeline (the reference's Deploy.in:14-18: microbenchmarks, then BenchToLookupTables.py.in:31-55
    and LinkPreprocessing.py.in:44-61) as one run of bin/paralia_deploy --quick into a scratch directory.  The tables it
    writes must load through the library's own parsers, and what it measures must agree with the database the
    library ships (paralia-framework_amd/db/mi355x) within a band that covers box-to-box differences."""
    import ctypes as C
    db = tmp_path / "db"
    r = run_program([os.path.join(bindir, "paralia_deploy"), str(db), "--quick"], dict(os.environ), 800)
    assert r["rc"] == 0, r["stderr"][-3000:]
    shipped = os.path.join(os.path.dirname(pkg.LIB_PATH), "..", "db", "mi355x", "Processed")
    fresh = str(db / "Processed")
    names = ["Dgemm_lookup-table_dev-0.log", "Sgemm_lookup-table_dev-0.log", "Dgemv_lookup-table_dev-0.log", "Daxpy_lookup-table_dev-0.log",
             "Ddot_lookup-table_dev-0.log", "Link-Stats_loc_dest-0_loc_src--1.log", "Link-Stats_loc_dest--1_loc_src-0.log"]
    for n in names:
        assert os.path.getsize(os.path.join(fresh, n)) > 0, n
    assert len(list((db / "Benchmark-Results").iterdir())) >= 16      # the raw logs of every sweep

    def close(a, b, band, what):
        assert abs(a - b) <= band * b, "%s: regenerated %.4e vs shipped %.4e" % (what, a, b)

    # link model: bytes -> seconds slope of both directions within 10 %, slowdown factors within 0.15
    for n in names[5:]:
        a, b = _link(os.path.join(fresh, n)), _link(os.path.join(shipped, n))
        close(a["Coefficient"], b["Coefficient"], 0.10, n + " coefficient")
        assert abs(a["Slowdown"] - b["Slowdown"]) <= 0.15, (n, a, b)
        assert 0 <= a["Intercept"] < 2e-4
    # tile kernels at the sizes the scheduler uses
    for n, keys, band in ((names[0], [("N", "N", "2048", "2048", "2048"), ("N", "T", "4096", "4096", "4096"), ("T", "N", "1024", "1024", "1024")], 0.10),
                          (names[1], [("N", "T", "4096", "4096", "4096"), ("N", "N", "2048", "2048", "2048")], 0.10)):
        a, b = _table(os.path.join(fresh, n), 5), _table(os.path.join(shipped, n), 5)
        for k in keys:
            close(a[k], b[k], band, n + str(k))
    # lone-launch times (a tile launch with the device to itself): never shorter than the filled-device time per launch
    # beyond noise, and for 2048^3 fp64 (one workgroup per compute unit) longer by the 5 - 20 % the shipped table shows
    for func in ("Dgemm", "Sgemm"):
        lone = _table(os.path.join(fresh, func + "_lone-launch_dev-0.log"), 3)
        filled = _table(os.path.join(fresh, func + "_lookup-table_dev-0.log"), 5)
        assert len(lone) == len(filled)
        for k, t in lone.items():
            assert t > 0.9 * filled[k + (k[2], k[2])], (func, k, t)
    lone = _table(os.path.join(fresh, "Dgemm_lone-launch_dev-0.log"), 3)
    lone_shipped = _table(os.path.join(shipped, "Dgemm_lone-launch_dev-0.log"), 3)
    close(lone[("N", "N", "2048")], lone_shipped[("N", "N", "2048")], 0.10, "lone 2048^3 fp64 launch")
    ratio = lone[("N", "N", "2048")] / _table(os.path.join(fresh, names[0]), 5)[("N", "N", "2048", "2048", "2048")]
    assert 1.03 < ratio < 1.25, ratio
    # the power-state transient of the tile kernels: present on this device, its constants of the shipped file's order
    def transient(path):
        return {k.strip(): float(v) for k, v in (line.split(":") for line in open(path))}
    tr, tr_shipped = transient(os.path.join(fresh, "Power-transient_dev-0.log")), transient(os.path.join(shipped, "Power-transient_dev-0.log"))
    # (the two time constants come out of a fit to a curve that is only roughly exponential: wide bands)
    assert 0.05 < tr["Amplitude"] < 0.6, tr
    assert 0.5 * tr_shipped["Amplitude"] < tr["Amplitude"] < 2.0 * tr_shipped["Amplitude"], (tr, tr_shipped)
    for k in ("Recovery", "Idle"):
        assert 0.25 * tr_shipped[k] < tr[k] < 4.0 * tr_shipped[k], (k, tr, tr_shipped)
    # the constants of the launcher's cost model and of the simulator (Kernel-fit_dev-0.log): per-k costs within 10 % of
    # the shipped fit, gains within 0.03, fixed costs (intercepts of a line through three to five points, a few
    # microseconds of tens) and the scale-add rate within a wider band; every name the shipped file has is there
    def fit(path):
        return {k.strip(): float(v) for k, v in (line.split(":") for line in open(path) if not line.startswith("#") and ":" in line)}
    kf, kf_shipped = fit(os.path.join(fresh, "Kernel-fit_dev-0.log")), fit(os.path.join(shipped, "Kernel-fit_dev-0.log"))
    assert set(kf) == set(kf_shipped), set(kf) ^ set(kf_shipped)
    for k in ("lone_us_per_k_f64", "lone_us_per_k_f32", "f32_small_us_per_k"):
        close(kf[k], kf_shipped[k], 0.10, k)
    for k in kf:
        if "gain" in k:
            assert abs(kf[k] - kf_shipped[k]) <= 0.03, (k, kf[k], kf_shipped[k])
        elif "fixed_us" in k:
            assert abs(kf[k] - kf_shipped[k]) <= max(4.0, 0.25 * kf_shipped[k]), (k, kf[k], kf_shipped[k])
        elif k.startswith("merge_saving_us_f32"):
            # 2 % of the difference of two 30 ms timings (the median of five): a few microseconds either way
            assert 0.0 <= kf[k] <= 30.0 and abs(kf[k] - kf_shipped[k]) <= 8.0, (k, kf[k], kf_shipped[k])
    # (a difference of two launch times of a millisecond each, as a share of a round)
    for k in ("edge_rounds_small", "edge_rounds_large"):
        assert 0.03 <= kf[k] <= 0.6 and abs(kf[k] - kf_shipped[k]) <= 0.10, (k, kf[k], kf_shipped[k])
    assert 0.5 * kf_shipped["lone_fixed_k"] < kf["lone_fixed_k"] < 2.0 * kf_shipped["lone_fixed_k"]
    assert 1.0 < kf["splitk_launch_us"] < 10.0 and 0 <= kf["slab_fixed_us"] < 6.0
    for k in ("pass_bytes_per_us", "geadd_bytes_per_s"):
        assert 0.5 * kf_shipped[k] < kf[k] < 2.0 * kf_shipped[k], (k, kf[k], kf_shipped[k])
    # matrix-vector and vector kernels take 40 - 80 us at the largest sizes of the quick sweep: launch and
    # synchronisation are a visible part of that, and working sets of 128 - 384 MiB sit partly inside the memory-side
    # cache, so these differ more between machines than the millisecond-scale GEMM tiles: a wider band
    a, b = _table(os.path.join(fresh, names[2]), 3), _table(os.path.join(shipped, names[2]), 3)
    for k in (("N", "4096", "4096"), ("T", "4096", "4096")):
        close(a[k], b[k], 0.30, names[2] + str(k))
    for n in names[3:5]:
        a, b = _table(os.path.join(fresh, n), 1), _table(os.path.join(shipped, n), 1)
        close(a[(str(1 << 24),)], b[(str(1 << 24),)], 0.30, n)
    # and through the library's own loaders: the autotuner prices the headline problem from the fresh tables within
    # 10 % of what it predicts from the shipped ones (same preset tile)
    loc = (C.c_int * 3)(-1, -1, -1)
    preds = []
    for d in (str(db), os.path.join(os.path.dirname(pkg.LIB_PATH), "..", "db", "mi355x")):
        info = pkg.atc_info()
        pkg.check(L.PARALiA_autotune(d.encode(), b"Dgemm", 16384, 16384, 16384, b"N", b"N", loc, 1, 2048, 0, C.byref(info)), "autotune")
        assert info.has_db == 1 and info.T == 2048
        preds.append(info.pred_t)
    L.PARALiA_set_db_dir(None)
    close(preds[0], preds[1], 0.10, "predicted seconds for dgemm 16384^3")
    # the loaders handed the launcher the fit of the database read last (the shipped one)
    from paralia_framework_amd import binding
    got = binding.gemm_fit()
    pkg.check(L.pl_gemm_get_fit(C.byref(got)), "get fit")
    assert abs(got.lone_us_per_k[0] - kf_shipped["lone_us_per_k_f64"]) < 1e-9 and abs(got.f32_large_gain[1] - kf_shipped["f32_large_gain_NT"]) < 1e-9
    assert abs(got.edge_rounds[0] - kf_shipped["edge_rounds_small"]) < 1e-9 and abs(got.edge_rounds[1] - kf_shipped["edge_rounds_large"]) < 1e-9
