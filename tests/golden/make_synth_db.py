"""Writes the synthetic autotuner database used by the host-logic tests (tests/golden/db_synth/Processed).

File formats are the reference's (Autotuner/src/GPUexec_lookup.cpp:79-82,311; CoModel.cpp:32-55):
  <Func>_lookup-table_dev-0.log   BLAS-3: TransA,TransB,M,N,K,t,W,J,err,n,bench   BLAS-1: T,t,W,J,err,n,bench
                                  BLAS-2 (GPUexec_lookup.cpp:196-198): TransA,M,N,t,W,J,err,n,bench
  Link-Stats_loc_dest-<to>_loc_src-<from>.log   Intercept / Coefficient / Slowdown([src]->[dst]) lines
Numbers are round on purpose so that tests can state expected predictions by hand:
  Dgemm NN tile time 1e-3 s at T=1024 scaling with T^3; H2D 0.5e-3 s and D2H 0.25e-3 s per 1024^2 fp64 tile;
  Dgemv N tile time 2e-5 s at T=1024 scaling with T^2 (T: 1.25 times that).
Also writes db_v100/, three real rows of the reference's own V100 logs re-cut into the Processed layout.
Run from the repository root: python tests/golden/make_synth_db.py
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def write(path, text):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write(text)


def synth():
    d = os.path.join(HERE, "db_synth", "Processed")
    scale = {("N", "N"): 1.0, ("N", "T"): 1.1, ("T", "N"): 1.2, ("T", "T"): 1.3}
    rows = []
    for T in (512, 1024, 2048, 4096):
        for (ta, tb), s in scale.items():
            t = 1e-3 * s * (T / 1024.0) ** 3
            rows.append("%s,%s,%d,%d,%d,%e,%e,%e,%e,%d,%e" % (ta, tb, T, T, T, t, 0.0, 0.0, t * 0.01, 100, 1.0))
    write(os.path.join(d, "Dgemm_lookup-table_dev-0.log"), "\n".join(rows) + "\n")
    rows = []
    for T in (512, 1024, 2048, 4096):
        for (ta, tb), s in scale.items():
            t = 0.5e-3 * s * (T / 1024.0) ** 3
            rows.append("%s,%s,%d,%d,%d,%e,%e,%e,%e,%d,%e" % (ta, tb, T, T, T, t, 0.0, 0.0, t * 0.01, 100, 1.0))
    write(os.path.join(d, "Sgemm_lookup-table_dev-0.log"), "\n".join(rows) + "\n")
    rows = []
    for T in (512, 1024, 2048, 4096):
        for ta, sc in (("N", 1.0), ("T", 1.25)):
            t = 2e-5 * sc * (T / 1024.0) ** 2
            rows.append("%s,%d,%d,%e,%e,%e,%e,%d,%e" % (ta, T, T, t, 0.0, 0.0, t * 0.01, 100, 1.0))
    write(os.path.join(d, "Dgemv_lookup-table_dev-0.log"), "\n".join(rows) + "\n")
    for func, per in (("Daxpy", 1e-4), ("Ddot", 0.8e-4)):
        rows = []
        for T in (1 << 16, 1 << 18, 1 << 20, 1 << 22):
            t = per * T / float(1 << 18)
            rows.append("%d,%e,%e,%e,%e,%d,%e" % (T, t, 0.0, 0.0, t * 0.01, 100, 1.0))
        write(os.path.join(d, "%s_lookup-table_dev-0.log" % func), "\n".join(rows) + "\n")
    tile = 1024 * 1024 * 8
    write(os.path.join(d, "Link-Stats_loc_dest-0_loc_src--1.log"),
          "Intercept: 0.0\nCoefficient: %.17e\nSlowdown([0]->[-1]): 1.25\n" % (0.5e-3 / tile))
    write(os.path.join(d, "Link-Stats_loc_dest--1_loc_src-0.log"),
          "Intercept: 0.0\nCoefficient: %.17e\nSlowdown([-1]->[0]): 1.5\n" % (0.25e-3 / tile))


def v100():
    # Rows 8, 16, 24 of the reference's
    # Benchmarking/Python_Scripts/CoCoPeLiA_plotters/results_2022/silver1/microbenchmarks/
    #   cublasDgemm_dev-0_TransA-N_TransB-N_1.1.log   (M,N,K, t, err, n, bench) and rows 8, 24 of
    #   CoCoMemcpy2DAsync_to-0_from--1_1.1.log        (dim,dim, t, err, n, t_bid, err, n, bench)
    # with the flag columns the reference's BenchToLookupTables.py prepends; W and J (absent in that log
    # generation) are written as 0.
    d = os.path.join(HERE, "db_v100", "Processed")
    write(os.path.join(d, "Dgemm_lookup-table_dev-0.log"),
          "N,N,2048,2048,2048,2.556160e-03,0.000000e+00,0.000000e+00,1.277293e-04,619,1.585487e+00\n"
          "N,N,4096,4096,4096,1.921535e-02,0.000000e+00,0.000000e+00,9.549759e-04,163,3.132950e+00\n"
          "N,N,8192,8192,8192,1.578847e-01,0.000000e+00,0.000000e+00,7.606750e-03,42,6.631360e+00\n")
    # two-point fit through (2048^2*8 B, 2.732534e-03 s) and (8192^2*8 B, 4.355426e-02 s); slowdown of the 2048
    # point under opposing traffic 3.130138e-03 / 2.732534e-03
    b0, t0, b1, t1 = 2048 * 2048 * 8, 2.732534e-03, 8192 * 8192 * 8, 4.355426e-02
    tb = (t1 - t0) / (b1 - b0)
    ti = abs(t0 - tb * b0)
    write(os.path.join(d, "Link-Stats_loc_dest-0_loc_src--1.log"),
          "Intercept: %.17e\nCoefficient: %.17e\nSlowdown([0]->[-1]): %.17e\n" % (ti, tb, 3.130138e-03 / 2.732534e-03))
    write(os.path.join(d, "Link-Stats_loc_dest--1_loc_src-0.log"),
          "Intercept: %.17e\nCoefficient: %.17e\nSlowdown([-1]->[0]): %.17e\n" % (ti, tb, 1.0))


if __name__ == "__main__":
    synth()
    v100()
