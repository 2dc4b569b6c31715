#!/usr/bin/env python3
"""Benchmark of the PARALiA hot path on one MI355X.

One "step" is one PARALiADgemm call, M = N = K = 16384, fp64, column-major, no transpose, alpha = 1, beta = 0
(BASELINE.json config 3), with the three operands already resident in HBM when the timed region starts: `value`
is 2*M*N*K / (mean wall time of a step).  The same JSON line also carries
  * host_operands : the same problem with A, B, C in pinned host memory, tiles streamed over PCIe (the configuration
                    the reference metric is quoted on), with its min(MFMA, PCIe) roofline;
  * daxpy_device  : daxpy N = 2^28 on device-resident vectors (config 2), GB/s and fraction of HBM peak;
  * roofline      : the dominant kernel (fp64 MFMA tile GEMM), timed with HIP events on the stream it is launched on;
  * cpu_baseline  : OpenBLAS cblas_dgemm on the host cores for a bounded slice of the same problem.
Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import ctypes as C
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

FP64_MFMA_PEAK = 78.6e12   # MI355X dense FP64 matrix peak, FLOP/s
HBM_PEAK = 8.0e12          # MI355X HBM3E peak, B/s
# HBM bytes of one 16384^3 launch of the tile kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a
# daxpy of known size: FETCH_SIZE 50,324,042 KiB x 2.0 + WRITE_SIZE 2,097,152 KiB x 1.0
# (profiles/dgemm_16384_daxpy_2p28_pmc_hbm_traffic.txt).
GEMM_TRAFFIC_BYTES = 1.0521e11


def load_package():
    name = "paralia_framework_amd"
    init = os.path.join(ROOT, "paralia-framework_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location(name, init, submodule_search_locations=[os.path.dirname(init)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--size", type=int, default=16384, help="M = N = K (default: the benchmark configuration)")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-host", action="store_true")
    ap.add_argument("--no-other-configs", dest="other_configs", action="store_false",
                    help="skip the streamed sgemm 32768^3 and dgemm 40000 x 40000 x 2048 extras (about 40 s)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="launch one daxpy (N=2^28: 4 GiB read, 2 GiB written) and one tile GEMM of --size, nothing else; "
                         "for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build drives one GPU; run with --gpus 1 (multi-GPU sharding is a design note only)")

    import numpy as np
    from gpu_util import Buf
    pkg = load_package()
    if not os.path.exists(pkg.LIB_PATH):
        pkg.build_library()
    L = pkg.load()
    n = args.size
    flops = 2.0 * n * n * n
    name = C.create_string_buffer(256)
    pkg.check(L.pl_device_name(0, name, 256), "device name")

    def stream():
        s = C.c_void_p()
        pkg.check(L.pl_stream_create(C.byref(s)), "stream")
        return s

    def event():
        e = C.c_void_p()
        pkg.check(L.pl_event_create(C.byref(e), 1), "event")
        return e

    if args.pmc_probe:
        m = 1 << 28
        dx, dy, dz = (Buf(pkg, max(m, n * n), np.float64, 0) for _ in range(3))
        for b, seed in ((dx, 0), (dy, 1)):
            pkg.check(L.PARALiA_vec_init_f64(b.ptr, b.n, seed, 0), "vec init")
        pkg.check(L.pl_daxpy(m, 0.7, dx.ptr, 1, dz.ptr, 1, None), "daxpy")
        pkg.check(L.pl_device_sync(), "sync")
        pkg.check(L.pl_dgemm_tile(b"N", b"N", n, n, n, 1.0, dx.ptr, n, dy.ptr, n, 0.0, dz.ptr, n, None), "tile")
        pkg.check(L.pl_device_sync(), "sync")
        print(json.dumps({"pmc_probe": True, "daxpy_n": m, "gemm_n": n}))
        return

    # ------------------------------------------------------------------ inputs (seeded, uniform [-1, 1))
    hA, hB, hC = (Buf(pkg, n * n, np.float64, -1) for _ in range(3))
    for b, seed in ((hA, 0), (hB, 1), (hC, 2)):
        pkg.check(L.PARALiA_vec_init_f64(b.ptr, n * n, seed, -1), "vec init")
    dA, dB, dC = (Buf(pkg, n * n, np.float64, 0) for _ in range(3))
    pkg.check(L.pl_copy(dA.ptr, hA.ptr, hA.nbytes), "copy")
    pkg.check(L.pl_copy(dB.ptr, hB.ptr, hB.nbytes), "copy")
    pkg.check(L.pl_copy(dC.ptr, hC.ptr, hC.nbytes), "copy")

    def step_device():
        pkg.check(L.PARALiA_dgemm(b"N", b"N", n, n, n, 1.0, dA.ptr, n, dB.ptr, n, 0.0, dC.ptr, n, -1, 0, None), "PARALiA_dgemm")

    # ------------------------------------------------------------------ value: device-resident PARALiADgemm
    for _ in range(args.warmup):
        step_device()
    pkg.check(L.pl_device_sync(), "sync")
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_device()
    pkg.check(L.pl_device_sync(), "sync")
    t_step = (time.perf_counter() - t0) / args.steps

    # parity of what was just timed: (A*B) v against A*(B*v), O(n^2) on the CPU
    v = np.linspace(-1.0, 1.0, n)
    Am, Bm = hA.host_view().reshape(n, n).T, hB.host_view().reshape(n, n).T
    got = dC.get().reshape(n, n).T @ v
    expect = Am @ (Bm @ v)
    parity = float(np.linalg.norm(got - expect) / (np.linalg.norm(Am) * np.linalg.norm(Bm) * np.linalg.norm(v)))

    # ------------------------------------------------------------------ roofline: the tile kernel under HIP events
    s = stream()
    e0, e1 = event(), event()
    pkg.check(L.pl_dgemm_tile(b"N", b"N", n, n, n, 1.0, dA.ptr, n, dB.ptr, n, 0.0, dC.ptr, n, s), "tile")
    pkg.check(L.pl_stream_sync(s), "sync")
    reps = max(3, min(args.steps, 10))
    pkg.check(L.pl_event_record(e0, s), "record")
    for _ in range(reps):
        pkg.check(L.pl_dgemm_tile(b"N", b"N", n, n, n, 1.0, dA.ptr, n, dB.ptr, n, 0.0, dC.ptr, n, s), "tile")
    pkg.check(L.pl_event_record(e1, s), "record")
    pkg.check(L.pl_stream_sync(s), "sync")
    ms = C.c_float()
    pkg.check(L.pl_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
    t_kernel = ms.value / reps / 1e3
    roofline = {"bound": "mfma", "kernel": "plk::gemm_kernel<double,false,true,128,128,16> (fp64 NN tile GEMM), one launch of %d^3" % n,
                "achieved": flops / t_kernel / 1e12, "peak": FP64_MFMA_PEAK / 1e12, "unit": "TFLOP/s",
                "frac": flops / t_kernel / FP64_MFMA_PEAK, "avg_launch_ms": t_kernel * 1e3,
                "flop_per_launch": flops, "traffic": GEMM_TRAFFIC_BYTES}

    # ------------------------------------------------------------------ host-resident operands (PCIe streaming)
    host = None
    if not args.skip_host:
        info = pkg.atc_info()

        def step_host():
            pkg.check(L.PARALiA_dgemm(b"N", b"N", n, n, n, 1.0, hA.ptr, n, hB.ptr, n, 0.0, hC.ptr, n, -1, 0, C.byref(info)), "PARALiA_dgemm host")

        t0 = time.perf_counter()
        step_host()                     # cold call: autotune + block pool allocation
        t_cold = time.perf_counter() - t0
        # untimed: the scheduler tries its four stream alignments on the four streamed calls after the cold one and keeps the best
        for _ in range(max(5, args.warmup)):
            step_host()
        times = []
        for _ in range(args.steps):
            t0 = time.perf_counter()
            step_host()
            times.append(time.perf_counter() - t0)
        t_host = sum(times) / len(times)
        goth = hC.host_view().reshape(n, n).T @ v
        parity_host = float(np.linalg.norm(goth - expect) / (np.linalg.norm(Am) * np.linalg.norm(Bm) * np.linalg.norm(v)))
        # measured pinned copy rates for the PCIe leg of the roofline (one large 2-D tile each way)
        T = int(info.T)
        tile = Buf(pkg, T * T, np.float64, 0)

        def copy_rate(dst, ldd, src, lds):
            pkg.check(L.pl_copy2d_async(dst, ldd, src, lds, T, T, 8, s), "copy")
            pkg.check(L.pl_stream_sync(s), "sync")
            t0 = time.perf_counter()
            for _ in range(8):
                pkg.check(L.pl_copy2d_async(dst, ldd, src, lds, T, T, 8, s), "copy")
            pkg.check(L.pl_stream_sync(s), "sync")
            return 8.0 * T * T * 8 / (time.perf_counter() - t0)

        h2d = copy_rate(tile.ptr, T, hA.ptr, n)
        d2h = copy_rate(hC.ptr, n, tile.ptr, T)
        t_roof = max(flops / FP64_MFMA_PEAK, 2.0 * n * n * 8 / h2d, 1.0 * n * n * 8 / d2h)
        host = {"workload": "same problem, A/B/C in pinned host memory, tiles streamed over PCIe", "gflops": flops / t_host / 1e9,
                "ms_per_call": t_host * 1e3, "min_ms": min(times) * 1e3, "max_ms": max(times) * 1e3, "cold_call_ms": t_cold * 1e3,
                "T": T, "subkernels": int(info.subkernel_num), "order_id": int(info.order_id), "T_selected_by": info.selected_by.decode(),
                "predicted_ms": info.pred_t * 1e3, "h2d_GBps": h2d / 1e9, "d2h_GBps": d2h / 1e9,
                "roof": "min(FP64 MFMA peak, PCIe-bound rate)", "roof_ms": t_roof * 1e3,
                "roof_bound": "mfma" if t_roof == flops / FP64_MFMA_PEAK else "pcie", "frac_of_roof": t_roof / t_host,
                "parity_checksum_err": parity_host}

    # ------------------------------------------------------------------ daxpy, device-resident (config 2)
    nd = 1 << 28
    dx, dy = dA, dB  # reuse the 2 GiB device buffers: 2^28 doubles each
    if dx.n >= nd:
        for _ in range(5):
            pkg.check(L.pl_daxpy(nd, 0.7, dx.ptr, 1, dy.ptr, 1, s), "daxpy")
        pkg.check(L.pl_stream_sync(s), "sync")
        pkg.check(L.pl_event_record(e0, s), "record")
        for _ in range(20):
            pkg.check(L.pl_daxpy(nd, 0.7, dx.ptr, 1, dy.ptr, 1, s), "daxpy")
        pkg.check(L.pl_event_record(e1, s), "record")
        pkg.check(L.pl_stream_sync(s), "sync")
        pkg.check(L.pl_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
        t_ax = ms.value / 20 / 1e3
        daxpy = {"workload": "daxpy N=2^28 fp64, x and y in HBM", "GBps": 24.0 * nd / t_ax / 1e9, "ms": t_ax * 1e3,
                 "frac_of_hbm_peak": 24.0 * nd / t_ax / HBM_PEAK}
        # ddot N = 2^28 and dgemv 16384 x 16384 (the 2 GiB of A as the matrix), device-resident, same event timing
        def timed(launch, reps):
            for _ in range(3):
                launch()
            pkg.check(L.pl_stream_sync(s), "sync")
            pkg.check(L.pl_event_record(e0, s), "record")
            for _ in range(reps):
                launch()
            pkg.check(L.pl_event_record(e1, s), "record")
            pkg.check(L.pl_stream_sync(s), "sync")
            pkg.check(L.pl_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
            return ms.value / reps / 1e3

        ws = Buf(pkg, max(int(L.pl_ddot_workspace_doubles()), int(L.pl_dgemv_workspace_doubles(b"N", 16384, 16384))) + 1, np.float64, 0)
        res, yv = Buf(pkg, 1, np.float64, 0), Buf(pkg, 16384, np.float64, 0)
        t_dot = timed(lambda: pkg.check(L.pl_ddot(nd, dx.ptr, 1, dy.ptr, 1, res.ptr, 0, ws.ptr, s), "ddot"), 20)
        t_mv = timed(lambda: pkg.check(L.pl_dgemv(b"N", 16384, 16384, 1.2, dx.ptr, 16384, dy.ptr, 1, 1.1, yv.ptr, 1, ws.ptr, s), "dgemv"), 20)
        daxpy["ddot_GBps"] = 16.0 * nd / t_dot / 1e9
        daxpy["ddot_frac_of_hbm_peak"] = 16.0 * nd / t_dot / HBM_PEAK
        daxpy["dgemv_16384_GBps"] = 8.0 * (16384.0 * 16384 + 3 * 16384) / t_mv / 1e9
        daxpy["dgemv_16384_frac_of_hbm_peak"] = 8.0 * (16384.0 * 16384 + 3 * 16384) / t_mv / HBM_PEAK
    else:
        daxpy = None

    # ------------------------------------------------------------------ CPU baseline: OpenBLAS on the host cores
    cpu = None
    if not args.skip_cpu:
        import oracle_binding as ob
        orc = ob.load()
        if orc.orc_openblas_open(None) == 0:
            cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
            cores = orc.orc_openblas_threads(cores) or cores
            ncols = max(256, min(n, 8192))  # a column panel of C: M x ncols x K of the same problem (a few seconds on 16 cores)
            ref = np.zeros(n * ncols)
            orc.orc_openblas_dgemm(b"N", b"N", n, 256, n, 1.0, hA.ptr, n, hB.ptr, n, 0.0, ob.ptr(ref), n)  # warm-up
            t0 = time.perf_counter()
            orc.orc_openblas_dgemm(b"N", b"N", n, ncols, n, 1.0, hA.ptr, n, hB.ptr, n, 0.0, ob.ptr(ref), n)
            t_cpu = time.perf_counter() - t0
            panel = dC.get()[: n * ncols]
            d = float(np.linalg.norm(Am) * np.linalg.norm(Bm[:, :ncols]))
            err = float(np.linalg.norm(panel - ref) / d)
            cpu = {"value": 2.0 * n * ncols * n / t_cpu / 1e9, "unit": "GFLOP/s", "cores": int(cores), "kind": "port",
                   "sample": "OpenBLAS cblas_dgemm (%s) on the first %d columns of C of the same problem (M=%d, N=%d, K=%d), %.1f s"
                             % (os.path.basename(orc.orc_openblas_path().decode()), ncols, n, ncols, n, t_cpu),
                   "gpu_vs_openblas_normwise_err": err}
            # the reference's own CPU-runnable configuration: dgemm 4096^3, alpha = 1.2, beta = 1.1, on the same cores
            m1 = min(n, 4096)
            c1 = np.ones(m1 * m1)
            orc.orc_openblas_dgemm(b"N", b"N", m1, m1, m1, 1.2, hA.ptr, n, hB.ptr, n, 1.1, ob.ptr(c1), m1)
            t0 = time.perf_counter()
            orc.orc_openblas_dgemm(b"N", b"N", m1, m1, m1, 1.2, hA.ptr, n, hB.ptr, n, 1.1, ob.ptr(c1), m1)
            cpu["dgemm_4096_alpha1.2_beta1.1_gflops"] = 2.0 * m1 ** 3 / (time.perf_counter() - t0) / 1e9
        else:
            cpu = {"value": None, "unit": "GFLOP/s", "cores": 0, "kind": "port", "sample": "OpenBLAS absent on this box"}

    # ------------------------------------------------------------------ the other two streamed GEMM configurations
    other = None
    if args.other_configs and not args.skip_host and n == 16384:
        other = {}
        for b in (dA, dB, dC):
            b.free()
        keep = []  # host buffers stay allocated until the end

        def streamed(tag, fn, dtype, ta, tb, M, N, K, alpha, beta, locs, roof_ms, roof_note):
            try:
                ra, ca = (M, K) if ta == b"N" else (K, M)
                rb, cb = (K, N) if tb == b"N" else (N, K)
                init = L.PARALiA_vec_init_f64 if dtype == np.float64 else L.PARALiA_vec_init_f32
                bufs = [Buf(pkg, ra * ca, dtype, locs[0]), Buf(pkg, rb * cb, dtype, locs[1]), Buf(pkg, M * N, dtype, locs[2])]
                for b, seed in zip(bufs, (42, 43, 44)):
                    pkg.check(init(b.ptr, b.n, seed, b.loc), "vec_init")
                inf = pkg.atc_info()

                def call():
                    pkg.check(fn(ta, tb, M, N, K, alpha, bufs[0].ptr, ra, bufs[1].ptr, rb, beta, bufs[2].ptr, M, -1, 0, C.byref(inf)), tag)
                # cold call, the four calls that settle the stream alignment, and as many warm-ups as the reference's
                # runner makes (dgemm_runner.cpp:121-125): after the device block pool has been re-allocated for a new
                # block size the link-bound configuration runs 4 % slow for its first ten calls or so
                for _ in range(13):
                    call()
                ts = []
                for _ in range(5):
                    t0 = time.perf_counter()
                    call()
                    ts.append(time.perf_counter() - t0)
                t = sum(ts) / len(ts)
                other[tag] = {"ms_per_call": t * 1e3, "gflops": 2.0 * M * N * K / t / 1e9, "T": int(inf.T), "order_id": int(inf.order_id),
                              "predicted_ms": inf.pred_t * 1e3, "roof_ms": roof_ms, "roof": roof_note, "frac_of_roof": roof_ms / (t * 1e3)}
                keep.extend(bufs)
            except Exception as e:  # these are extras: the headline line must come out whatever happens here
                other[tag] = {"error": str(e)[:200]}
        streamed("sgemm_32768_NT_AB_host_C_device", L.PARALiA_sgemm, np.float32, b"N", b"T", 32768, 32768, 32768, 1.0, 1.0, (-1, -1, 0),
                 2.0 * 32768 ** 3 / 157.3e12 * 1e3, "fp32 MFMA peak 157.3 TFLOP/s")
        streamed("dgemm_40000x40000x2048_host_beta0.5", L.PARALiA_dgemm, np.float64, b"N", b"N", 40000, 40000, 2048, 1.5, 0.5, (-1, -1, -1),
                 (40000.0 * 2048 * 2 + 40000.0 * 40000) * 8 / 56.25e9 * 1e3, "H2D bytes at the measured 56.25 GB/s")

    out = {
        "metric": "PARALiA_dgemm GFLOP/s (16K fp64)", "value": flops / t_step / 1e9, "unit": "GFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": t_step * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": "dgemm M=N=K=%d fp64 column-major NN alpha=1 beta=0, A/B/C resident in HBM (BASELINE config 3 shape)" % n,
                   "device": name.value.decode(), "entry_point": "PARALiA_dgemm (C ABI of PARALiADgemm)"},
        "parity_checksum_err": parity,
        "roofline": roofline, "cpu_baseline": cpu, "host_operands": host, "daxpy_device": daxpy, "other_configs": other,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
