// Deploy-time microbenchmarks and database builder for one MI355X.
//
//   paralia_deploy <db_dir> [--quick] [--only gemm|gemv|blas1|link|fit]
//
// Measures (1) the tile GEMM kernels over square T for the four transpose combinations, fp64 and fp32,
// (2) daxpy / ddot over vector lengths and dgemv over square T for both transposes, (3) pinned-host <-> device 2-D tile copies in both directions and the
// slowdown of each direction while the other is busy, (4) the power-state transient of the tile kernels after idle time, (5) the constants of the tile-GEMM launcher's cost model;
// writes the raw logs to <db_dir>/Benchmark-Results and the
// tables the autotuner reads to <db_dir>/Processed.
//
// What it re-does from the reference: Database_builder/CuCuBLAS/src/dgemm_microbench.cu:26-230 (T sweep from
// 256 in steps of 256, the step doubling once T >= 16*step, up to < 10000; alpha = 1.1234;
// stop when the 95% confidence half-width is within 5% of the mean and more than 10 samples were taken),
// dgemv_microbench.cu:26-250 (the same T sweep, MIN/STEP/MAX_DIM_BLAS2 of microbenchmarks.hpp:31-33; table line
// TransA,M,N,t,W,J,err,n,bench as GPUexec_lookup.cpp:196-198 reads it),
// daxpy_microbench.cu / ddot_microbench.cu (sweep from 4096 in steps of 4096 with the same doubling),
// transfer_link_microbench.cu:24-218 (square tiles with a host leading dimension of maxDim + 1, then the
// overlap run), Python-DataManage/BenchToLookupTables.py.in:31-55 (flag columns prepended, sorted by T) and
// LinkPreprocessing.py.in:44-61 (least-squares line bytes -> seconds, |intercept|, slowdown ratios).
// File formats are unchanged so the tables are interchangeable with the reference's.
// Kernel times are taken the way the scheduler runs the kernels: dense tiles (leading dimension = T, as in the
// device block pool), beta = 1 (every K-step but the first accumulates), launches round-robin over its compute
// streams, time per launch = wall time of a batch / launches in it.  (The reference benchmarks with the leading
// dimension of the largest size and beta = 1.2345.)
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <sys/stat.h>
#include <vector>

#include "Autotuner.hpp"
#include "backend_wrappers.hpp"
#include "paralia_hip.h"

#define DEPLOY_VERSION "2.0"
#define MICRO_MIN_ITER 10
#define MICRO_MAX_ITER 100

static void must(int rc, const char* what) {
  if (rc != 0) {
    fprintf(stderr, "paralia_deploy: %s failed (%d): %s\n", what, rc, pl_last_error());
    exit(1);
  }
}

// two-sided 95% Student-t quantile
static double t975(int df) {
  static const double tab[] = {0,      12.706, 4.303, 3.182, 2.776, 2.571, 2.447, 2.365, 2.306, 2.262, 2.228,
                               2.201,  2.179,  2.160, 2.145, 2.131, 2.120, 2.110, 2.101, 2.093, 2.086, 2.080,
                               2.074,  2.069,  2.064, 2.060, 2.056, 2.052, 2.048, 2.045, 2.042};
  if (df < 1) return 1e9;
  if (df <= 30) return tab[df];
  return 1.96 + 2.5 / df;
}

struct Sample { double mean = 0, margin = 0, bench_t = 0; long n = 0; };

// Repeats run() until the 95% CI half-width is within 5% of the mean (n > MICRO_MIN_ITER) or MICRO_MAX_ITER.
template <typename F> static Sample sample_until_stable(F&& run) {
  std::vector<double> v;
  Sample s;
  const double t_start = csecond();
  double sum = 0;
  for (int i = 1; i <= MICRO_MAX_ITER; ++i) {
    const double t = run();
    v.push_back(t);
    sum += t;
    s.mean = sum / i;
    s.n = i;
    if (i < 2) continue;
    double var = 0;
    for (double x : v) var += (x - s.mean) * (x - s.mean);
    const double sd = sqrt(var / i);
    s.margin = t975(i - 1) * sd / sqrt((double)i);
    if (i > MICRO_MIN_ITER && s.margin / s.mean * 100 <= 5) break;
  }
  s.bench_t = csecond() - t_start;
  return s;
}

static std::vector<long> sweep(long start, long step, long limit, int double_at) {
  std::vector<long> out;
  for (long T = start; T < limit; T += step) {
    if (T >= step * double_at) step *= 2;
    out.push_back(T);
  }
  return out;
}

struct Row { char ta, tb; long T; Sample s; Sample lone; };

static void mkdirs(const std::string& d) {
  mkdir(d.c_str(), 0755);
  mkdir((d + "/Benchmark-Results").c_str(), 0755);
  mkdir((d + "/Processed").c_str(), 0755);
}

template <typename T>
static void bench_gemm(const std::string& db, const char* func, bool quick, int queues) {
  const long maxDim = quick ? 4352 : 10000;
  std::vector<long> Ts = sweep(256, 256, maxDim, 16);
  if (quick) {
    std::vector<long> few;
    for (long t : Ts) if (t == 512 || t == 1024 || t == 2048 || t == 3072 || t == 4096) few.push_back(t);
    Ts = few;
  }
  const long ld = maxDim;  // allocation edge; every measured tile is dense (its own T as leading dimension)
  T *A, *B, *C;
  A = (T*)CoCoMalloc(ld * ld * sizeof(T), 0, 0);
  B = (T*)CoCoMalloc(ld * ld * sizeof(T), 0, 0);
  C = (T*)CoCoMalloc(2 * ld * ld * sizeof(T), 0, 1);
  CoCoVecInit(A, ld * ld, 42, 0);
  CoCoVecInit(B, ld * ld, 43, 0);
  CoCoVecInit(C, 2 * ld * ld, 44, 0);
  std::vector<void*> st(queues);
  for (auto& s : st) must(pl_stream_create(&s), "stream");
  const long ws_cap = 512L << 20;
  std::vector<void*> ws(queues);
  for (auto& w : ws) w = CoCoMalloc(ws_cap, 0, 1);
  const T alpha = (T)1.1234, beta = (T)1;
  std::vector<Row> rows;
  const char flags[2] = {'N', 'T'};
  for (char ta : flags)
    for (char tb : flags) {
      char raw[1024];
      snprintf(raw, sizeof raw, "%s/Benchmark-Results/hip%s_dev-0_TransA-%c_TransB-%c_%s.log", db.c_str(), func, ta, tb, DEPLOY_VERSION);
      FILE* fp = fopen(raw, "w");
      if (!fp) { fprintf(stderr, "cannot write %s\n", raw); exit(1); }
      for (long Tt : Ts) {
        // launched the way the runtime launches a subkernel: with a split-K workspace per stream
        const long ws_bytes = pl_gemm_tile_workspace_bytes(Tt, Tt, Tt, (int)sizeof(T));
        if (ws_bytes > ws_cap) { fprintf(stderr, "split-K workspace larger than expected\n"); exit(1); }
        auto launch = [&](int q) {
          if (sizeof(T) == 8)
            must(pl_dgemm_tile_ws(ta, tb, Tt, Tt, Tt, alpha, (const double*)A, Tt, (const double*)B, Tt, beta, (double*)(C + (long)q * ld * ld), Tt,
                                  ws[q], ws_bytes, st[q]), "gemm");
          else
            must(pl_sgemm_tile_ws(ta, tb, Tt, Tt, Tt, alpha, (const float*)A, Tt, (const float*)B, Tt, beta, (float*)(C + (long)q * ld * ld), Tt,
                                  ws[q], ws_bytes, st[q]), "gemm");
        };
        // long enough that the ramp at both ends of a batch does not weigh on the steady-state rate
        const int batch = (Tt <= 2048 ? 16 : Tt <= 4096 ? 6 : 2) * queues;
        auto run = [&]() {
          const double t0 = csecond();
          for (int i = 0; i < batch; ++i) launch(i % queues);
          for (auto s : st) must(pl_stream_sync(s), "sync");
          return (csecond() - t0) / batch;
        };
        run();  // warm-up
        Row r{ta, tb, Tt, sample_until_stable(run), Sample()};
        // the same launches on one stream only: what a subkernel takes when nothing runs beside it
        auto run_lone = [&]() {
          const int n = std::max(2, batch / queues);
          const double t0 = csecond();
          for (int i = 0; i < n; ++i) launch(0);
          must(pl_stream_sync(st[0]), "sync");
          return (csecond() - t0) / n;
        };
        run_lone();
        r.lone = sample_until_stable(run_lone);
        rows.push_back(r);
        fprintf(fp, "%ld,%ld,%ld, %e,%e,%e,%e,%ld,%e\n", Tt, Tt, Tt, r.s.mean, -1.0, -1.0, r.s.margin, r.s.n, r.s.bench_t);
        fprintf(stderr, "%s %c%c T=%ld: %.3f ms (%.1f GFLOP/s), margin %.2f%%, %ld samples\n", func, ta, tb, Tt, r.s.mean * 1e3,
                2.0 * Tt * Tt * Tt / r.s.mean / 1e9, r.s.margin / r.s.mean * 100, r.s.n);
      }
      fclose(fp);
    }
  // Processed table: flag columns prepended, rows of all four files concatenated and sorted by T
  std::stable_sort(rows.begin(), rows.end(), [](const Row& a, const Row& b) { return a.T < b.T; });
  char out[1024];
  snprintf(out, sizeof out, "%s/Processed/%s_lookup-table_dev-0.log", db.c_str(), func);
  FILE* fp = fopen(out, "w");
  if (!fp) { fprintf(stderr, "cannot write %s\n", out); exit(1); }
  for (const Row& r : rows)
    fprintf(fp, "%c,%c,%ld,%ld,%ld,%e,%e,%e,%e,%ld,%e\n", r.ta, r.tb, r.T, r.T, r.T, r.s.mean, -1.0, -1.0, r.s.margin, r.s.n, r.s.bench_t);
  fclose(fp);
  // not a table of the reference: the lone-launch times, TransA,TransB,T,seconds
  snprintf(out, sizeof out, "%s/Processed/%s_lone-launch_dev-0.log", db.c_str(), func);
  fp = fopen(out, "w");
  if (!fp) { fprintf(stderr, "cannot write %s\n", out); exit(1); }
  for (const Row& r : rows) fprintf(fp, "%c,%c,%ld,%e\n", r.ta, r.tb, r.T, r.lone.mean);
  fclose(fp);
  for (auto s : st) pl_stream_destroy(s);
  CoCoFree(A, 0); CoCoFree(B, 0); CoCoFree(C, 0);
  for (auto w : ws) CoCoFree(w, 0);
}

static void bench_gemv(const std::string& db, bool quick) {
  const long maxDim = quick ? 4352 : 10000;
  std::vector<long> Ts = sweep(256, 256, maxDim, 16);
  if (quick) {
    std::vector<long> few;
    for (long t : Ts) if (t == 512 || t == 1024 || t == 2048 || t == 4096) few.push_back(t);
    Ts = few;
  }
  double* A = (double*)CoCoMalloc(maxDim * maxDim * sizeof(double), 0, 0);
  double* x = (double*)CoCoMalloc(maxDim * sizeof(double), 0, 0);
  double* y = (double*)CoCoMalloc(maxDim * sizeof(double), 0, 1);
  CoCoVecInit(A, maxDim * maxDim, 42, 0);
  CoCoVecInit(x, maxDim, 43, 0);
  CoCoVecInit(y, maxDim, 44, 0);
  long long ws_doubles = 8;
  for (long Tt : Ts) ws_doubles = std::max(ws_doubles, std::max(pl_dgemv_workspace_doubles('N', Tt, Tt), pl_dgemv_workspace_doubles('T', Tt, Tt)));
  double* ws = (double*)CoCoMalloc(ws_doubles * 8, 0, 1);
  void* st;
  must(pl_stream_create(&st), "stream");
  std::vector<Row> rows;
  for (char ta : {'N', 'T'}) {
    char raw[1024];
    snprintf(raw, sizeof raw, "%s/Benchmark-Results/hipDgemv_dev-0_TransA-%c_%s.log", db.c_str(), ta, DEPLOY_VERSION);
    FILE* fp = fopen(raw, "w");
    if (!fp) { fprintf(stderr, "cannot write %s\n", raw); exit(1); }
    for (long Tt : Ts) {
      const int batch = Tt <= 2048 ? 16 : 4;
      auto run = [&]() {
        const double t0 = csecond();
        // dense tile, beta = 1: the way the scheduler runs every subkernel but the first of a y tile
        for (int i = 0; i < batch; ++i) must(pl_dgemv(ta, Tt, Tt, 1.1234, A, Tt, x, 1, 1.0, y, 1, ws, st), "dgemv");
        must(pl_stream_sync(st), "sync");
        return (csecond() - t0) / batch;
      };
      run();
      Row r{ta, 'N', Tt, sample_until_stable(run), Sample()};
      rows.push_back(r);
      fprintf(fp, "%ld,%ld, %e,%e,%e,%e,%ld,%e\n", Tt, Tt, r.s.mean, -1.0, -1.0, r.s.margin, r.s.n, r.s.bench_t);
      fprintf(stderr, "Dgemv %c T=%ld: %.4f ms (%.1f GB/s), margin %.2f%%, %ld samples\n", ta, Tt, r.s.mean * 1e3,
              8.0 * Tt * Tt / r.s.mean / 1e9, r.s.margin / r.s.mean * 100, r.s.n);
    }
    fclose(fp);
  }
  std::stable_sort(rows.begin(), rows.end(), [](const Row& a, const Row& b) { return a.T < b.T; });
  char out[1024];
  snprintf(out, sizeof out, "%s/Processed/Dgemv_lookup-table_dev-0.log", db.c_str());
  FILE* fp = fopen(out, "w");
  if (!fp) { fprintf(stderr, "cannot write %s\n", out); exit(1); }
  for (const Row& r : rows)
    fprintf(fp, "%c,%ld,%ld,%e,%e,%e,%e,%ld,%e\n", r.ta, r.T, r.T, r.s.mean, -1.0, -1.0, r.s.margin, r.s.n, r.s.bench_t);
  fclose(fp);
  pl_stream_destroy(st);
  CoCoFree(A, 0); CoCoFree(x, 0); CoCoFree(y, 0); CoCoFree(ws, 0);
}

static void bench_blas1(const std::string& db, const char* func, bool quick) {
  const long maxN = quick ? (1L << 24) + 1 : (1L << 27) + 1;
  std::vector<long> Ns = sweep(4096, 4096, maxN, 16);
  if (quick) {
    std::vector<long> few;
    for (long n : Ns) if ((n & (n - 1)) == 0 && n >= (1 << 16)) few.push_back(n);
    Ns = few;
  }
  double* x = (double*)CoCoMalloc(maxN * 8, 0, 0);
  double* y = (double*)CoCoMalloc(maxN * 8, 0, 1);
  CoCoVecInit(x, maxN, 42, 0);
  CoCoVecInit(y, maxN, 43, 0);
  double* ws = (double*)CoCoMalloc((pl_ddot_workspace_doubles() + 1) * 8, 0, 1);
  void* st;
  must(pl_stream_create(&st), "stream");
  const bool axpy = !strcmp(func, "Daxpy");
  char raw[1024], out[1024];
  snprintf(raw, sizeof raw, "%s/Benchmark-Results/hip%s_dev-0_%s.log", db.c_str(), func, DEPLOY_VERSION);
  snprintf(out, sizeof out, "%s/Processed/%s_lookup-table_dev-0.log", db.c_str(), func);
  FILE* fr = fopen(raw, "w");
  FILE* fo = fopen(out, "w");
  if (!fr || !fo) { fprintf(stderr, "cannot write %s\n", out); exit(1); }
  for (long N : Ns) {
    const int batch = 4;
    auto run = [&]() {
      const double t0 = csecond();
      for (int i = 0; i < batch; ++i) {
        if (axpy) must(pl_daxpy(N, 1.1234, x, 1, y, 1, st), "daxpy");
        else must(pl_ddot(N, x, 1, y, 1, ws + pl_ddot_workspace_doubles(), 0, ws, st), "ddot");
      }
      must(pl_stream_sync(st), "sync");
      return (csecond() - t0) / batch;
    };
    run();
    Sample s = sample_until_stable(run);
    fprintf(fr, "%ld, %e,%e,%e,%e,%ld,%e\n", N, s.mean, -1.0, -1.0, s.margin, s.n, s.bench_t);
    fprintf(fo, "%ld,%e,%e,%e,%e,%ld,%e\n", N, s.mean, -1.0, -1.0, s.margin, s.n, s.bench_t);
    fprintf(stderr, "%s N=%ld: %.4f ms (%.1f GB/s)\n", func, N, s.mean * 1e3, (axpy ? 24.0 : 16.0) * N / s.mean / 1e9);
  }
  fclose(fr);
  fclose(fo);
  pl_stream_destroy(st);
  CoCoFree(x, 0); CoCoFree(y, 0); CoCoFree(ws, 0);
}

// The device's power-state transient, as the tile kernels see it: pairs of 2048^3 fp64 launches on two streams, 100 pairs
// back to back (the first burst brings the device to its steady state), then after a host-side gap of 2, 5, 10, 20 and
// 50 ms without kernels another 100, every pair timed with events.  Against the steady pair time of a burst's last 40
// pairs a burst after a gap loses L(gap) seconds in its first 60 pairs, the slowest pair being (1 + amplitude) x steady.
// With the deficit decaying exponentially while kernels run, L(50 ms) = amplitude x recovery constant; with it growing
// as 1 - exp(-gap / idle constant) while none run, the idle constant is the one that fits L(gap) / L(50 ms) over the
// five gaps best (least squares over a grid of constants).  Three repetitions, medians.
// Written to Processed/Power-transient_dev-0.log (seconds); not a file of the reference.
static void bench_transient(const std::string& db) {
  const long Tt = 2048;
  const int pairs = 100;
  double *A, *B, *C;
  A = (double*)CoCoMalloc(Tt * Tt * sizeof(double), 0, 0);
  B = (double*)CoCoMalloc(Tt * Tt * sizeof(double), 0, 0);
  C = (double*)CoCoMalloc(2 * Tt * Tt * sizeof(double), 0, 1);
  CoCoVecInit(A, Tt * Tt, 42, 0);
  CoCoVecInit(B, Tt * Tt, 43, 0);
  CoCoVecInit(C, 2 * Tt * Tt, 44, 0);
  void* st[2];
  for (auto& s : st) must(pl_stream_create(&s), "stream");
  std::vector<void*> ev(pairs + 1);
  for (auto& e : ev) must(pl_event_create(&e, 1), "event");
  auto burst = [&](std::vector<double>& t) {
    must(pl_event_record(ev[0], st[0]), "record");
    for (int i = 0; i < pairs; ++i) {
      for (int q = 0; q < 2; ++q)
        must(pl_dgemm_tile_ws('N', 'N', Tt, Tt, Tt, 1e-9, A, Tt, B, Tt, 1.0, C + (long)q * Tt * Tt, Tt, nullptr, 0, st[q]), "gemm");
      must(pl_event_record(ev[i + 1], st[0]), "record");
    }
    for (auto s : st) must(pl_stream_sync(s), "sync");
    t.resize(pairs);
    for (int i = 0; i < pairs; ++i) {
      float ms = 0;
      must(pl_event_elapsed_ms(ev[i], ev[i + 1], &ms), "elapsed");
      t[i] = ms * 1e-3;
    }
  };
  auto median3 = [](double a, double b, double c) { return std::max(std::min(a, b), std::min(std::max(a, b), c)); };
  constexpr int NG = 5;
  const double gaps[NG] = {2e-3, 5e-3, 10e-3, 20e-3, 50e-3};
  double loss[NG][3], peak[3], steady_t = 0;
  std::vector<double> t;
  for (int rep = 0; rep < 3; ++rep)
    for (int g = 0; g < NG; ++g) {
      burst(t);  // warm: whatever came before, the device is in its steady state afterwards
      const double t0 = csecond();
      while (csecond() - t0 < gaps[g]) {
      }
      burst(t);
      double steady = 0;
      for (int i = 60; i < pairs; ++i) steady += t[i] / (pairs - 60);
      double l = 0, p = 0;
      for (int i = 0; i < 60; ++i) l += t[i] - steady;
      for (int i = 0; i < 20; ++i) p = std::max(p, t[i] / steady - 1.0);
      loss[g][rep] = std::max(l, 0.0);
      if (g == NG - 1) { peak[rep] = p; steady_t = steady; }
    }
  double L[NG];
  for (int g = 0; g < NG; ++g) L[g] = median3(loss[g][0], loss[g][1], loss[g][2]);
  double amp = median3(peak[0], peak[1], peak[2]);
  double recover = 0, idle = 0;
  if (amp < 0.02 || L[NG - 1] <= 0) {
    amp = 0;  // nothing to model on this device
  } else {
    recover = L[NG - 1] / amp;
    double best = 1e300;
    for (double tau = 1e-3; tau <= 60e-3; tau += 0.25e-3) {
      // the longest gap is not quite infinite: compare with the curve normalised at that gap
      const double full = 1.0 - exp(-gaps[NG - 1] / tau);
      double sq = 0;
      for (int g = 0; g < NG - 1; ++g) {
        const double d = L[g] / L[NG - 1] - (1.0 - exp(-gaps[g] / tau)) / full;
        sq += d * d;
      }
      if (sq < best) { best = sq; idle = tau; }
    }
  }
  char out[1024];
  snprintf(out, sizeof out, "%s/Processed/Power-transient_dev-0.log", db.c_str());
  FILE* fp = fopen(out, "w");
  if (!fp) { fprintf(stderr, "cannot write %s\n", out); exit(1); }
  fprintf(fp, "Amplitude: %e\nRecovery: %e\nIdle: %e\n", amp, recover, idle);
  fclose(fp);
  fprintf(stderr, "power transient: steady pair %.3f ms, after 2 / 5 / 10 / 20 / 50 ms idle %.2f / %.2f / %.2f / %.2f / %.2f ms lost, slowest pair +%.1f %% -> recovery %.1f ms, idle %.1f ms\n",
          steady_t * 1e3, L[0] * 1e3, L[1] * 1e3, L[2] * 1e3, L[3] * 1e3, L[4] * 1e3, amp * 100, recover * 1e3, idle * 1e3);
  for (auto e : ev) pl_event_destroy(e);
  for (auto s : st) pl_stream_destroy(s);
  CoCoFree(A, 0); CoCoFree(B, 0); CoCoFree(C, 0);
}

// Least-squares line y = a + b x.
static void fit_line(const std::vector<double>& x, const std::vector<double>& y, double* a, double* b) {
  const double n = (double)x.size();
  double sx = 0, sy = 0, sxx = 0, sxy = 0;
  for (size_t i = 0; i < x.size(); ++i) { sx += x[i]; sy += y[i]; sxx += x[i] * x[i]; sxy += x[i] * y[i]; }
  *b = (n * sxy - sx * sy) / (n * sxx - sx * sx);
  *a = (sy - *b * sx) / n;
}

// The constants of the tile-GEMM launcher's cost model and of the plan simulator that are not table rows
// (pl_gemm_fit, KernelFit): time per launch of a product with one workgroup per compute unit over K (per-k cost and
// fixed part of a lone 128 x 128 workgroup), of M = N = 8192 products over K with each fp32 macro tile pinned (per-k
// cost and fixed cost per round of the small, wide and large tile, per transpose and for beta == 0 / != 0), the gap
// between two launches of a stream, the rate of the scale-add pass, and what a slab of a thin start costs beyond its
// share of the tile.  Written to Processed/Kernel-fit_dev-0.log as "name: value" lines; not a file of the reference.
static void bench_fit(const std::string& db, bool quick) {
  const long big = 8192, one_round = 2048;
  void* A = CoCoMalloc(big * big * 8, 0, 0);
  void* B = CoCoMalloc(big * big * 8, 0, 0);
  void* C = CoCoMalloc(big * big * 8, 0, 1);
  CoCoVecInit((double*)A, big * big, 42, 0);
  CoCoVecInit((double*)B, big * big, 43, 0);
  CoCoVecInit((double*)C, big * big, 44, 0);
  void* st[2];
  for (auto& s : st) must(pl_stream_create(&s), "stream");
  const std::vector<long> Ks = quick ? std::vector<long>{1024, 4096, 8192} : std::vector<long>{512, 1024, 2048, 4096, 8192};
  // time per launch in microseconds: n launches on `queues` streams round-robin, wall time / n
  auto per_launch_us = [&](bool f64, char ta, char tb, long M, long N, long K, double beta, int queues) {
    auto launch = [&](int q) {
      char* c = (char*)C + (size_t)q * M * N * 8;   // a C of its own per stream
      const long lda = ta == 'N' ? M : K, ldb = tb == 'N' ? K : N;
      if (f64) must(pl_dgemm_tile(ta, tb, M, N, K, 1e-3, (const double*)A, lda, (const double*)B, ldb, beta, (double*)c, M, st[q]), "gemm");
      else must(pl_sgemm_tile(ta, tb, M, N, K, 1e-3f, (const float*)A, lda, (const float*)B, ldb, (float)beta, (float*)c, M, st[q]), "gemm");
    };
    const double flop = 2.0 * M * N * K;
    const int n = std::max(2 * queues, std::min(64, (int)(2.0e12 / flop)) / queues * queues);
    auto run = [&]() {
      const double t0 = csecond();
      for (int i = 0; i < n; ++i) launch(i % queues);
      for (int q = 0; q < queues; ++q) must(pl_stream_sync(st[q]), "sync");
      return (csecond() - t0) / n;
    };
    run();
    return sample_until_stable(run).mean * 1e6;
  };
  auto over_k = [&](bool f64, char ta, char tb, long MN, double beta, double rounds, double* fixed_us, double* us_per_k, const std::vector<long>* ks = nullptr) {
    std::vector<double> x, y;
    for (long K : (ks ? *ks : Ks)) { x.push_back((double)K); y.push_back(per_launch_us(f64, ta, tb, MN, MN, K, beta, 1) / rounds); }
    fit_line(x, y, fixed_us, us_per_k);
  };
  KernelFit k;
  pl_gemm_fit& f = k.launcher;
  // the gap between two launches of a stream: a scale-add over a 16 x 16 tile, 400 in a row
  {
    auto run = [&]() {
      const double t0 = csecond();
      for (int i = 0; i < 400; ++i) must(pl_dgeadd_tile(16, 16, 1.0, (const double*)A, 16, (const double*)C, 16, (double*)C, 16, st[0]), "geadd");
      must(pl_stream_sync(st[0]), "sync");
      return (csecond() - t0) / 400;
    };
    run();
    f.splitk_launch_us = sample_until_stable(run).mean * 1e6;
  }
  // the scale-add pass over a tile, 3 T^2 elements.  At T = 1024 on one and the same tile: the slices a split-K product
  // adds up were written a moment ago and are still in the caches.  At T = 2048 over twelve different tiles in turn
  // (768 MiB, more than the memory-side cache holds): the lazy reduce reads a C tile the copy engine has just brought in.
  auto geadd_rate = [&](long T, int tiles) {
    auto run = [&]() {
      const double t0 = csecond();
      for (int i = 0; i < 48; ++i) {
        const size_t off = (size_t)(i % tiles) * T * T;
        must(pl_dgeadd_tile(T, T, 0.5, (const double*)A + off, T, (const double*)C + off, T, (double*)C + off, T, st[0]), "geadd");
      }
      must(pl_stream_sync(st[0]), "sync");
      return (csecond() - t0) / 48;
    };
    run();
    return 3.0 * T * T * 8 / sample_until_stable(run).mean;
  };
  f.pass_bytes_per_us = geadd_rate(1024, 1) / 1e6;
  k.geadd_bytes_per_s = geadd_rate(2048, 12);
  // one 128 x 128 workgroup per compute unit (2048 x 2048: 256 tiles), small tile, no split: time over K
  setenv("PARALIA_GEMM_LARGE_TILE", "0", 1);
  double a = 0, b = 0;
  // (beta == 0, as the kernels of a split product run: they write their slice and read nothing of C; K up to 4096: the
  // chunks of a split are short, and from K = 8192 on A and B of these repeated launches no longer fit the memory-side
  // cache, which a lone workgroup per compute unit feels -- another regime than the one the split decision prices)
  const std::vector<long> lone_ks = quick ? std::vector<long>{1024, 2048, 4096} : std::vector<long>{512, 1024, 2048, 4096};
  over_k(true, 'N', 'N', one_round, 0.0, 1.0, &a, &b, &lone_ks);
  f.lone_us_per_k[0] = b;
  const double fixed_k64 = a / b;
  over_k(false, 'N', 'N', one_round, 0.0, 1.0, &a, &b, &lone_ks);
  f.lone_us_per_k[1] = b;
  f.lone_fixed_k = std::max(0.0, 0.5 * (fixed_k64 + a / b));
  // fp32, M = N = 8192: 8 rounds of 512 small tiles (beta == 0 and != 0 pooled), 4 rounds of 512 wide tiles (NN), 4 rounds
  // of 256 large tiles per transpose
  double a0 = 0, b0 = 0, a1 = 0, b1 = 0;
  over_k(false, 'N', 'N', big, 0.0, 8.0, &a0, &b0);
  over_k(false, 'N', 'N', big, 1.0, 8.0, &a1, &b1);
  f.f32_small_us_per_k = 0.5 * (b0 + b1);
  f.f32_small_fixed_us = std::max(0.0, 0.5 * (a0 + a1));
  setenv("PARALIA_GEMM_LARGE_TILE", "2", 1);
  over_k(false, 'N', 'N', big, 0.0, 4.0, &a0, &b0);
  over_k(false, 'N', 'N', big, 1.0, 4.0, &a1, &b1);
  f.f32_wide_gain = 2.0 * f.f32_small_us_per_k / (0.5 * (b0 + b1));
  f.f32_wide_fixed_us[0] = std::max(0.0, a0);
  f.f32_wide_fixed_us[1] = std::max(0.0, a1);
  setenv("PARALIA_GEMM_LARGE_TILE", "1", 1);
  const char tas[4] = {'N', 'N', 'T', 'T'}, tbs[4] = {'N', 'T', 'N', 'T'};
  for (int t = 0; t < 4; ++t) {
    over_k(false, tas[t], tbs[t], big, 0.0, 4.0, &a0, &b0);
    over_k(false, tas[t], tbs[t], big, 1.0, 4.0, &a1, &b1);
    f.f32_large_gain[t] = 2.0 * f.f32_small_us_per_k / (0.5 * (b0 + b1)) - 1.0;
    f.f32_large_fixed_us[t][0] = std::max(0.0, a0);
    f.f32_large_fixed_us[t][1] = std::max(0.0, a1);
  }
  // what the guarded edge workgroups of a ragged grid add to a product alone on the device, in rounds: 4000 x 4096 x 4096
  // against 4096^3, fp32 NT -- one round of 256 large tiles, two rounds of 512 small ones
  {
    const double whole_l = per_launch_us(false, 'N', 'T', 4096, 4096, 4096, 0.0, 1), ragged_l = per_launch_us(false, 'N', 'T', 4000, 4096, 4096, 0.0, 1);
    f.edge_rounds[1] = std::min(2.0, std::max(0.0, (ragged_l - whole_l) / whole_l));
    setenv("PARALIA_GEMM_LARGE_TILE", "0", 1);
    const double whole_s = per_launch_us(false, 'N', 'T', 4096, 4096, 4096, 0.0, 1), ragged_s = per_launch_us(false, 'N', 'T', 4000, 4096, 4096, 0.0, 1);
    f.edge_rounds[0] = std::min(2.0, std::max(0.0, (ragged_s - whole_s) / (0.5 * whole_s)));
  }
  unsetenv("PARALIA_GEMM_LARGE_TILE");
  // what joining the k-steps of a C tile into one launch saves per launch saved, as the scheduler issues them (beta = 1,
  // two streams, the launcher's own tile choice): 32 launches of 4096^3 against 8 of 4096 x 4096 x 16384, the same
  // flops, 24 launches fewer.  The saving is 2 % of either time, so the two are timed in turn and the median of the
  // differences is taken.  Per 4096 x 4096 of C, i.e. per round of 256 large or two rounds of 512 small tiles; the
  // planner scales it by the area.
  for (int t = 0; t < 4; ++t) {
    auto timed = [&](long K, int n) {
      const long lda = tas[t] == 'N' ? 4096 : K, ldb = tbs[t] == 'N' ? K : 4096;
      const double t0 = csecond();
      for (int i = 0; i < n; ++i)
        must(pl_sgemm_tile(tas[t], tbs[t], 4096, 4096, K, 1e-3f, (const float*)A, lda, (const float*)B, ldb, 1.0f,
                           (float*)((char*)C + (size_t)(i % 2) * 4096 * 4096 * 4), 4096, st[i % 2]), "gemm");
      for (auto& q : st) must(pl_stream_sync(q), "sync");
      return csecond() - t0;
    };
    timed(4096, 8); timed(16384, 2);
    std::vector<double> saved;
    for (int rep = 0; rep < (quick ? 5 : 9); ++rep) saved.push_back((timed(4096, 32) - timed(16384, 8)) / 24.0 * 1e6);
    std::sort(saved.begin(), saved.end());
    k.merge_saving_us_f32[t] = std::max(0.0, saved[saved.size() / 2]);
  }
  k.merge_saving_us_f64 = f.splitk_launch_us;
  // a slab of a thin start, two launches sharing the device: 2048 x 2048 x 1024 against half of 2048^3
  {
    const double full = per_launch_us(true, 'N', 'N', 2048, 2048, 2048, 1.0, 2);
    const double half = per_launch_us(true, 'N', 'N', 2048, 2048, 1024, 1.0, 2);
    k.slab_fixed_us = std::max(0.0, half - 0.5 * full);
  }
  char out[1024];
  snprintf(out, sizeof out, "%s/Processed/Kernel-fit_dev-0.log", db.c_str());
  FILE* fp = fopen(out, "w");
  if (!fp) { fprintf(stderr, "cannot write %s\n", out); exit(1); }
  fprintf(fp, "# constants of the tile-GEMM launcher's cost model and of the plan simulator, microseconds unless named otherwise\n");
  fprintf(fp, "lone_us_per_k_f64: %.6g\nlone_us_per_k_f32: %.6g\nlone_fixed_k: %.6g\nsplitk_launch_us: %.6g\npass_bytes_per_us: %.6g\n",
          f.lone_us_per_k[0], f.lone_us_per_k[1], f.lone_fixed_k, f.splitk_launch_us, f.pass_bytes_per_us);
  fprintf(fp, "f32_small_us_per_k: %.6g\nf32_small_fixed_us: %.6g\nf32_wide_gain: %.6g\nf32_wide_fixed_us_beta0: %.6g\nf32_wide_fixed_us_beta1: %.6g\n",
          f.f32_small_us_per_k, f.f32_small_fixed_us, f.f32_wide_gain, f.f32_wide_fixed_us[0], f.f32_wide_fixed_us[1]);
  fprintf(fp, "edge_rounds_small: %.6g\nedge_rounds_large: %.6g\n", f.edge_rounds[0], f.edge_rounds[1]);
  static const char* const trans[4] = {"NN", "NT", "TN", "TT"};
  for (int t = 0; t < 4; ++t)
    fprintf(fp, "f32_large_gain_%s: %.6g\nf32_large_fixed_us_beta0_%s: %.6g\nf32_large_fixed_us_beta1_%s: %.6g\nmerge_saving_us_f32_%s: %.6g\n", trans[t],
            f.f32_large_gain[t], trans[t], f.f32_large_fixed_us[t][0], trans[t], f.f32_large_fixed_us[t][1], trans[t], k.merge_saving_us_f32[t]);
  fprintf(fp, "merge_saving_us_f64: %.6g\ngeadd_bytes_per_s: %.6g\nslab_fixed_us: %.6g\n", k.merge_saving_us_f64, k.geadd_bytes_per_s, k.slab_fixed_us);
  fprintf(fp, "# not measured by this tool: the share of a streamed call's launches that run without a partner, fitted to streamed calls\n");
  fprintf(fp, "lone_share: %.6g\n", k.lone_share);
  fclose(fp);
  fprintf(stderr, "kernel fit: lone workgroup %.4f (fp64) / %.4f (fp32) us per k + %.0f k, launch gap %.2f us, scale-add %.2f / %.2f TB/s\n",
          f.lone_us_per_k[0], f.lone_us_per_k[1], f.lone_fixed_k, f.splitk_launch_us, f.pass_bytes_per_us / 1e6, k.geadd_bytes_per_s / 1e12);
  fprintf(stderr, "kernel fit: fp32 small %.4f us per k + %.1f us; wide gain %.3f, fixed %.1f | %.1f us; slab +%.2f us\n", f.f32_small_us_per_k,
          f.f32_small_fixed_us, f.f32_wide_gain, f.f32_wide_fixed_us[0], f.f32_wide_fixed_us[1], k.slab_fixed_us);
  fprintf(stderr, "kernel fit: ragged edge + %.3f (128 x 128 tiles) / + %.3f (256-wide) of a round\n", f.edge_rounds[0], f.edge_rounds[1]);
  for (int t = 0; t < 4; ++t)
    fprintf(stderr, "kernel fit: fp32 large %s gain %.3f, fixed %.1f | %.1f us\n", trans[t], f.f32_large_gain[t], f.f32_large_fixed_us[t][0], f.f32_large_fixed_us[t][1]);
  for (auto s : st) pl_stream_destroy(s);
  CoCoFree(A, 0); CoCoFree(B, 0); CoCoFree(C, 0);
}

static void bench_link(const std::string& db, bool quick) {
  const long maxDim = quick ? 4352 : 10000;
  std::vector<long> dims = sweep(256, 256, maxDim, 8);
  const long ldh = maxDim + 1;
  double* host = (double*)CoCoMalloc(ldh * maxDim * 8, -1, 1);
  double* host2 = (double*)CoCoMalloc(ldh * maxDim * 8, -1, 1);
  double* dev = (double*)CoCoMalloc(maxDim * maxDim * 8, 0, 1);
  double* dev2 = (double*)CoCoMalloc(maxDim * maxDim * 8, 0, 1);
  CoCoVecInit(host, ldh * maxDim, 42, -1);
  void *s1, *s2;
  must(pl_stream_create(&s1), "stream");
  must(pl_stream_create(&s2), "stream");
  void* ev;
  must(pl_event_create(&ev, 0), "event");
  struct Dir { int to, from; } dirs[2] = {{0, -1}, {-1, 0}};
  for (const Dir& d : dirs) {
    const bool h2d = d.to == 0;
    char raw[1024];
    snprintf(raw, sizeof raw, "%s/Benchmark-Results/hip_link_benchmark_loc_dest-%d_loc_src-%d_%s.log", db.c_str(), d.to, d.from, DEPLOY_VERSION);
    FILE* fp = fopen(raw, "w");
    if (!fp) { fprintf(stderr, "cannot write %s\n", raw); exit(1); }
    auto copy = [&](long dim, void* st, bool forward, double* h, double* dv) {
      if (forward) must(pl_copy2d_async(dv, dim, h, ldh, dim, dim, 8, st), "h2d copy");
      else must(pl_copy2d_async(h, ldh, dv, dim, dim, dim, 8, st), "d2h copy");
    };
    double sx = 0, sy = 0, sxx = 0, sxy = 0;
    long np = 0;
    for (long dim : dims) {
      // the cadence of a stream of tile copies as the scheduler issues them: every copy is followed by an event
      // record (its consumers wait on it), and the batch is long enough that the final sync does not weigh
      const int batch = dim <= 2048 ? 16 : dim <= 4096 ? 8 : 4;
      auto run = [&]() {
        const double t0 = csecond();
        for (int i = 0; i < batch; ++i) {
          copy(dim, s1, h2d, host, dev);
          must(pl_event_record(ev, s1), "event record");
        }
        must(pl_stream_sync(s1), "sync");
        return (csecond() - t0) / batch;
      };
      run();
      Sample s = sample_until_stable(run);
      fprintf(fp, "%ld,%ld, %e,%e,%ld, %e\n", dim, dim, s.mean, s.margin, s.n, s.bench_t);
      fprintf(stderr, "link %d<-%d dim=%ld: %.3f ms (%.1f GB/s)\n", d.to, d.from, dim, s.mean * 1e3, dim * dim * 8.0 / s.mean / 1e9);
      const double b = (double)dim * dim * 8;
      sx += b; sy += s.mean; sxx += b * b; sxy += b * s.mean;
      ++np;
    }
    fclose(fp);
    const double tb = (np * sxy - sx * sy) / (np * sxx - sx * sx);
    const double ti = fabs((sy - tb * sx) / np);
    // overlap: this direction alone vs. while the opposite direction streams tiles of the same size
    const long dim = 2048;
    const int reps = 10;
    auto alone = [&]() {
      const double t0 = csecond();
      for (int i = 0; i < reps; ++i) copy(dim, s1, h2d, host, dev);
      must(pl_stream_sync(s1), "sync");
      return (csecond() - t0) / reps;
    };
    auto shared = [&]() {
      for (int i = 0; i < 3 * reps; ++i) copy(dim, s2, !h2d, host2, dev2);  // keeps the other direction busy throughout
      const double t0 = csecond();
      for (int i = 0; i < reps; ++i) copy(dim, s1, h2d, host, dev);
      must(pl_stream_sync(s1), "sync");
      const double t = (csecond() - t0) / reps;
      must(pl_stream_sync(s2), "sync");
      return t;
    };
    alone();
    const double bench0 = csecond();
    double t_alone = 0, t_shared = 0;
    for (int i = 0; i < 5; ++i) { t_alone += alone() / 5; t_shared += shared() / 5; }
    snprintf(raw, sizeof raw, "%s/Benchmark-Results/hip_link_overlap_benchmark_loc_dest-%d_loc_src-%d_%s.log", db.c_str(), d.to, d.from, DEPLOY_VERSION);
    fp = fopen(raw, "w");
    if (!fp) { fprintf(stderr, "cannot write %s\n", raw); exit(1); }
    fprintf(fp, "%d,%d, %e,%e,%d, %e\n", d.from, d.to, t_alone, t_shared, reps, csecond() - bench0);
    fclose(fp);
    char out[1024];
    snprintf(out, sizeof out, "%s/Processed/Link-Stats_loc_dest-%d_loc_src-%d.log", db.c_str(), d.to, d.from);
    fp = fopen(out, "w");
    if (!fp) { fprintf(stderr, "cannot write %s\n", out); exit(1); }
    fprintf(fp, "Intercept: %.12e\nCoefficient: %.12e\n", ti, tb);
    // the "other link" is the opposite direction: traffic from d.to to d.from
    fprintf(fp, "Slowdown([%d]->[%d]): %.6f\n", d.to, d.from, t_shared / t_alone);
    fclose(fp);
    fprintf(stderr, "link %d<-%d: ti = %.3e s, tb = %.3e s/B (%.1f GB/s), slowdown under opposing traffic %.3f\n", d.to, d.from, ti, tb,
            1e-9 / tb, t_shared / t_alone);
  }
  pl_stream_destroy(s1);
  pl_stream_destroy(s2);
  pl_event_destroy(ev);
  CoCoFree(host, -1); CoCoFree(host2, -1); CoCoFree(dev, 0); CoCoFree(dev2, 0);
}

int main(int argc, char** argv) {
  if (argc < 2) {
    fprintf(stderr, "usage: %s <db_dir> [--quick] [--only gemm|gemv|blas1|link|fit]\n", argv[0]);
    return 2;
  }
  const std::string db = argv[1];
  bool quick = false;
  std::string only;
  for (int i = 2; i < argc; ++i) {
    if (!strcmp(argv[i], "--quick")) quick = true;
    else if (!strcmp(argv[i], "--only") && i + 1 < argc) only = argv[++i];
  }
  try {
    mkdirs(db);
    must(pl_set_device(0), "set device");
    char name[256];
    must(pl_device_name(0, name, sizeof name), "device name");
    fprintf(stderr, "paralia_deploy: device 0 = %s, database -> %s%s\n", name, db.c_str(), quick ? " (quick sweep)" : "");
    const char* q_env = getenv("PARALIA_EXEC_QUEUES");
    const int queues = (q_env && atoi(q_env) > 0) ? std::min(atoi(q_env), 8) : 2;
    if (only.empty() || only == "link") bench_link(db, quick);
    if (only.empty() || only == "gemm") {
      bench_gemm<double>(db, "Dgemm", quick, queues);
      bench_gemm<float>(db, "Sgemm", quick, queues);
      bench_transient(db);
    }
    if (only.empty() || only == "gemm" || only == "fit") bench_fit(db, quick);
    if (only.empty() || only == "gemv") bench_gemv(db, quick);
    if (only.empty() || only == "blas1") {
      bench_blas1(db, "Daxpy", quick);
      bench_blas1(db, "Ddot", quick);
    }
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s\n", e.what());
    return 1;
  }
  return 0;
}
