///
/// Shared pieces of the PARALiA drivers: command-line parsing, log rows, the OpenBLAS loader used for
/// validation.  Argument order, location codes, row formats and the warm-up / iteration protocol follow the
/// reference's Benchmarking/CuCuBLAS/src/testing.cpp:159-428 and PARALia/dgemm_runner.cpp:16-160; validation is
/// against OpenBLAS (the reference's own CPU library) instead of cuBLASXt.
///
#ifndef PARALIA_TESTING_HPP
#define PARALIA_TESTING_HPP

#include <dlfcn.h>
#include <glob.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "PARALiA.hpp"
#include "backend_wrappers.hpp"

#define DRIVER_VERSION "2.0"

inline std::string test_log_dir() {
  const char* d = getenv("PARALIA_TESTLIBDIR");
  return d && *d ? d : ".";
}

/// Names the reference's drivers build their log file names from (dgemm_runner.cpp:33-37:
/// "%s/CoCoPeLiaDgemmRunner_%s_%s.log" with TESTLIBDIR, CoCoImplementationPrint() and VERSION).  There TESTLIBDIR and
/// VERSION are compile definitions of its build; here they default to $PARALIA_TESTLIBDIR (or ".") and the driver
/// version, and a build may still define them.
inline const char* CoCoImplementationPrint() { return "MI355X"; }
inline const char* paralia_testlibdir_cstr() {
  static const std::string dir = test_log_dir();
  return dir.c_str();
}
#ifndef TESTLIBDIR
#define TESTLIBDIR (paralia_testlibdir_cstr())
#endif
#ifndef VERSION
#define VERSION DRIVER_VERSION
#endif

inline ATC_p parse_control(const char* fn, const char* argv[]) {
  const int active_unit_num = atoi(argv[1]);
  long dev_ids_token = atoi(argv[2]);
  const int T = atoi(argv[3]);
  const long long cache_limit = (long long)atof(argv[4]);
  if (active_unit_num < 0 && cache_limit <= 0 && T <= 0) return NULL;
  fprintf(stderr, "Using predefined control parameters from input\n");
  ATC_p p = new ATC();
  p->cache_limit = cache_limit > 0 ? cache_limit : 0;
  p->T = T > 0 ? T : -1;
  if (active_unit_num < 0) p->active_unit_num = -1;
  else {
    p->active_unit_num = active_unit_num;
    int ctr = 0, itter = 0;
    do {
      if (dev_ids_token % 10 == 1 && ctr < LOC_NUM) p->active_unit_id_list[ctr++] = deidxize(itter);
      itter++;
      dev_ids_token /= 10;
    } while (dev_ids_token > 0);
    if (ctr != active_unit_num)
      error("%s: Read different device Ids in total (%d) than active_unit_num implied (%d)\n", fn, ctr, active_unit_num);
  }
  return p;
}

inline void ParseInputLvl1(const int argc, const char* argv[], ATC_p* predef, double* alpha, long int* D1, long int* inc1,
                           long int* inc2, short* loc1, short* loc2, short* outloc1, short* outloc2) {
  if (argc != 13)
    error("Incorrect input arguments. Usage: ./correct_run\n\tactive_unit_num(auto if <0)\n\tdev_ids(form example: 0101 for "
          "devices 0,2 - ignore if active_unit_num < 0)\n\tT(auto if <=0)\n\tcache_max_size(auto if <0)\n\t alpha D1 inc1 inc2 "
          "loc1 loc2 outloc1 outloc2\n");
  *predef = parse_control("ParseInputLvl1", argv);
  *alpha = atof(argv[5]);
  *D1 = atol(argv[6]);
  *inc1 = atol(argv[7]);
  *inc2 = atol(argv[8]);
  *loc1 = atoi(argv[9]);
  *loc2 = atoi(argv[10]);
  *outloc1 = atoi(argv[11]);
  *outloc2 = atoi(argv[12]);
  fprintf(stderr, "ParseInputLvl1: ");
  if (*predef) (*predef)->print();
  fprintf(stderr, "Routine values:\talpha: %lf\n\tD1: %zu, inc1: %zu, inc2: %zu\n\tloc1: %d, loc2: %d, outloc1: %d, outloc2: %d\n",
          *alpha, (size_t)*D1, (size_t)*inc1, (size_t)*inc2, *loc1, *loc2, *outloc1, *outloc2);
}

/// argv of the BLAS-2 drivers (testing.cpp:215-271):
///   active_unit_num dev_ids_token T cache_limit TransA alpha beta D1 D2 inc1 inc2 loc1 loc2 loc3 outloc
inline void ParseInputLvl2(const int argc, const char* argv[], ATC_p* predef, char* TransA, double* alpha, double* beta,
                           long int* D1, long int* D2, long int* inc1, long int* inc2, short* loc1, short* loc2, short* loc3,
                           short* outloc) {
  if (argc != 16)
    error("Incorrect input arguments. Usage: ./correct_run\n\tactive_unit_num(auto if <0)\n\tdev_ids(form example: 0101 for devices 0,2 - "
          "ignore if active_unit_num < 0)\n\tT(auto if <=0)\n\tcache_max_size(auto if <0)\n\tTransA alpha beta D1 D2 inc1 inc2 loc1 loc2 loc3 "
          "outloc \n");
  *predef = parse_control("ParseInputLvl2", argv);
  *TransA = argv[5][0];
  *alpha = atof(argv[6]);
  *beta = atof(argv[7]);
  *D1 = atol(argv[8]);
  *D2 = atol(argv[9]);
  *inc1 = atol(argv[10]);
  *inc2 = atol(argv[11]);
  *loc1 = atoi(argv[12]);
  *loc2 = atoi(argv[13]);
  *loc3 = atoi(argv[14]);
  *outloc = atoi(argv[15]);
  fprintf(stderr, "ParseInputLvl2: ");
  if (*predef) (*predef)->print();
  fprintf(stderr, "Routine values:\n\tTransA: %c\n\talpha: %lf, beta: %lf\n\tD1: %zu, D2: %zu, inc1: %zu, inc2: %zu\n\tloc1: %d, loc2: %d, "
          "loc3: %d, outloc: %d\n", *TransA, *alpha, *beta, (size_t)*D1, (size_t)*D2, (size_t)*inc1, (size_t)*inc2, *loc1, *loc2, *loc3, *outloc);
}

inline void ParseInputLvl3(const int argc, const char* argv[], ATC_p* predef, char* TransA, char* TransB, double* alpha,
                           double* beta, long int* D1, long int* D2, long int* D3, short* loc1, short* loc2, short* loc3,
                           short* outloc) {
  if (argc != 16)
    error("Incorrect input arguments. Usage: ./correct_run\n\tactive_unit_num(auto if <0)\n\tdev_ids(form example: 0101 for "
          "devices 0,2 - ignore if active_unit_num < 0)\n\tT(auto if <=0)\n\tcache_max_size(auto if <0)\n\tTransA TransB alpha "
          "beta D1 D2 D3 loc1 loc2 loc3 outloc \n");
  *predef = parse_control("ParseInputLvl3", argv);
  *TransA = argv[5][0];
  *TransB = argv[6][0];
  *alpha = atof(argv[7]);
  *beta = atof(argv[8]);
  *D1 = atol(argv[9]);
  *D2 = atol(argv[10]);
  *D3 = atol(argv[11]);
  *loc1 = atoi(argv[12]);
  *loc2 = atoi(argv[13]);
  *loc3 = atoi(argv[14]);
  *outloc = atoi(argv[15]);
  fprintf(stderr, "ParseInputLvl3: ");
  if (*predef) (*predef)->print();
  fprintf(stderr, "Routine values:\n\tTransA: %c, TransB: %c\n\talpha: %lf, beta: %lf\n\tD1: %zu, D2: %zu, D3: %zu\n\tloc1: %d, "
          "loc2: %d, loc3: %d, outloc: %d\n", *TransA, *TransB, *alpha, *beta, (size_t)*D1, (size_t)*D2, (size_t)*D3, *loc1, *loc2,
          *loc3, *outloc);
}

/// "T,units,dev_token,cache, alpha,D1,inc1,inc2,loc1,loc2,outloc1,outloc2, t,pred_t,pred_J"
/// (the reference row, testing.cpp:402, ends after outloc2 without a newline; the timing columns are added here)
inline void StoreLogLvl1(const char* filename, ATC_p ctl, double alpha, long int D1, long int inc1, long int inc2, short loc1,
                         short loc2, short outloc1, short outloc2, double timer, double pred_t, double pred_J) {
  FILE* fp = fopen(filename, "a");
  if (!fp) error("report_results: LogFile failed to open");
  const char* control_str = ctl ? ctl->print_csv() : "-1,-1,-1,-1";
  fprintf(fp, "%s, %.5lf,%zu,%zu,%zu,%d,%d,%d,%d, %e,%e,%e\n", control_str, alpha, (size_t)D1, (size_t)inc1, (size_t)inc2, loc1, loc2,
          outloc1, outloc2, timer, pred_t, pred_J);
  fclose(fp);
}

/// "T,units,dev_token,cache, TransA,alpha,beta,D1,D2,inc1,inc2,loc1,loc2,loc3,outloc, t,pred_t,pred_J" (testing.cpp:414)
inline void StoreLogLvl2(const char* filename, ATC_p ctl, char TransA, double alpha, double beta, long int D1, long int D2,
                         long int inc1, long int inc2, short loc1, short loc2, short loc3, short outloc, double timer, double pred_t,
                         double pred_J) {
  FILE* fp = fopen(filename, "a");
  if (!fp) error("report_results: LogFile failed to open");
  const char* control_str = ctl ? ctl->print_csv() : "-1,-1,-1,-1";
  fprintf(fp, "%s, %c,%.5lf,%.5lf,%zu,%zu,%zu,%zu,%d,%d,%d,%d, %e,%e,%e\n", control_str, TransA, alpha, beta, (size_t)D1, (size_t)D2,
          (size_t)inc1, (size_t)inc2, loc1, loc2, loc3, outloc, timer, pred_t, pred_J);
  fclose(fp);
}

/// "T,units,dev_token,cache, TransA,TransB,alpha,beta,D1,D2,D3,loc1,loc2,loc3,outloc, t,pred_t,pred_J" (testing.cpp:424)
inline void StoreLogLvl3(const char* filename, ATC_p ctl, char TransA, char TransB, double alpha, double beta, long int D1,
                         long int D2, long int D3, short loc1, short loc2, short loc3, short outloc, double timer, double pred_t,
                         double pred_J) {
  FILE* fp = fopen(filename, "a");
  if (!fp) error("report_results: LogFile failed to open");
  const char* control_str = ctl ? ctl->print_csv() : "-1,-1,-1,-1";
  fprintf(fp, "%s, %c,%c,%.5lf,%.5lf,%zu,%zu,%zu,%d,%d,%d,%d, %e,%e,%e\n", control_str, TransA, TransB, alpha, beta, (size_t)D1,
          (size_t)D2, (size_t)D3, loc1, loc2, loc3, outloc, timer, pred_t, pred_J);
  fclose(fp);
}

/// The CHECKLOG step of the reference's drivers (testing.cpp:331-397): when the log already holds a row for exactly
/// this configuration the benchmark is not repeated -- the program says so and exits with status 1.  A missing log
/// file is created.  `ctl` is the preset controller before the run and the returned one after it.
inline void paralia_check_log(const char* who, const char* filename, const char* search_string) {
  FILE* fp = fopen(filename, "r");
  if (!fp) {
    fp = fopen(filename, "w+");
    if (!fp) error("%s: LogFile %s failed to open\n", who, filename);
    warning("%s: Generating Logfile %s...\n", who, filename);
  }
  char buffer[1024];
  while (fgets(buffer, sizeof(buffer), fp) != NULL)
    if (strstr(buffer, search_string) != NULL) {
      fprintf(stderr, "%s: entry %s found. Quiting...\n", who, search_string);
      fclose(fp);
      exit(1);
    }
  fclose(fp);
}
inline void CheckLogLvl1(const char* filename, ATC_p ctl, double alpha, long int D1, long int inc1, long int inc2, short loc1,
                         short loc2, short outloc1, short outloc2) {
  char key[1024];
  snprintf(key, sizeof key, "%s, %.5lf,%zu,%zu,%zu,%d,%d,%d,%d", ctl ? ctl->print_csv() : "-1,-1,-1,-1", alpha, (size_t)D1, (size_t)inc1,
           (size_t)inc2, loc1, loc2, outloc1, outloc2);
  paralia_check_log("CheckLogLvl1", filename, key);
}
inline void CheckLogLvl2(const char* filename, ATC_p ctl, char TransA, double alpha, double beta, long int D1, long int D2,
                         long int inc1, long int inc2, short loc1, short loc2, short loc3, short outloc) {
  char key[1024];
  snprintf(key, sizeof key, "%s, %c,%.5lf,%.5lf,%zu,%zu,%zu,%zu,%d,%d,%d,%d", ctl ? ctl->print_csv() : "-1,-1,-1,-1", TransA, alpha, beta,
           (size_t)D1, (size_t)D2, (size_t)inc1, (size_t)inc2, loc1, loc2, loc3, outloc);
  paralia_check_log("CheckLogLvl2", filename, key);
}
inline void CheckLogLvl3(const char* filename, ATC_p ctl, char TransA, char TransB, double alpha, double beta, long int D1,
                         long int D2, long int D3, short loc1, short loc2, short loc3, short outloc) {
  char key[1024];
  snprintf(key, sizeof key, "%s, %c,%c,%.5lf,%.5lf,%zu,%zu,%zu,%d,%d,%d,%d", ctl ? ctl->print_csv() : "-1,-1,-1,-1", TransA, TransB, alpha,
           beta, (size_t)D1, (size_t)D2, (size_t)D3, loc1, loc2, loc3, outloc);
  paralia_check_log("CheckLogLvl3", filename, key);
}

// ------------------------------------------------------------------------------------------------------------------
// OpenBLAS, found at run time: $PARALIA_OPENBLAS_LIB, a system libopenblas, or the copy bundled with NumPy / SciPy
// (symbols scipy_cblas_*64_ with 64-bit integers, or scipy_cblas_* / cblas_* with 32-bit ones).
struct OpenBlas {
  void* h = nullptr;
  bool ilp64 = false;
  void *dgemm = nullptr, *sgemm = nullptr, *dgemv = nullptr, *daxpy = nullptr, *ddot = nullptr, *cfg = nullptr, *setthr = nullptr;
  std::string path;
  bool try_open(const char* p) {
    void* hh = dlopen(p, RTLD_NOW | RTLD_LOCAL);
    if (!hh) return false;
    const char* pre[] = {"cblas_", "scipy_cblas_"};
    const char* suf[] = {"", "64_"};
    for (int s = 0; s < 2; ++s)
      for (int q = 0; q < 2; ++q) {
        const std::string base = pre[q], tail = suf[s];
        void* f = dlsym(hh, (base + "dgemm" + tail).c_str());
        if (!f) continue;
        dgemm = f;
        sgemm = dlsym(hh, (base + "sgemm" + tail).c_str());
        dgemv = dlsym(hh, (base + "dgemv" + tail).c_str());
        daxpy = dlsym(hh, (base + "daxpy" + tail).c_str());
        ddot = dlsym(hh, (base + "ddot" + tail).c_str());
        const std::string ob = q ? "scipy_openblas_" : "openblas_";
        cfg = dlsym(hh, (ob + "get_config" + tail).c_str());
        setthr = dlsym(hh, (ob + "set_num_threads" + tail).c_str());
        ilp64 = s == 1;
        h = hh;
        path = p;
        return sgemm && daxpy && ddot;
      }
    dlclose(hh);
    return false;
  }
  bool open() {
    if (h) return true;
    const char* env = getenv("PARALIA_OPENBLAS_LIB");
    if (env && !strcmp(env, "none")) return false;  // run as on a machine without OpenBLAS (the host-computed references)
    if (env && *env && try_open(env)) return true;
    for (const char* p : {"libopenblas.so.0", "libopenblas.so", "libopenblas64_.so.0"})
      if (try_open(p)) return true;
    for (const char* pat : {"/usr/local/lib/python3*/dist-packages/numpy.libs/libscipy_openblas*.so",
                            "/usr/local/lib/python3*/dist-packages/scipy.libs/libscipy_openblas*.so",
                            "/usr/lib/python3*/dist-packages/numpy.libs/libscipy_openblas*.so",
                            "/opt/conda/lib/python3*/site-packages/numpy.libs/libscipy_openblas*.so"}) {
      glob_t g;
      if (glob(pat, 0, NULL, &g) == 0) {
        for (size_t k = 0; k < g.gl_pathc; ++k)
          if (try_open(g.gl_pathv[k])) { globfree(&g); return true; }
        globfree(&g);
      }
    }
    return false;
  }
  const char* config() const { return cfg ? ((const char* (*)(void))cfg)() : "unknown"; }
  void threads(int n) const { if (setthr) ((void (*)(int))setthr)(n); }
  void Dgemm(char ta, char tb, long M, long N, long K, double al, const double* A, long lda, const double* B, long ldb, double be,
             double* C, long ldc) const {
    const int a = (ta == 'T') ? 112 : 111, b = (tb == 'T') ? 112 : 111;
    if (ilp64) ((void (*)(int, int, int, int64_t, int64_t, int64_t, double, const double*, int64_t, const double*, int64_t, double, double*, int64_t))dgemm)(102, a, b, M, N, K, al, A, lda, B, ldb, be, C, ldc);
    else ((void (*)(int, int, int, int, int, int, double, const double*, int, const double*, int, double, double*, int))dgemm)(102, a, b, (int)M, (int)N, (int)K, al, A, (int)lda, B, (int)ldb, be, C, (int)ldc);
  }
  void Sgemm(char ta, char tb, long M, long N, long K, float al, const float* A, long lda, const float* B, long ldb, float be,
             float* C, long ldc) const {
    const int a = (ta == 'T') ? 112 : 111, b = (tb == 'T') ? 112 : 111;
    if (ilp64) ((void (*)(int, int, int, int64_t, int64_t, int64_t, float, const float*, int64_t, const float*, int64_t, float, float*, int64_t))sgemm)(102, a, b, M, N, K, al, A, lda, B, ldb, be, C, ldc);
    else ((void (*)(int, int, int, int, int, int, float, const float*, int, const float*, int, float, float*, int))sgemm)(102, a, b, (int)M, (int)N, (int)K, al, A, (int)lda, B, (int)ldb, be, C, (int)ldc);
  }
  void Dgemv(char ta, long M, long N, double al, const double* A, long lda, const double* x, long incx, double be, double* y,
             long incy) const {
    const int a = (ta == 'T') ? 112 : 111;
    if (ilp64) ((void (*)(int, int, int64_t, int64_t, double, const double*, int64_t, const double*, int64_t, double, double*, int64_t))dgemv)(102, a, M, N, al, A, lda, x, incx, be, y, incy);
    else ((void (*)(int, int, int, int, double, const double*, int, const double*, int, double, double*, int))dgemv)(102, a, (int)M, (int)N, al, A, (int)lda, x, (int)incx, be, y, (int)incy);
  }
  void Daxpy(long n, double al, const double* x, long incx, double* y, long incy) const {
    if (ilp64) ((void (*)(int64_t, double, const double*, int64_t, double*, int64_t))daxpy)(n, al, x, incx, y, incy);
    else ((void (*)(int, double, const double*, int, double*, int))daxpy)((int)n, al, x, (int)incx, y, (int)incy);
  }
  double Ddot(long n, const double* x, long incx, const double* y, long incy) const {
    if (ilp64) return ((double (*)(int64_t, const double*, int64_t, const double*, int64_t))ddot)(n, x, incx, y, incy);
    return ((double (*)(int, const double*, int, const double*, int))ddot)((int)n, x, (int)incx, y, (int)incy);
  }
};

/// Validation without OpenBLAS: `samples` entries of C, spread over the matrix by a fixed stride walk, are recomputed
/// with a long double dot product from the same host copies of A, B and the original C, and the worst number of
/// matching decimal digits is returned (differences are taken relative to max(|ref|, |x|, rms of the sampled refs), as
/// Dtest_equality does).  A wrong tile index, a dropped k-step or a wrong beta schedule hits every sample of its tile.
template <typename T>
inline short sampled_gemm_digits(char ta, char tb, long M, long N, long K, T alpha, const T* A, long ldA, const T* B, long ldB, T beta,
                                 const T* C0, const T* C, long ldC, int samples = 512) {
  const bool at = ta == 'T' || ta == 't', bt = tb == 'T' || tb == 't';
  const int cap = sizeof(T) == 8 ? 16 : 7;
  std::vector<long double> ref(samples);
  std::vector<double> got(samples);
  uint64_t state = 0x9E3779B97F4A7C15ULL;
  long double ss = 0;
  for (int s = 0; s < samples; ++s) {
    state = state * 6364136223846793005ULL + 1442695040888963407ULL;
    const long i = (long)((state >> 33) % (uint64_t)M);
    state = state * 6364136223846793005ULL + 1442695040888963407ULL;
    const long j = (long)((state >> 33) % (uint64_t)N);
    long double acc = 0;
    for (long k = 0; k < K; ++k)
      acc += (long double)(at ? A[k + i * ldA] : A[i + k * ldA]) * (long double)(bt ? B[j + k * ldB] : B[k + j * ldB]);
    ref[s] = (long double)alpha * acc + (beta == T(0) ? 0.0L : (long double)beta * (long double)C0[i + j * ldC]);
    got[s] = (double)C[i + j * ldC];
    ss += ref[s] * ref[s];
  }
  const double rms = samples > 0 ? (double)sqrtl(ss / samples) : 0.0;
  int worst = cap;
  for (int s = 0; s < samples; ++s) {
    const double d = fabs((double)ref[s] - got[s]);
    if (d == 0) continue;
    if (std::isnan(d)) return 0;
    const double scale = fmax(fmax(fabs((double)ref[s]), fabs(got[s])), rms);
    int digits = (int)floor(-log10(d / scale));
    if (digits < 0) digits = 0;
    if (digits < worst) worst = digits;
  }
  return (short)worst;
}

/// Host copy of a buffer at any location (caller frees with free()).
template <typename T> inline T* host_copy(T* src, long long n, short loc) {
  T* out = (T*)malloc(n * sizeof(T));
  if (!out) error("host_copy: out of memory\n");
  CoCoMemcpy(out, src, n * sizeof(T), -2, loc);
  return out;
}


/// The timing protocol the runners share (PARALia/dgemm_runner.cpp:165-215 and its siblings): optionally one timed
/// first call, `warmups` untimed calls, then `iterations` calls timed one by one, each handed to log_row(seconds,
/// returned control values).  Where there is a first call the minimum starts from its time, as the reference's does.
struct ProtocolTimes {
  double first = -1, avg = 0, min = 1e9, max = 0;
  ATC_p info = NULL;
};
template <typename Call, typename AfterFirst, typename Log>
inline ProtocolTimes run_protocol(Call&& call, bool timed_first, int warmups, int iterations, AfterFirst&& after_first, Log&& log_row) {
  ProtocolTimes t;
  if (timed_first) {
    const double t0 = csecond();
    t.info = call();
    CoCoSyncCheckErr();
    t.first = t.min = csecond() - t0;
    after_first(t.info);
  }
  for (int it = 0; it < warmups; ++it) t.info = call();
  CoCoSyncCheckErr();
  for (int it = 0; it < iterations; ++it) {
    const double t0 = csecond();
    t.info = call();
    CoCoSyncCheckErr();
    const double dt = csecond() - t0;
    log_row(dt, t.info);
    if (dt < t.min) t.min = dt;
    if (dt > t.max) t.max = dt;
    t.avg += dt;
  }
  t.avg /= iterations;
  return t;
}

/// The block every runner ends with: first / avg / min / max in ms with Gflops/s (and GB/s of `bytes` when bytes > 0),
/// and the predicted time with `selected` behind it when there is one.
inline void report_protocol(const ProtocolTimes& t, double flops, double bytes, const char* selected) {
  auto line = [&](const char* name, double seconds) {
    if (bytes > 0) fprintf(stderr, "\t%s = %lf ms ( %lf Gflops/s, %lf GB/s )\n", name, seconds * 1000, Gval_per_s(flops, seconds), bytes / seconds / 1e9);
    else fprintf(stderr, "\t%s = %lf ms ( %lf Gflops/s )\n", name, seconds * 1000, Gval_per_s(flops, seconds));
  };
  fprintf(stderr, "CoCopeLia (%s):\n", t.info->print_csv());
  if (t.first >= 0) line("first_it_t", t.first);
  line("avg_t", t.avg);
  line("min_t", t.min);
  line("max_t", t.max);
  if (selected) fprintf(stderr, "\tpredicted_t = %lf ms [%s]\n", t.info->pred_t * 1000, selected);
}

#endif
