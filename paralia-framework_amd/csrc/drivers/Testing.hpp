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

#include "PARALiA.hpp"
#include "backend_wrappers.hpp"

#define DRIVER_VERSION "2.0"

inline std::string test_log_dir() {
  const char* d = getenv("PARALIA_TESTLIBDIR");
  return d && *d ? d : ".";
}

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

/// Host copy of a buffer at any location (caller frees with free()).
template <typename T> inline T* host_copy(T* src, long long n, short loc) {
  T* out = (T*)malloc(n * sizeof(T));
  if (!out) error("host_copy: out of memory\n");
  CoCoMemcpy(out, src, n * sizeof(T), -2, loc);
  return out;
}

#endif
