///
/// PARALiA dgemm / sgemm benchmark driver, shared by dgemm_runner and sgemm_runner.
/// argv (reference Benchmarking/CuCuBLAS/src/testing.cpp:273-329):
///   active_unit_num dev_ids_token T cache_limit TransA TransB alpha beta M N K A_loc B_loc C_loc C_out_loc
/// ("-1 -1 -1 -1" for the first four = fully automatic).  Locations: 0 device, -1 pinned host, -2 pageable host.
/// Protocol of dgemm_runner.cpp:16-160 (fp32 twin: the sgemm path of Library_scheduler/src/Functions/sgemm.cpp:296):
/// validation (two calls, the second through the metadata cache, compared with OpenBLAS, at least 9 matching digits
/// for fp64 / 4 for fp32), one timed first call, 10 warm-ups (2 for >= 20000^3), 10 timed and logged iterations,
/// first / avg / min / max report.  Set PARALIA_SKIP_VALIDATION=1 to skip the OpenBLAS run.
///
#ifndef PARALIA_GEMM_RUNNER_HPP
#define PARALIA_GEMM_RUNNER_HPP
#include "Testing.hpp"

template <typename T> struct RunnerFns;
template <> struct RunnerFns<double> {
  static constexpr const char* name = "Dgemm";
  static constexpr const char* cblas = "cblas_dgemm";
  static constexpr short min_digits = 9;
  static ATC_p gemm(char ta, char tb, long M, long N, long K, double al, double* A, long lda, double* B, long ldb, double be, double* C, long ldc) {
    return PARALiADgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static ATC_p controlled(char ta, char tb, long M, long N, long K, double al, double* A, long lda, double* B, long ldb, double be, double* C, long ldc, ATC_p ctl) {
    return PARALiADgemmControled(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ctl);
  }
  static void blas(const OpenBlas& ob, char ta, char tb, long M, long N, long K, double al, double* A, long lda, double* B, long ldb, double be, double* C, long ldc) {
    ob.Dgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static short digits(double* ref, double* x, long long n) { return Dtest_equality(ref, x, n); }
};
template <> struct RunnerFns<float> {
  static constexpr const char* name = "Sgemm";
  static constexpr const char* cblas = "cblas_sgemm";
  static constexpr short min_digits = 4;
  static ATC_p gemm(char ta, char tb, long M, long N, long K, float al, float* A, long lda, float* B, long ldb, float be, float* C, long ldc) {
    return PARALiASgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static ATC_p controlled(char ta, char tb, long M, long N, long K, float al, float* A, long lda, float* B, long ldb, float be, float* C, long ldc, ATC_p ctl) {
    return PARALiASgemmControled(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ctl);
  }
  static void blas(const OpenBlas& ob, char ta, char tb, long M, long N, long K, float al, float* A, long lda, float* B, long ldb, float be, float* C, long ldc) {
    ob.Sgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static short digits(float* ref, float* x, long long n) { return Stest_equality(ref, x, n); }
};


template <typename T> int run_gemm_runner(const int argc, const char* argv[]) {
  using F = RunnerFns<T>;
  try {
    char TransA, TransB;
    double alpha, beta;
    long int M, N, K;
    short A_loc, B_loc, C_loc, C_out_loc;
    ATC_p predef_control_values = NULL, return_values = NULL;
    ParseInputLvl3(argc, argv, &predef_control_values, &TransA, &TransB, &alpha, &beta, &M, &N, &K, &A_loc, &B_loc, &C_loc, &C_out_loc);

    char filename[1024];
    if (predef_control_values != NULL) {
      if (predef_control_values->T > 0) {
        if (predef_control_values->T > M || predef_control_values->T > N)
          error("Given Tin=%ld bigger than problem dim\n", predef_control_values->T);
        else if (predef_control_values->T > K)
          warning("Given Tin=%ld bigger than K=%ld: tiles are %ld deep\n", predef_control_values->T, K, K);
      }
      snprintf(filename, sizeof filename, "%s/CoCoPeLia%sRunner_predefined_vals_MI355X_%s.log", test_log_dir().c_str(), F::name, DRIVER_VERSION);
    } else {
      snprintf(filename, sizeof filename, "%s/CoCoPeLia%sRunner_MI355X_%s.log", test_log_dir().c_str(), F::name, DRIVER_VERSION);
    }
    // the reference builds its drivers with or without CHECKLOG (dgemm_runner.cpp:38-40,106-108); here it is a switch
    const char* checklog_env = getenv("PARALIA_CHECKLOG");
    const bool checklog = checklog_env && atoi(checklog_env);
    if (checklog) CheckLogLvl3(filename, predef_control_values, TransA, TransB, alpha, beta, M, N, K, A_loc, B_loc, C_loc, C_out_loc);

    long int ldA, ldB, ldC = M;
    TransposeTranslate(TransA, &ldA, M, K);
    TransposeTranslate(TransB, &ldB, K, N);

    double cpu_timer = csecond();
    fprintf(stderr, "\nAllocating memory...");
    T* A = (T*)CoCoMalloc(M * K * sizeof(T), A_loc, 0);
    T* B = (T*)CoCoMalloc(N * K * sizeof(T), B_loc, 0);
    T* C = (T*)CoCoMalloc(M * N * sizeof(T), C_loc, 1);
    CoCoSyncCheckErr();
    cpu_timer = csecond() - cpu_timer;
    fprintf(stderr, "done.\nAlloc time:\t%lf ms\n\n", cpu_timer * 1000);
    cpu_timer = csecond();
    fprintf(stderr, "Initializing to random values...");
    CoCoVecInit(A, K * M, 42, A_loc);
    CoCoVecInit(B, K * N, 43, B_loc);
    CoCoVecInit(C, M * N, 44, C_loc);
    CoCoSyncCheckErr();
    cpu_timer = csecond() - cpu_timer;
    fprintf(stderr, "done.\nInit time:\t%lf ms\n\n", cpu_timer * 1000);

    auto call = [&]() {
      if (predef_control_values != NULL)
        return F::controlled(TransA, TransB, M, N, K, (T)alpha, A, ldA, B, ldB, (T)beta, C, ldC, predef_control_values);
      return F::gemm(TransA, TransB, M, N, K, (T)alpha, A, ldA, B, ldB, (T)beta, C, ldC);
    };

    const char* skip = getenv("PARALIA_SKIP_VALIDATION");
    if (!(skip && atoi(skip))) {
      OpenBlas ob;
      T* C_start = host_copy(C, M * N, C_loc);
      return_values = call();
      CoCoSyncCheckErr();
      T* C_out = host_copy(C, M * N, C_loc);
      CoCoMemcpy(C, C_start, M * N * sizeof(T), C_loc, -2);
      return_values = call();  // second call: tuned problem served from the metadata cache
      CoCoSyncCheckErr();
      T* C_out1 = host_copy(C, M * N, C_loc);
      if (F::digits(C_out1, C_out, M * N) < F::min_digits) error("Insufficient accuracy for benchmarks, metadata reuse is bugged\n");
      if (ob.open()) {
        fprintf(stderr, "Validating against OpenBLAS (%s)\n%s\n", ob.path.c_str(), ob.config());
        T* hA = host_copy(A, M * K, A_loc);
        T* hB = host_copy(B, N * K, B_loc);
        T* C_ref = (T*)malloc(M * N * sizeof(T));
        memcpy(C_ref, C_start, M * N * sizeof(T));
        cpu_timer = csecond();
        F::blas(ob, TransA, TransB, M, N, K, (T)alpha, hA, ldA, hB, ldB, (T)beta, C_ref, ldC);
        cpu_timer = csecond() - cpu_timer;
        fprintf(stderr, "OpenBLAS %s: %lf ms ( %lf Gflops/s )\n", F::cblas, cpu_timer * 1000, Gval_per_s(gemm_flops(M, N, K), cpu_timer));
        const short digits = F::digits(C_ref, C_out, M * N);
        fprintf(stderr, "Matching digits vs OpenBLAS: %d\n", digits);
        if (digits < F::min_digits) error("Insufficient accuracy for benchmarks\n");
        free(hA); free(hB); free(C_ref);
      } else {
        // no OpenBLAS on this machine: sampled entries against a long double dot product instead
        T* hA = host_copy(A, M * K, A_loc);
        T* hB = host_copy(B, N * K, B_loc);
        const short digits = sampled_gemm_digits<T>(TransA, TransB, M, N, K, (T)alpha, hA, ldA, hB, ldB, (T)beta, C_start, C_out, ldC);
        fprintf(stderr, "OpenBLAS absent: 512 sampled entries against a long double dot product\nMatching digits vs long double samples: %d\n", digits);
        if (digits < F::min_digits) error("Insufficient accuracy for benchmarks\n");
        free(hA); free(hB);
      }
      CoCoMemcpy(C, C_start, M * N * sizeof(T), C_loc, -2);
      free(C_start); free(C_out); free(C_out1);
    }

    // the protocol of the reference's runner: a timed first call, 10 warm-ups (2 for the largest problems), 10 timed
    // and logged iterations
    const int warmups = (M >= 20000 && N >= 20000 && K >= 20000) ? 2 : 10;
    const ProtocolTimes times = run_protocol(
        call, true, warmups, 10,
        [&](ATC_p first) { if (checklog) CheckLogLvl3(filename, first, TransA, TransB, alpha, beta, M, N, K, A_loc, B_loc, C_loc, C_out_loc); },
        [&](double seconds, ATC_p info) {
          StoreLogLvl3(filename, info, TransA, TransB, alpha, beta, M, N, K, A_loc, B_loc, C_loc, C_out_loc, seconds, info->pred_t, info->pred_J);
        });
    return_values = times.info;
    char selected[128];
    snprintf(selected, sizeof selected, "T selected by %s, order %d", return_values->T_selected_by, return_values->order_id);
    report_protocol(times, (double)gemm_flops(M, N, K), 0.0, selected);

    for (int i = 0; i < LOC_NUM; i++) PARALiADevCacheFree(deidxize(i));
    CoCoSyncCheckErr();
    CoCoFree(A, A_loc);
    CoCoFree(B, B_loc);
    CoCoFree(C, C_loc);
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s", e.what());
    return 1;
  }
  return 0;
}

#endif
