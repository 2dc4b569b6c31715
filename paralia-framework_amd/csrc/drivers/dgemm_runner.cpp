///
/// PARALiA dgemm benchmark driver.  argv (reference Benchmarking/CuCuBLAS/src/testing.cpp:273-329):
///   active_unit_num dev_ids_token T cache_limit TransA TransB alpha beta M N K A_loc B_loc C_loc C_out_loc
/// ("-1 -1 -1 -1" for the first four = fully automatic).  Locations: 0 device, -1 pinned host, -2 pageable host.
/// Protocol of dgemm_runner.cpp:16-160: validation (two calls, the second through the metadata cache, compared with
/// OpenBLAS, at least 9 matching digits), one timed first call, 10 warm-ups (2 for >= 20000^3), 10 timed and logged
/// iterations, first / avg / min / max report.  Set PARALIA_SKIP_VALIDATION=1 to skip the OpenBLAS run.
///
#include "Testing.hpp"

int main(const int argc, const char* argv[]) {
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
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDgemmRunner_predefined_vals_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    } else {
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDgemmRunner_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    }

    long int ldA, ldB, ldC = M;
    TransposeTranslate(TransA, &ldA, M, K);
    TransposeTranslate(TransB, &ldB, K, N);

    double cpu_timer = csecond();
    fprintf(stderr, "\nAllocating memory...");
    double* A = (double*)CoCoMalloc(M * K * sizeof(double), A_loc, 0);
    double* B = (double*)CoCoMalloc(N * K * sizeof(double), B_loc, 0);
    double* C = (double*)CoCoMalloc(M * N * sizeof(double), C_loc, 1);
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
        return PARALiADgemmControled(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef_control_values);
      return PARALiADgemm(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC);
    };

    const char* skip = getenv("PARALIA_SKIP_VALIDATION");
    if (!(skip && atoi(skip))) {
      OpenBlas ob;
      double* C_start = host_copy(C, M * N, C_loc);
      return_values = call();
      CoCoSyncCheckErr();
      double* C_out = host_copy(C, M * N, C_loc);
      CoCoMemcpy(C, C_start, M * N * sizeof(double), C_loc, -2);
      return_values = call();  // second call: tuned problem served from the metadata cache
      CoCoSyncCheckErr();
      double* C_out1 = host_copy(C, M * N, C_loc);
      if (Dtest_equality(C_out1, C_out, M * N) < 9) error("Insufficient accuracy for benchmarks, metadata reuse is bugged\n");
      if (ob.open()) {
        fprintf(stderr, "Validating against OpenBLAS (%s)\n%s\n", ob.path.c_str(), ob.config());
        double* hA = host_copy(A, M * K, A_loc);
        double* hB = host_copy(B, N * K, B_loc);
        double* C_ref = (double*)malloc(M * N * sizeof(double));
        memcpy(C_ref, C_start, M * N * sizeof(double));
        cpu_timer = csecond();
        ob.Dgemm(TransA, TransB, M, N, K, alpha, hA, ldA, hB, ldB, beta, C_ref, ldC);
        cpu_timer = csecond() - cpu_timer;
        fprintf(stderr, "OpenBLAS cblas_dgemm: %lf ms ( %lf Gflops/s )\n", cpu_timer * 1000, Gval_per_s(gemm_flops(M, N, K), cpu_timer));
        const short digits = Dtest_equality(C_ref, C_out, M * N);
        fprintf(stderr, "Matching digits vs OpenBLAS: %d\n", digits);
        if (digits < 9) error("Insufficient accuracy for benchmarks\n");
        free(hA); free(hB); free(C_ref);
      } else {
        warning("OpenBLAS absent: result compared only with itself across calls\n");
      }
      CoCoMemcpy(C, C_start, M * N * sizeof(double), C_loc, -2);
      free(C_start); free(C_out); free(C_out1);
    }

    cpu_timer = csecond();
    return_values = call();
    CoCoSyncCheckErr();
    cpu_timer = csecond() - cpu_timer;
    const double first_over_t = cpu_timer;

    short warmup_bench_it = 10;
    if (M >= 20000 && N >= 20000 && K >= 20000) warmup_bench_it = 2;
    for (int it = 0; it < warmup_bench_it; it++) return_values = call();
    CoCoSyncCheckErr();

    double min_t = first_over_t, max_t = 0, avg_t = 0;
    const short bench_it = 10;
    for (int it = 0; it < bench_it; it++) {
      cpu_timer = csecond();
      return_values = call();
      CoCoSyncCheckErr();
      cpu_timer = csecond() - cpu_timer;
      StoreLogLvl3(filename, return_values, TransA, TransB, alpha, beta, M, N, K, A_loc, B_loc, C_loc, C_out_loc, cpu_timer,
                   return_values->pred_t, return_values->pred_J);
      if (cpu_timer < min_t) min_t = cpu_timer;
      if (cpu_timer > max_t) max_t = cpu_timer;
      avg_t += cpu_timer;
    }
    avg_t /= bench_it;
    fprintf(stderr, "CoCopeLia (%s):\n\tfirst_it_t = %lf ms ( %lf Gflops/s )\n\tavg_t = %lf ms ( %lf Gflops/s )\n\tmin_t = %lf ms ( %lf "
            "Gflops/s )\n\tmax_t = %lf ms ( %lf Gflops/s )\n\tpredicted_t = %lf ms [T selected by %s, order %d]\n",
            return_values->print_csv(), first_over_t * 1000, Gval_per_s(gemm_flops(M, N, K), first_over_t), avg_t * 1000,
            Gval_per_s(gemm_flops(M, N, K), avg_t), min_t * 1000, Gval_per_s(gemm_flops(M, N, K), min_t), max_t * 1000,
            Gval_per_s(gemm_flops(M, N, K), max_t), return_values->pred_t * 1000, return_values->T_selected_by, return_values->order_id);

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
