///
/// PARALiA dgemv benchmark driver.  argv (reference Benchmarking/CuCuBLAS/src/testing.cpp:215-271):
///   active_unit_num dev_ids_token T cache_limit TransA alpha beta M N incx incy A_loc x_loc y_loc y_out_loc
/// Protocol of PARALia/dgemv_runner.cpp:15-187: one validated call (against OpenBLAS here, at least 9 matching digits),
/// one timed first call, 100 warm-ups and 100 timed and logged iterations (20 / 20 for M, N >= 20000),
/// first / avg / min / max report in Gflops/s and in GB/s of the matrix bytes the routine must read (8 * M * N).
/// Set PARALIA_SKIP_VALIDATION=1 to skip the OpenBLAS run.
///
#include "Testing.hpp"

int main(const int argc, const char* argv[]) {
  try {
    char TransA;
    double alpha, beta;
    long int M, N, incx, incy;
    short A_loc, x_loc, y_loc, y_out_loc;
    ATC_p predef_control_values = NULL, return_values = NULL;
    ParseInputLvl2(argc, argv, &predef_control_values, &TransA, &alpha, &beta, &M, &N, &incx, &incy, &A_loc, &x_loc, &y_loc, &y_out_loc);

    char filename[1024];
    if (predef_control_values != NULL) {
      if (predef_control_values->T > 0) {
        if (predef_control_values->T > M || predef_control_values->T > N)
          error("Given Tin=%ld bigger than problem dim\n", predef_control_values->T);
        else if (predef_control_values->T > M / 1.5 && predef_control_values->T > N / 1.5)
          warning("Given Tin=%ld bigger than all problem dims/1.5\n", predef_control_values->T);
      }
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDgemvRunner_predefined_vals_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    } else {
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDgemvRunner_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    }

    const long ldA = M;
    const long x_dim = TransA == 'N' ? N : M, y_dim = TransA == 'N' ? M : N;
    const long ax = labs(incx), ay = labs(incy);
    double cpu_timer = csecond();
    fprintf(stderr, "\nAllocating memory...");
    double* A = (double*)CoCoMalloc(M * N * sizeof(double), A_loc, 0);
    double* x = (double*)CoCoMalloc(x_dim * ax * sizeof(double), x_loc, 0);
    double* y = (double*)CoCoMalloc(y_dim * ay * sizeof(double), y_loc, 1);
    CoCoSyncCheckErr();
    cpu_timer = csecond() - cpu_timer;
    fprintf(stderr, "done.\nAlloc time:\t%lf ms\n\n", cpu_timer * 1000);
    cpu_timer = csecond();
    fprintf(stderr, "Initializing to random values...");
    CoCoVecInit(A, M * N, 42, A_loc);
    CoCoVecInit(x, x_dim * ax, 43, x_loc);
    CoCoVecInit(y, y_dim * ay, 44, y_loc);
    CoCoSyncCheckErr();
    cpu_timer = csecond() - cpu_timer;
    fprintf(stderr, "done.\nInit time:\t%lf ms\n\n", cpu_timer * 1000);

    auto call = [&]() {
      if (predef_control_values != NULL)
        return PARALiADgemvControled(TransA, M, N, alpha, A, ldA, x, incx, beta, y, incy, predef_control_values);
      return PARALiADgemv(TransA, M, N, alpha, A, ldA, x, incx, beta, y, incy);
    };

    const char* skip = getenv("PARALIA_SKIP_VALIDATION");
    if (!(skip && atoi(skip))) {
      OpenBlas ob;
      double* y_start = host_copy(y, y_dim * ay, y_loc);
      return_values = call();
      CoCoSyncCheckErr();
      double* y_out = host_copy(y, y_dim * ay, y_loc);
      if (ob.open() && ob.dgemv) {
        fprintf(stderr, "Validating against OpenBLAS (%s)\n", ob.path.c_str());
        double* hA = host_copy(A, M * N, A_loc);
        double* hx = host_copy(x, x_dim * ax, x_loc);
        double* y_ref = (double*)malloc(y_dim * ay * sizeof(double));
        memcpy(y_ref, y_start, y_dim * ay * sizeof(double));
        cpu_timer = csecond();
        ob.Dgemv(TransA, M, N, alpha, hA, ldA, hx, incx, beta, y_ref, incy);
        cpu_timer = csecond() - cpu_timer;
        fprintf(stderr, "OpenBLAS cblas_dgemv: %lf ms ( %lf Gflops/s, %lf GB/s )\n", cpu_timer * 1000, Gval_per_s(gemv_flops(M, N), cpu_timer),
                8.0 * M * N / cpu_timer / 1e9);
        const short digits = Dtest_equality(y_ref, y_out, y_dim * ay);
        fprintf(stderr, "Matching digits vs OpenBLAS: %d\n", digits);
        if (digits < 9) error("Insufficient accuracy for benchmarks\n");
        free(hA); free(hx); free(y_ref);
      } else {
        // no OpenBLAS on this machine: long double dot products computed here
        double* hA = host_copy(A, ldA * N, A_loc);
        double* hx = host_copy(x, x_dim * ax, x_loc);
        double* y_ref = (double*)malloc(y_dim * ay * sizeof(double));
        memcpy(y_ref, y_start, y_dim * ay * sizeof(double));
        const double* xs = incx < 0 ? hx + (1 - x_dim) * incx : hx;
        double* ys = incy < 0 ? y_ref + (1 - y_dim) * incy : y_ref;
        const bool tr = TransA == 'T' || TransA == 't';
        for (long o = 0; o < y_dim; ++o) {
          long double acc = 0;
          for (long r = 0; r < x_dim; ++r) acc += (long double)(tr ? hA[r + o * ldA] : hA[o + r * ldA]) * xs[r * incx];
          ys[o * incy] = (double)((long double)alpha * acc + (beta == 0.0 ? 0.0L : (long double)beta * ys[o * incy]));
        }
        const short digits = Dtest_equality(y_ref, y_out, y_dim * ay);
        fprintf(stderr, "OpenBLAS absent: compared with long double dot products computed on the host\nMatching digits vs host reference: %d\n", digits);
        if (digits < 9) error("Insufficient accuracy for benchmarks\n");
        free(hA); free(hx); free(y_ref);
      }
      CoCoMemcpy(y, y_start, y_dim * ay * sizeof(double), y_loc, -2);
      free(y_start); free(y_out);
    }

    // a timed first call, 100 warm-ups and 100 timed and logged iterations (20 / 20 for the largest problems); rates in
    // Gflops/s and in GB/s of the matrix bytes the routine must read
    const int rounds = (M >= 20000 && N >= 20000) ? 20 : 100;
    const ProtocolTimes times = run_protocol(
        call, true, rounds, rounds, [](ATC_p) {},
        [&](double seconds, ATC_p info) {
          StoreLogLvl2(filename, info, TransA, alpha, beta, M, N, incx, incy, A_loc, x_loc, y_loc, y_out_loc, seconds, info->pred_t, info->pred_J);
        });
    return_values = times.info;
    char selected[128];
    snprintf(selected, sizeof selected, "T selected by %s", return_values->T_selected_by);
    report_protocol(times, (double)gemv_flops(M, N), 8.0 * M * N, selected);

    for (int i = 0; i < LOC_NUM; i++) PARALiADevCacheFree(deidxize(i));
    CoCoSyncCheckErr();
    CoCoFree(A, A_loc);
    CoCoFree(x, x_loc);
    CoCoFree(y, y_loc);
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s", e.what());
    return 1;
  }
  return 0;
}
