///
/// PARALiA daxpy benchmark driver.  argv (reference testing.cpp:159-215):
///   active_unit_num dev_ids_token T cache_limit alpha N incx incy x_loc y_loc x_out_loc y_out_loc
/// Protocol of PARALia/daxpy_runner.cpp:16-150: validation against the CPU library (at least 9 matching digits),
/// 10 warm-ups, timed iterations, report in GB/s of algorithmic traffic (3 * 8 * N bytes) and Gflops/s.
///
#include "Testing.hpp"

int main(const int argc, const char* argv[]) {
  try {
    double alpha;
    long int N, incx, incy;
    short x_loc, y_loc, x_out_loc, y_out_loc;
    ATC_p predef_control_values = NULL;
    ParseInputLvl1(argc, argv, &predef_control_values, &alpha, &N, &incx, &incy, &x_loc, &y_loc, &x_out_loc, &y_out_loc);
    char filename[1024];
    if (predef_control_values != NULL) {
      if (predef_control_values->T > N) error("Given Tin=%ld bigger than problem dim\n", predef_control_values->T);
      else if (predef_control_values->T > N / 1.5) warning("Given Tin=%ld bigger than all problem dims/1.5\n", predef_control_values->T);
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDaxpyRunnerBest_predefined_vals_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    } else {
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDaxpyRunnerBest_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    }
    const long ax = labs(incx), ay = labs(incy);
    double* x = (double*)CoCoMalloc(N * ax * sizeof(double), x_loc, 0);
    double* y = (double*)CoCoMalloc(N * ay * sizeof(double), y_loc, 1);
    CoCoSyncCheckErr();
    CoCoVecInit(x, N * ax, 42, x_loc);
    CoCoVecInit(y, N * ay, 43, y_loc);
    CoCoSyncCheckErr();
    auto call = [&]() {
      if (predef_control_values != NULL) return PARALiADaxpyControled(N, alpha, x, incx, y, incy, predef_control_values);
      return PARALiADaxpy(N, alpha, x, incx, y, incy);
    };
    const char* skip = getenv("PARALIA_SKIP_VALIDATION");
    if (!(skip && atoi(skip))) {
      OpenBlas ob;
      double* y_start = host_copy(y, N * ay, y_loc);
      call();
      CoCoSyncCheckErr();
      double* y_out = host_copy(y, N * ay, y_loc);
      if (ob.open()) {
        double* hx = host_copy(x, N * ax, x_loc);
        double* y_ref = (double*)malloc(N * ay * sizeof(double));
        memcpy(y_ref, y_start, N * ay * sizeof(double));
        double t = csecond();
        ob.Daxpy(N, alpha, hx, incx, y_ref, incy);
        t = csecond() - t;
        fprintf(stderr, "OpenBLAS cblas_daxpy: %lf ms ( %lf GB/s )\n", t * 1000, 24.0 * N / t / 1e9);
        const short digits = Dtest_equality(y_ref, y_out, N * ay);
        fprintf(stderr, "Matching digits vs OpenBLAS: %d\n", digits);
        if (digits < 9) error("Insufficient accuracy for benchmarks\n");
        free(hx); free(y_ref);
      } else {
        // no OpenBLAS on this machine: the fused multiply-add of every element, computed here
        double* hx = host_copy(x, N * ax, x_loc);
        double* y_ref = (double*)malloc(N * ay * sizeof(double));
        memcpy(y_ref, y_start, N * ay * sizeof(double));
        const double* xs = incx < 0 ? hx + (1 - N) * incx : hx;
        double* ys = incy < 0 ? y_ref + (1 - N) * incy : y_ref;
        for (long i = 0; i < N; ++i) ys[i * incy] = fma(alpha, xs[i * incx], ys[i * incy]);
        const short digits = Dtest_equality(y_ref, y_out, N * ay);
        fprintf(stderr, "OpenBLAS absent: compared with fma(alpha, x, y) computed on the host\nMatching digits vs host reference: %d\n", digits);
        if (digits < 9) error("Insufficient accuracy for benchmarks\n");
        free(hx); free(y_ref);
      }
      CoCoMemcpy(y, y_start, N * ay * sizeof(double), y_loc, -2);
      free(y_start); free(y_out);
    }
    // 10 warm-ups, 10 timed and logged iterations; GB/s of the algorithmic traffic (x and y read, y written)
    const ProtocolTimes times = run_protocol(
        call, false, 10, 10, [](ATC_p) {},
        [&](double seconds, ATC_p info) { StoreLogLvl1(filename, info, alpha, N, incx, incy, x_loc, y_loc, x_out_loc, y_out_loc, seconds, info->pred_t, info->pred_J); });
    report_protocol(times, (double)axpy_flops(N), 24.0 * N, NULL);
    for (int i = 0; i < LOC_NUM; i++) PARALiADevCacheFree(deidxize(i));
    CoCoFree(x, x_loc);
    CoCoFree(y, y_loc);
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s", e.what());
    return 1;
  }
  return 0;
}
