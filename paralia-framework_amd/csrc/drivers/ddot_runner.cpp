///
/// PARALiA ddot benchmark driver.  argv as for daxpy_runner (alpha is parsed and ignored, as in the reference's
/// PARALia/ddot_runner.cpp:17-150).  The routine ADDS the dot product into *result (reference ddot.cpp:431), so the
/// scalar is cleared before every call here.
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
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDdotRunnerBest_predefined_vals_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    } else {
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDdotRunnerBest_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    }
    const long ax = labs(incx), ay = labs(incy);
    double* x = (double*)CoCoMalloc(N * ax * sizeof(double), x_loc, 0);
    double* y = (double*)CoCoMalloc(N * ay * sizeof(double), y_loc, 0);
    CoCoSyncCheckErr();
    CoCoVecInit(x, N * ax, 42, x_loc);
    CoCoVecInit(y, N * ay, 43, y_loc);
    CoCoSyncCheckErr();
    double result[1] = {0};
    auto call = [&]() {
      result[0] = 0;
      if (predef_control_values != NULL) return PARALiADdotControled(N, x, incx, y, incy, result, predef_control_values);
      return PARALiADdot(N, x, incx, y, incy, result);
    };
    const char* skip = getenv("PARALIA_SKIP_VALIDATION");
    if (!(skip && atoi(skip))) {
      OpenBlas ob;
      call();
      CoCoSyncCheckErr();
      if (ob.open()) {
        double* hx = host_copy(x, N * ax, x_loc);
        double* hy = host_copy(y, N * ay, y_loc);
        double t = csecond();
        double ref[1] = {ob.Ddot(N, hx, incx, hy, incy)};
        t = csecond() - t;
        fprintf(stderr, "OpenBLAS cblas_ddot: %lf ms ( %lf GB/s ) -> %.15e, PARALiA -> %.15e\n", t * 1000, 16.0 * N / t / 1e9, ref[0], result[0]);
        // a dot product can cancel: judge against |x||y| as well as by digits
        long double nx = 0, ny = 0;
        for (long i = 0; i < N; ++i) { nx += (long double)hx[i * ax] * hx[i * ax]; ny += (long double)hy[i * ay] * hy[i * ay]; }
        const double bound = 1e-13 * (double)sqrtl(nx * ny);
        if (Dtest_equality(ref, result, 1) < 9 && fabs(ref[0] - result[0]) > bound) error("Insufficient accuracy for benchmarks\n");
        free(hx); free(hy);
      } else {
        // no OpenBLAS on this machine: a long double sum computed here
        double* hx = host_copy(x, N * ax, x_loc);
        double* hy = host_copy(y, N * ay, y_loc);
        const double* xs = incx < 0 ? hx + (1 - N) * incx : hx;
        const double* ys = incy < 0 ? hy + (1 - N) * incy : hy;
        long double acc = 0, nx = 0, ny = 0;
        for (long i = 0; i < N; ++i) {
          acc += (long double)xs[i * incx] * ys[i * incy];
          nx += (long double)xs[i * incx] * xs[i * incx];
          ny += (long double)ys[i * incy] * ys[i * incy];
        }
        fprintf(stderr, "OpenBLAS absent: long double sum on the host -> %.15e, PARALiA -> %.15e\n", (double)acc, result[0]);
        if (fabs((double)acc - result[0]) > 1e-13 * (double)sqrtl(nx * ny)) error("Insufficient accuracy for benchmarks\n");
        free(hx); free(hy);
      }
    }
    // 10 warm-ups, 10 timed and logged iterations; GB/s of the algorithmic traffic (x and y read once)
    const ProtocolTimes times = run_protocol(
        call, false, 10, 10, [](ATC_p) {},
        [&](double seconds, ATC_p info) { StoreLogLvl1(filename, info, alpha, N, incx, incy, x_loc, y_loc, x_out_loc, y_out_loc, seconds, info->pred_t, info->pred_J); });
    report_protocol(times, (double)dot_flops(N), 16.0 * N, NULL);
    for (int i = 0; i < LOC_NUM; i++) PARALiADevCacheFree(deidxize(i));
    CoCoFree(x, x_loc);
    CoCoFree(y, y_loc);
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s", e.what());
    return 1;
  }
  return 0;
}
