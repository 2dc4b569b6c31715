///
/// PARALiA dgemm predictor: runs only the autotuner for a problem and logs its choice and predicted time; no GPU work.
/// argv as dgemm_runner (reference Benchmarking/CuCuBLAS/src/testing.cpp:273-329):
///   active_unit_num dev_ids_token T cache_limit TransA TransB alpha beta M N K A_loc B_loc C_loc C_out_loc
/// Follows PARALia/dgemm_predictor.cpp:12-93: build the problem description from the arguments (operand locations
/// come from the loc codes, nothing is allocated), ATC::autotune_problem("Dgemm"), print the controller, append one
/// runner-format row whose time column is the autotuning time.  In addition the prediction of every benchmarked tile
/// size is listed, so that a sweep of dgemm_runner over T can be compared with the model.
///
#include "Testing.hpp"

int main(const int argc, const char* argv[]) {
  try {
    char TransA, TransB;
    double alpha, beta;
    long int M, N, K;
    short A_loc, B_loc, C_loc, C_out_loc;
    ATC_p predef_control_values = NULL;
    ParseInputLvl3(argc, argv, &predef_control_values, &TransA, &TransB, &alpha, &beta, &M, &N, &K, &A_loc, &B_loc, &C_loc, &C_out_loc);
    char filename[1024];
    if (predef_control_values != NULL) {
      if (predef_control_values->T > 0 && (predef_control_values->T > M || predef_control_values->T > N))
        error("Given Tin=%ld bigger than problem dim\n", predef_control_values->T);
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDgemmPredictor_predefined_vals_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    } else {
      snprintf(filename, sizeof filename, "%s/CoCoPeLiaDgemmPredictor_MI355X_%s.log", test_log_dir().c_str(), DRIVER_VERSION);
    }

    auto describe = [&](long T_in) {
      ProblemDesc d;
      d.func = "Dgemm"; d.problem = BLAS3;
      d.D1 = M; d.D2 = N; d.D3 = K;
      d.TransA = TransA; d.TransB = TransB; d.dtype_sz = sizeof(double); d.numT = 3;
      const short locs[3] = {A_loc, B_loc, C_loc};
      for (int i = 0; i < 3; ++i) d.loc[i] = d.out_loc[i] = locs[i] >= 0 ? 0 : -1;
      d.beta_is_zero = beta == 0.0;
      // no device is queried here: only an explicit limit bounds the block pool
      if (predef_control_values && predef_control_values->cache_limit > 0) d.pool_budget_bytes = predef_control_values->cache_limit;
      (void)T_in;
      return d;
    };

    ATC controller;
    if (predef_control_values) {
      controller.T = predef_control_values->T;
      controller.cache_limit = predef_control_values->cache_limit;
      controller.active_unit_num = predef_control_values->active_unit_num;
      for (int i = 0; i < std::min(LOC_NUM, std::max(0, predef_control_values->active_unit_num)); ++i)
        controller.active_unit_id_list[i] = predef_control_values->active_unit_id_list[i];
    }
    const double autotune_timer = controller.autotune_problem("Dgemm", describe(controller.T));
    fprintf(stderr, "CoCoPeLiaDgemmPredictor: t_autotune = %lf ms\n", autotune_timer * 1000);
    controller.print();
    fprintf(stderr, "Predicted: T = %ld [%s], order %d, %ld subkernels, t = %lf ms ( %lf Gflops/s )\n", controller.T,
            controller.T_selected_by, controller.order_id, controller.subkernel_num, controller.pred_t * 1000,
            controller.pred_t > 0 ? Gval_per_s(gemm_flops(M, N, K), controller.pred_t) : 0.0);
    StoreLogLvl3(filename, &controller, TransA, TransB, alpha, beta, M, N, K, A_loc, B_loc, C_loc, C_out_loc, autotune_timer,
                 controller.pred_t, controller.pred_J);

    if (controller.has_db && controller.unit_modeler_list[0]) {
      fprintf(stderr, "Per-tile predictions:\n");
      long prev = -1;
      const GPUexecModel* ex = controller.unit_modeler_list[0]->exec;
      for (long i = 0; i < ex->lines(); ++i) {
        const long T = ex->T[i];
        if (T == prev || T > std::max(M, N)) continue;
        prev = T;
        ATC trial;
        trial.T = T;
        try {
          trial.autotune_problem("Dgemm", describe(T));
          fprintf(stderr, "\tT = %5ld: order %5d, %6ld subkernels, t = %10.3lf ms\n", T, trial.order_id, trial.subkernel_num, trial.pred_t * 1000);
        } catch (const paralia_error&) {
          fprintf(stderr, "\tT = %5ld: does not fit\n", T);
        }
      }
    }
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s", e.what());
    return 1;
  }
  return 0;
}
