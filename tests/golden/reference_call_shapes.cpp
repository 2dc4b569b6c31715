// A small driver written against the call shapes of the reference's benchmark programs
// (Benchmarking/CuCuBLAS/src/PARALia/dgemm_runner.cpp:16-160, dgemv_runner.cpp:47, daxpy_runner.cpp, ddot_runner.cpp):
// the same helper names, argument orders and types a maintainer's own driver would use.  tests/test_abi.py compiles it
// with g++ against include/ and links libparalia.so; run with "host" it exercises only the helpers that need no GPU,
// with "gpu" it makes the routine calls as well.
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "PARALiA.hpp"
#include "Testing.hpp"
#include "backend_wrappers.hpp"

// stand-ins for the operation enums of the host and device BLAS a driver was written for
enum host_blas_op { HostNoTrans = 111, HostTrans = 112 };
enum device_blas_op { DeviceOpN = 0, DeviceOpT = 1 };

int main(const int argc, const char* argv[]) {
  const bool gpu = argc > 1 && !strcmp(argv[1], "gpu");
  char TransA = 'N', TransB = 'T';
  double alpha = 1.2, beta = 1.1;
  long int M = 300, N = 200, K = 100;
  short A_loc = -1, B_loc = -1, C_loc = -1, C_out_loc = -1;
  ATC_p predef_control_values = NULL, return_values = NULL;

  char* filename = (char*)malloc(1024 * sizeof(char));
  sprintf(filename, "%s/CoCoPeLiaDgemmRunner_%s_%s.log", TESTLIBDIR, CoCoImplementationPrint(), VERSION);
  CheckLogLvl3(filename, predef_control_values, TransA, TransB, alpha, beta, M, N, K, A_loc, B_loc, C_loc, C_out_loc);

  host_blas_op cpu_op_A, cpu_op_B;
  device_blas_op gpu_op_A, gpu_op_B;
  long int ldA, ldB, ldC = M;
  TransposeTranslate(TransA, &cpu_op_A, &gpu_op_A, &ldA, M, K);
  TransposeTranslate(TransB, &cpu_op_B, &gpu_op_B, &ldB, K, N);
  if (cpu_op_A != HostNoTrans || gpu_op_A != DeviceOpN || ldA != M) return 10;
  if (cpu_op_B != HostTrans || gpu_op_B != DeviceOpT || ldB != N) return 11;
  if (gemm_flops(M, N, K) != (long long)M * K * (2 * N + 1)) return 12;
  if (Gval_per_s(2000000000LL, 2.0) != 1.0) return 13;
  if (idxize(-1) != LOC_NUM - 1 || deidxize(LOC_NUM - 1) != -1) return 14;

  double cpu_timer = csecond();
  if (gpu) {
    double *A, *B, *C;
    A = (double*)CoCoMalloc(M * K * sizeof(double), A_loc, 0);
    B = (double*)CoCoMalloc(N * K * sizeof(double), B_loc, 0);
    C = (double*)CoCoMalloc(M * N * sizeof(double), C_loc, 1);
    CoCoSyncCheckErr();
    CoCoVecInit(A, K * M, 42, A_loc);
    CoCoVecInit(B, K * N, 43, B_loc);
    CoCoVecInit(C, M * N, 44, C_loc);
    double* C_buf = (double*)malloc(M * N * sizeof(double));
    CoCoMemcpy(C_buf, C, M * N * sizeof(double), -2, C_loc);
    if (predef_control_values != NULL)
      return_values = PARALiADgemmControled(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef_control_values);
    else
      return_values = PARALiADgemm(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC);
    CoCoSyncCheckErr();
    double* C_out = (double*)malloc(M * N * sizeof(double));
    CoCoMemcpy(C_out, C, M * N * sizeof(double), -2, C_loc);
    CoCoMemcpy(C, C_buf, M * N * sizeof(double), C_loc, -2);
    return_values = PARALiA_dgemm(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC);
    double* C_out1 = (double*)malloc(M * N * sizeof(double));
    CoCoMemcpy(C_out1, C, M * N * sizeof(double), -2, C_loc);
    if (Dtest_equality(C_out1, C_out, M * N) < 9) error("Insufficient accuracy for benchmarks\n");
    for (int i = 0; i < LOC_NUM; i++) PARALiADevCacheFree(deidxize(i));
    CoCoFree(A, A_loc);
    CoCoFree(B, B_loc);
    CoCoFree(C, C_loc);
    free(C_buf); free(C_out); free(C_out1);
  } else {
    return_values = new ATC();
    return_values->T = 128;
    return_values->active_unit_num = 1;
    return_values->active_unit_id_list[0] = 0;
    return_values->pred_t = 0.001;
    return_values->pred_J = -1;
  }
  cpu_timer = csecond() - cpu_timer;
  StoreLogLvl3(filename, return_values, TransA, TransB, alpha, beta, M, N, K, A_loc, B_loc, C_loc, C_out_loc, cpu_timer,
               return_values->pred_t, return_values->pred_J);
  fprintf(stderr, "CoCopeLia (%s):\n\tfirst_it_t = %lf ms ( %lf Gflops/s )\n", return_values->print_csv(), cpu_timer * 1000,
          Gval_per_s(gemm_flops(M, N, K), cpu_timer));
  return 0;
}
