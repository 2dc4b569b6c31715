/// dgemm_runner: the fp64 instance of the shared GEMM benchmark driver (see gemm_runner.hpp).
#include "gemm_runner.hpp"

int main(const int argc, const char* argv[]) { return run_gemm_runner<double>(argc, argv); }
