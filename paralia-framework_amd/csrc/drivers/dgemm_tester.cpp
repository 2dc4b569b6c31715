/// PARALiA dgemm correctness sweep (reference PARALia/dgemm_tester.cpp:15-510); see gemm_tester.hpp.
#include "gemm_tester.hpp"

int main(const int argc, const char* argv[]) { return run_gemm_tester<double>(argc, argv); }
