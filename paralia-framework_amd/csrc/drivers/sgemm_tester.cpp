/// PARALiA sgemm correctness sweep (reference PARALia/sgemm_tester.cpp:15-512); see gemm_tester.hpp.
#include "gemm_tester.hpp"

int main(const int argc, const char* argv[]) { return run_gemm_tester<float>(argc, argv); }
