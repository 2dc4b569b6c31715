///
/// Correctness sweep shared by dgemm_tester and sgemm_tester: the grid of the reference's PARALia/dgemm_tester.cpp:15-510
/// and sgemm_tester.cpp:15-512 on one GPU -- squares 256 ... 8192 (x2), non-square {256, 1024, 4096}^3, "weird"
/// dimensions 289 / 353 / 307 (x4), both operands transposed, every combination of host / device residency of A, B
/// and C, all as sub-matrix views of 8192 x 8192 buffers (ld = 8192), alpha = 1.23, beta = 0.9876 (:74-75).  Each result
/// is compared with OpenBLAS and must agree to at least min_digits digits; unlike the reference's testers, a mismatch
/// makes the program fail.  Optional argument "quick" stops the square sweep at 2048 and skips the largest cases.
///
#ifndef PARALIA_GEMM_TESTER_HPP
#define PARALIA_GEMM_TESTER_HPP
#include "Testing.hpp"

template <typename T> struct TesterFns;
template <> struct TesterFns<double> {
  static constexpr const char* name = "dgemm_tester";
  static constexpr short min_digits = 9, cap = 16;
  static ATC_p gemm(char ta, char tb, long M, long N, long K, double al, double* A, long lda, double* B, long ldb, double be, double* C, long ldc) {
    return PARALiADgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static void blas(const OpenBlas& ob, char ta, char tb, long M, long N, long K, double al, double* A, long lda, double* B, long ldb, double be, double* C, long ldc) {
    ob.Dgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static short digits(double* ref, double* x, long long n) { return Dtest_equality(ref, x, n); }
};
template <> struct TesterFns<float> {
  static constexpr const char* name = "sgemm_tester";
  static constexpr short min_digits = 4, cap = 7;
  static ATC_p gemm(char ta, char tb, long M, long N, long K, float al, float* A, long lda, float* B, long ldb, float be, float* C, long ldc) {
    return PARALiASgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static void blas(const OpenBlas& ob, char ta, char tb, long M, long N, long K, float al, float* A, long lda, float* B, long ldb, float be, float* C, long ldc) {
    ob.Sgemm(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc);
  }
  static short digits(float* ref, float* x, long long n) { return Stest_equality(ref, x, n); }
};

template <typename T> int run_gemm_tester(const int argc, const char* argv[]) {
  using F = TesterFns<T>;
  const long ES = (long)sizeof(T);

  const bool quick = argc > 1 && !strcmp(argv[1], "quick");
  int failures = 0, cases = 0;
  try {
    OpenBlas ob;
    const bool have_blas = ob.open();
    if (have_blas) fprintf(stderr, "%s: OpenBLAS = %s\n", F::name, ob.path.c_str());
    else fprintf(stderr, "%s: OpenBLAS not found: every case is checked on 512 sampled entries against a long double dot product\n", F::name);
    const long ld = 8192;
    const T alpha = (T)1.23, beta = (T)0.9876;
    T* hA = (T*)CoCoMalloc(ld * ld * ES, -1, 1);
    T* hB = (T*)CoCoMalloc(ld * ld * ES, -1, 1);
    T* hC = (T*)CoCoMalloc(ld * ld * ES, -1, 1);
    T* C_ref = (T*)CoCoMalloc(ld * ld * ES, -2, 1);
    T* C_got = (T*)CoCoMalloc(ld * ld * ES, -2, 1);
    T* dA = (T*)CoCoMalloc(ld * ld * ES, 0, 1);
    T* dB = (T*)CoCoMalloc(ld * ld * ES, 0, 1);
    T* dC = (T*)CoCoMalloc(ld * ld * ES, 0, 1);
    CoCoVecInit(hA, ld * ld, 42, -1);
    CoCoVecInit(hB, ld * ld, 43, -1);
    CoCoMemcpy(dA, hA, ld * ld * ES, 0, -1);
    CoCoMemcpy(dB, hB, ld * ld * ES, 0, -1);

    auto run_case = [&](const char* label, char ta, char tb, long M, long N, long K, short la, short lb, short lc) {
      CoCoVecInit(hC, ld * ld, 44, -1);
      const long cols = N;
      memcpy(C_ref, hC, ld * cols * ES);
      if (lc >= 0) CoCoMemcpy(dC, hC, ld * cols * ES, 0, -1);
      double t = csecond();
      ATC_p r = F::gemm(ta, tb, M, N, K, alpha, la >= 0 ? dA : hA, ld, lb >= 0 ? dB : hB, ld, beta, lc >= 0 ? dC : hC, ld);
      CoCoSyncCheckErr();
      t = csecond() - t;
      CoCoMemcpy(C_got, lc >= 0 ? dC : hC, ld * cols * ES, -2, lc >= 0 ? 0 : -1);
      double t_ref = csecond();
      short worst = F::cap;
      bool pad_ok = true;  // rows M..ld of every column belong to the caller
      for (long j = 0; j < N && pad_ok; ++j)
        for (long i = M; i < ld && i < M + 4; ++i) pad_ok &= (C_got[i + j * ld] == C_ref[i + j * ld]);
      if (have_blas) {
        F::blas(ob, ta, tb, M, N, K, alpha, hA, ld, hB, ld, beta, C_ref, ld);
        for (long j = 0; j < N; ++j) worst = std::min(worst, F::digits(C_ref + j * ld, C_got + j * ld, M));
      } else {
        worst = sampled_gemm_digits<T>(ta, tb, M, N, K, alpha, hA, ld, hB, ld, beta, C_ref, C_got, ld);
      }
      t_ref = csecond() - t_ref;
      ++cases;
      const bool ok = worst >= F::min_digits && pad_ok;
      if (!ok) ++failures;
      fprintf(stderr, "%-22s %c%c M=%-5ld N=%-5ld K=%-5ld locs(%d,%d,%d): PARALiA %.1lf Gflops/s, reference %.1lf, T=%ld, digits=%d %s\n", label, ta, tb,
              M, N, K, la, lb, lc, Gval_per_s(gemm_flops(M, N, K), t), Gval_per_s(gemm_flops(M, N, K), t_ref), r->T, worst, ok ? "ok" : "FAIL");
      delete r;
    };

    const long maxsq = quick ? 2048 : 8192;
    for (long dim = 256; dim <= maxsq; dim *= 2) run_case("square host", 'N', 'N', dim, dim, dim, -1, -1, -1);
    const long big = quick ? 1024 : 4096;
    for (long d1 = 256; d1 <= big; d1 *= 4)
      for (long d2 = 256; d2 <= big; d2 *= 4)
        for (long d3 = 256; d3 <= big; d3 *= 4)
          if (d1 != d2 || d2 != d3) run_case("non-square host", 'N', 'N', d1, d2, d3, -1, -1, -1);
    for (long d1 = 289; d1 <= big * 2; d1 *= 4)
      for (long d2 = 353; d2 <= big * 2; d2 *= 4)
        for (long d3 = 307; d3 <= big * 2; d3 *= 4) run_case("weird dims host", 'N', 'N', d1, d2, d3, -1, -1, -1);
    for (long dim = 256; dim <= maxsq; dim *= 4) run_case("transposed host", 'T', 'T', dim, dim + 33, dim - 7, -1, -1, -1);
    for (short la : {short(-1), short(0)})
      for (short lb : {short(-1), short(0)})
        for (short lc : {short(-1), short(0)}) run_case("mixed residency", 'N', 'T', 1500, 1300, 1100, la, lb, lc);
    run_case("device resident", 'N', 'N', 2048, 2048, 2048, 0, 0, 0);

    for (int i = 0; i < LOC_NUM; i++) PARALiADevCacheFree(deidxize(i));
    CoCoFree(hA, -1); CoCoFree(hB, -1); CoCoFree(hC, -1); CoCoFree(C_ref, -2); CoCoFree(C_got, -2);
    CoCoFree(dA, 0); CoCoFree(dB, 0); CoCoFree(dC, 0);
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s", e.what());
    return 1;
  }
  fprintf(stderr, "%s: %d cases, %d failures\n", F::name, cases, failures);
  return failures ? 1 : 0;
}

#endif
