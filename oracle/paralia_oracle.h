/*
 * paralia_oracle.h -- CPU restatement of the PARALiA tiled-BLAS hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the shipped library links, loads or calls this code: it exists so that tests, the smoke check and
 * the cpu_baseline leg of the benchmark have an independent statement of what the reference computes.
 * Every function cites the reference file:line it follows (paths relative to the reference tree).
 *
 * What pins each function (checked by tests/test_oracle_*.py):
 *   orc_*gemm_bruteforce      OpenBLAS cblas_dgemm/sgemm on seeded inputs; closed forms (identity, all-ones,
 *                             alpha = 0, beta = 0 with NaN C); exact small-integer data
 *   orc_*gemm_tiled           equality with the brute force on integer-valued data for every T; T-invariance
 *   orc_daxpy / orc_ddot_*    OpenBLAS cblas_daxpy/ddot; exact cases (power-of-two alpha, x = y = 1)
 *   orc_dgemv_bruteforce /    OpenBLAS cblas_dgemv; closed forms (identity, all-ones, alpha = 0, beta = 0 over NaN);
 *   orc_dgemv_tiled           exact small-integer data for every T and both transposes; gemv as a one-column gemm
 *   orc_predict_blas2         hand-evaluated closed forms on synthetic (t_exec, ti, tb, sl)
 *   orc_get_T_slowdowns /     hand-derived values: 16384^3 -> T 2048 (sl 0.00390625, 512 subkernels),
 *   orc_optimize_tile         4096^3 -> 2048 (sl 0.25), 32768^3 -> 4096, 40000x40000x2048 -> 2048
 *   orc_t_com_* / orc_predict_* hand-evaluated closed forms on synthetic (t_exec, ti, tb, sl)
 *   orc_exec_lookup_*         rows copied from the reference's own V100 logs
 *   orc_gemm_block_num        the worked example 16384^3, T = 2048 -> 257 blocks
 * PARITY UNPINNED (no reference execution is possible, their code lives in an absent submodule):
 *   the value stream of CoCoVecInit, the digit rule of Dtest_equality, SubkernelSelect's rand() tie-breaks,
 *   Buffer eviction order.  orc_rand_* and orc_digits_equal are this build's own documented definitions.
 */
#ifndef PARALIA_ORACLE_H
#define PARALIA_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- seeded data (own definition; stands where CoCoVecInit stands, dgemm_runner.cpp:64-66) ---- */
uint64_t orc_splitmix64(uint64_t* state);
void orc_rand_fill_f64(double* p, long long n, uint64_t seed); /* uniform in [-1, 1) */
void orc_rand_fill_f32(float* p, long long n, uint64_t seed);

/* ---- error metrics ---- */
double orc_normwise_err_f64(const double* c, const double* ref, long M, long N, long ldc, long ldref, double denom);
double orc_normwise_err_f32(const float* c, const float* ref, long M, long N, long ldc, long ldref, double denom);
double orc_fro_norm_f64(const double* a, long rows, long cols, long ld);
double orc_fro_norm_f32(const float* a, long rows, long cols, long ld);
long long orc_max_ulp_f64(const double* a, const double* b, long long n);
int orc_digits_equal(const double* ref, const double* x, long long n); /* min matching decimal digits, cap 16 */

/* ---- GEMM ---- */
/* C = alpha*op(A)*op(B) + beta*C with long double accumulation, one rounding per element. */
void orc_dgemm_bruteforce(char ta, char tb, long M, long N, long K, double alpha, const double* A, long lda,
                          const double* B, long ldb, double beta, double* C, long ldc);
void orc_sgemm_bruteforce(char ta, char tb, long M, long N, long K, float alpha, const float* A, long lda,
                          const float* B, long ldb, float beta, float* C, long ldc);
/* The reference's schedule: T x T x T subkernels in index order mi*Ng*Kg + ni*Kg + ki, beta schedule and
 * lazy write-back (dgemm.cpp:123-205, 273-279, 173-179).  c_resident != 0 promotes C tiles to plain WR
 * (dgemm.cpp:259-260).  Returns the number of subkernels. */
long orc_dgemm_tiled(long T, int c_resident, char ta, char tb, long M, long N, long K, double alpha, const double* A,
                     long lda, const double* B, long ldb, double beta, double* C, long ldc);
long orc_sgemm_tiled(long T, int c_resident, char ta, char tb, long M, long N, long K, float alpha, const float* A,
                     long lda, const float* B, long ldb, float beta, float* C, long ldc);

/* ---- BLAS-1 (daxpy.cpp:35-93, ddot.cpp:36-94,431) ---- */
void orc_daxpy(long n, double alpha, const double* x, long incx, double* y, long incy); /* fma(alpha, x, y) */
void orc_daxpy_mul_add(long n, double alpha, const double* x, long incx, double* y, long incy); /* two roundings */
long orc_daxpy_tiled(long T, long n, double alpha, const double* x, long incx, double* y, long incy);
/* *result += sum over 1-D tiles of the tile's partial dot (the reference adds into *result, ddot.cpp:431) */
long orc_ddot_tiled(long T, long n, const double* x, long incx, const double* y, long incy, double* result);
long double orc_ddot_longdouble(long n, const double* x, long incx, const double* y, long incy);

/* ---- BLAS-2 (dgemv.cpp:41-126) ---- */
void orc_dgemv_bruteforce(char ta, long M, long N, double alpha, const double* A, long lda, const double* x, long incx,
                          double beta, double* y, long incy); /* long double accumulation */
/* T x T tiles in index order mi*Ng + ni, beta on the first subkernel of a y tile, 1 afterwards */
long orc_dgemv_tiled(long T, char ta, long M, long N, double alpha, const double* A, long lda, const double* x, long incx,
                     double beta, double* y, long incy);

/* ---- tile-size heuristic (Autotuner.cpp:571-655; constants CMakeLists.txt:157-165) ---- */
long orc_sk_num_blas3(long D1, long D2, long D3, long T);                     /* ModelLvl3.cpp GetSKNumBLAS3 */
void orc_get_T_slowdowns(long D1, long D2, long D3, int active_unit_num, long T, double sl[6]);
long orc_optimize_tile(long D1, long D2, long D3, int active_unit_num, double best_sl[6]);
/* block pool size of one location (dgemm.cpp:23-36,80-82): 1 + |A| + |B| + |C| (+ |C| when lazy) */
long orc_gemm_block_num(long M, long N, long K, long T, int lazy);

/* ---- link model (CoModel.cpp:107-162) ---- */
typedef struct { double ti, tb, sl; } orc_link; /* t = ti + tb*bytes; sl = slowdown under opposing traffic */
double orc_t_com_predict(const orc_link* m, double bytes);
double orc_t_com_sl(const orc_link* m, double bytes);
double orc_t_com_bid_predict(const orc_link* m1, const orc_link* m2, double bytes1, double bytes2);
/* slowdown clamp applied when a Link-Stats file is read (CoModel.cpp:40-54) */
double orc_clamp_slowdown(double sl);

/* ---- exec-time lookup (GPUexec_lookup.cpp:15-129, 250-359) ---- */
typedef struct {
  int lines;
  const long* T;      /* sorted ascending per (TransA, TransB) */
  const double* t;    /* seconds */
  const char* ta;     /* per line, 'N' / 'T' (ignored for BLAS-1 when null) */
  const char* tb;
} orc_exec_table;
long orc_exec_nearest_T(const orc_exec_table* tab, long Tin);
double orc_exec_predict(const orc_exec_table* tab, long T, char ta, char tb);

/* ---- overlap models (ModelLvl3.cpp:20-551, ModelLvl1.cpp:262-326, Model_functions.cpp:195-244) ---- */
enum { ORC_BASELINE = 3, ORC_DATALOC = 4, ORC_BIDIRECTIONAL = 5, ORC_REUSE = 6, ORC_FULL_OVERLAP = 9, ORC_NO_OVERLAP = 10 };
typedef struct {
  long D1, D2, D3;       /* M, N, K (BLAS-1: N, 1, 1) */
  int dtype_sz;
  char ta, tb;
  int remote[3];         /* operand i (A, B, C / x, y) lives off the executing device */
  int out_remote[3];     /* ... and its output location does */
  orc_link h2d, d2h;     /* host -> device and device -> host link of the executing device */
  const orc_exec_table* exec;
} orc_problem;
double orc_predict_blas3(int mode, const orc_problem* p, long T);
double orc_predict_blas1_bidirectional(const orc_problem* p, int numT, const int* in, const int* out, long T);
double orc_predict_blas2(int mode, const orc_problem* p, long T); /* ModelLvl2.cpp:89-259; D1 = M, D2 = N */
/* argmin over the T values present in the lookup table, T <= min dim (Model_functions.cpp:195-244) */
long orc_optimize_tile_model(int mode, const orc_problem* p, double* pred_t);

/* ---- OpenBLAS (the parity target; loaded at run time, never linked) ---- */
int orc_openblas_open(const char* path_or_null); /* 0 ok; searches env PARALIA_OPENBLAS_LIB, system, numpy/scipy wheels */
const char* orc_openblas_path(void);
const char* orc_openblas_config(void);
int orc_openblas_threads(int set_to_or_0);
int orc_openblas_dgemm(char ta, char tb, long M, long N, long K, double alpha, const double* A, long lda,
                       const double* B, long ldb, double beta, double* C, long ldc);
int orc_openblas_sgemm(char ta, char tb, long M, long N, long K, float alpha, const float* A, long lda, const float* B,
                       long ldb, float beta, float* C, long ldc);
int orc_openblas_dgemv(char ta, long M, long N, double alpha, const double* A, long lda, const double* x, long incx,
                       double beta, double* y, long incy);
int orc_openblas_daxpy(long n, double alpha, const double* x, long incx, double* y, long incy);
int orc_openblas_ddot(long n, const double* x, long incx, const double* y, long incy, double* out);

#ifdef __cplusplus
}
#endif
#endif
