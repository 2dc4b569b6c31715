/*
 * paralia_oracle.c -- CPU restatement of the PARALiA tiled-BLAS hot path.  TEST INFRASTRUCTURE ONLY
 * (see paralia_oracle.h for what pins each function and what stays unpinned).
 * Plain C, no dependency on the shipped library.
 */
#define _GNU_SOURCE
#include "paralia_oracle.h"

#include <dlfcn.h>
#include <float.h>
#include <glob.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------ data */

/* splitmix64 (Steele, Lea, Flood 2014; public-domain reference by S. Vigna). */
uint64_t orc_splitmix64(uint64_t* state) {
  uint64_t z = (*state += 0x9E3779B97F4A7C15ULL);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

/* Element i of stream `seed` is a pure function of (seed, i): the state before the draw is
 * seed * 0xD1342543DE82EF95 + i * 0x9E3779B97F4A7C15, so any slice can be generated independently. */
static inline uint64_t draw(uint64_t seed, uint64_t i) {
  uint64_t s = seed * 0xD1342543DE82EF95ULL + i * 0x9E3779B97F4A7C15ULL;
  return orc_splitmix64(&s);
}
void orc_rand_fill_f64(double* p, long long n, uint64_t seed) {
  for (long long i = 0; i < n; ++i) p[i] = (double)(draw(seed, (uint64_t)i) >> 11) * (2.0 / 9007199254740992.0) - 1.0;
}
void orc_rand_fill_f32(float* p, long long n, uint64_t seed) {
  for (long long i = 0; i < n; ++i) p[i] = (float)(draw(seed, (uint64_t)i) >> 40) * (2.0f / 16777216.0f) - 1.0f;
}

/* --------------------------------------------------------------------------------------------- metrics */

double orc_fro_norm_f64(const double* a, long rows, long cols, long ld) {
  long double s = 0;
  for (long j = 0; j < cols; ++j)
    for (long i = 0; i < rows; ++i) s += (long double)a[i + j * ld] * a[i + j * ld];
  return (double)sqrtl(s);
}
double orc_fro_norm_f32(const float* a, long rows, long cols, long ld) {
  long double s = 0;
  for (long j = 0; j < cols; ++j)
    for (long i = 0; i < rows; ++i) s += (long double)a[i + j * ld] * a[i + j * ld];
  return (double)sqrtl(s);
}
/* ||C - ref||_F / denom ; the caller passes denom = |alpha| ||A||_F ||B||_F + |beta| ||C0||_F */
double orc_normwise_err_f64(const double* c, const double* ref, long M, long N, long ldc, long ldref, double denom) {
  long double s = 0;
  for (long j = 0; j < N; ++j)
    for (long i = 0; i < M; ++i) {
      long double d = (long double)c[i + j * ldc] - ref[i + j * ldref];
      if (isnan((double)d)) return NAN;
      s += d * d;
    }
  return (double)(sqrtl(s) / (denom > 0 ? denom : 1.0));
}
double orc_normwise_err_f32(const float* c, const float* ref, long M, long N, long ldc, long ldref, double denom) {
  long double s = 0;
  for (long j = 0; j < N; ++j)
    for (long i = 0; i < M; ++i) {
      long double d = (long double)c[i + j * ldc] - ref[i + j * ldref];
      if (isnan((double)d)) return NAN;
      s += d * d;
    }
  return (double)(sqrtl(s) / (denom > 0 ? denom : 1.0));
}

static int64_t ordered(double x) {
  int64_t i;
  memcpy(&i, &x, 8);
  return i < 0 ? INT64_MIN - i : i;
}
long long orc_max_ulp_f64(const double* a, const double* b, long long n) {
  long long worst = 0;
  for (long long i = 0; i < n; ++i) {
    if (isnan(a[i]) || isnan(b[i])) return (isnan(a[i]) && isnan(b[i])) ? worst : INT64_MAX;
    int64_t d = ordered(a[i]) - ordered(b[i]);
    if (d < 0) d = -d;
    if (d > worst) worst = d;
  }
  return worst;
}

/* Own definition of "matching digits" (the reference's Dtest_equality is not in its tree): the smallest over
 * all elements of floor(-log10(|ref_i - x_i| / max(|ref_i|, |x_i|, rms(ref)))), capped at 16; the drivers demand
 * >= 9 (dgemm_runner.cpp:99).  The rms term keeps elements that are small by cancellation on the vector's scale. */
int orc_digits_equal(const double* ref, const double* x, long long n) {
  long double ss = 0;
  for (long long i = 0; i < n; ++i) ss += (long double)ref[i] * ref[i];
  const double rms = n > 0 ? (double)sqrtl(ss / n) : 0.0;
  int worst = 16;
  for (long long i = 0; i < n; ++i) {
    double d = fabs(ref[i] - x[i]);
    if (d == 0) continue;
    if (isnan(d)) return 0;
    double scale = fmax(fmax(fabs(ref[i]), fabs(x[i])), rms);
    int digits = (int)floor(-log10(d / scale));
    if (digits < 0) digits = 0;
    if (digits < worst) worst = digits;
  }
  return worst;
}

/* ------------------------------------------------------------------------------------------------ GEMM */

static inline int is_t(char c) { return c == 'T' || c == 't'; }

#define DEF_BRUTE(NAME, T)                                                                                        \
  void NAME(char ta, char tb, long M, long N, long K, T alpha, const T* A, long lda, const T* B, long ldb, T beta, \
            T* C, long ldc) {                                                                                    \
    const int at = is_t(ta), bt = is_t(tb);                                                                      \
    for (long j = 0; j < N; ++j)                                                                                 \
      for (long i = 0; i < M; ++i) {                                                                             \
        long double s = 0;                                                                                       \
        if (alpha != 0)                                                                                          \
          for (long k = 0; k < K; ++k) {                                                                         \
            long double a = at ? A[k + i * lda] : A[i + k * lda];                                                \
            long double b = bt ? B[j + k * ldb] : B[k + j * ldb];                                                \
            s += a * b;                                                                                          \
          }                                                                                                      \
        long double r = (long double)alpha * s;                                                                  \
        if (beta != 0) r += (long double)beta * C[i + j * ldc]; /* beta == 0: C is not read (BLAS) */            \
        C[i + j * ldc] = (T)r;                                                                                   \
      }                                                                                                          \
  }
DEF_BRUTE(orc_dgemm_bruteforce, double)
DEF_BRUTE(orc_sgemm_bruteforce, float)

/* One subkernel: Ct = alpha * op(At) * op(Bt) + beta * Ct in the working precision, k ascending
 * (what cublasDgemm does for the reference at Subkernel.cpp:168). */
#define DEF_TILE(NAME, T)                                                                                         \
  static void NAME(int at, int bt, long m, long n, long k, T alpha, const T* A, long lda, const T* B, long ldb,   \
                   T beta, T* C, long ldc) {                                                                      \
    for (long j = 0; j < n; ++j)                                                                                 \
      for (long i = 0; i < m; ++i) {                                                                             \
        T s = 0;                                                                                                 \
        for (long kk = 0; kk < k; ++kk) {                                                                        \
          T a = at ? A[kk + i * lda] : A[i + kk * lda];                                                          \
          T b = bt ? B[j + kk * ldb] : B[kk + j * ldb];                                                          \
          s += a * b;                                                                                            \
        }                                                                                                        \
        C[i + j * ldc] = (beta == 0) ? alpha * s : alpha * s + beta * C[i + j * ldc];                            \
      }                                                                                                          \
  }
DEF_TILE(tile_gemm_f64, double)
DEF_TILE(tile_gemm_f32, float)

/* dgemm.cpp:123-205: grids Mg x Ng x Kg of T-sized tiles (edge tiles smaller); the *stored* matrix is tiled,
 * so for op = 'T' subkernel (mi, ki) reads stored tile (ki, mi) (dgemm.cpp:184-191).
 * dgemm.cpp:273-279: the first K-step of a C tile runs with beta' = 0 into a device-local accumulator when
 * the tile is lazily written (ALGO_WR_LAZY), or with the caller's beta directly on C when C is resident;
 * every later K-step runs with beta' = 1.
 * dgemm.cpp:173-179: after the last K-step a lazy tile is combined as C <- reduce_mult * C_src + C_local with
 * reduce_mult = beta.  With beta == 0 the source tile is neither fetched nor read (BLAS convention; the
 * reference's own handling is inside its absent backend). */
#define DEF_TILED(NAME, T, TILE)                                                                                  \
  long NAME(long Tt, int c_resident, char ta, char tb, long M, long N, long K, T alpha, const T* A, long lda,      \
            const T* B, long ldb, T beta, T* C, long ldc) {                                                       \
    if (Tt <= 0 || M <= 0 || N <= 0) return 0;                                                                    \
    const int at = is_t(ta), bt = is_t(tb);                                                                      \
    const long Mg = (M + Tt - 1) / Tt, Ng = (N + Tt - 1) / Tt, Kg = K > 0 ? (K + Tt - 1) / Tt : 1;                 \
    T* acc = (T*)malloc(sizeof(T) * (size_t)Tt * (size_t)Tt);                                                     \
    long fired = 0;                                                                                              \
    for (long mi = 0; mi < Mg; ++mi)                                                                             \
      for (long ni = 0; ni < Ng; ++ni) {                                                                         \
        const long m = (mi == Mg - 1) ? M - mi * Tt : Tt, n = (ni == Ng - 1) ? N - ni * Tt : Tt;                  \
        T* Ct = C + mi * Tt + ni * Tt * ldc;                                                                     \
        for (long ki = 0; ki < Kg; ++ki) {                                                                       \
          const long k = (K <= 0) ? 0 : ((ki == Kg - 1) ? K - ki * Tt : Tt);                                      \
          const T* At = at ? A + ki * Tt + mi * Tt * lda : A + mi * Tt + ki * Tt * lda;                          \
          const T* Bt = bt ? B + ni * Tt + ki * Tt * ldb : B + ki * Tt + ni * Tt * ldb;                          \
          if (c_resident)                                                                                        \
            TILE(at, bt, m, n, k, alpha, At, lda, Bt, ldb, ki == 0 ? beta : (T)1, Ct, ldc);                       \
          else                                                                                                   \
            TILE(at, bt, m, n, k, alpha, At, lda, Bt, ldb, ki == 0 ? (T)0 : (T)1, acc, Tt);                       \
          ++fired;                                                                                               \
        }                                                                                                        \
        if (!c_resident)                                                                                         \
          for (long j = 0; j < n; ++j)                                                                           \
            for (long i = 0; i < m; ++i)                                                                         \
              Ct[i + j * ldc] = (beta == 0) ? acc[i + j * Tt] : beta * Ct[i + j * ldc] + acc[i + j * Tt];         \
      }                                                                                                          \
    free(acc);                                                                                                   \
    return fired;                                                                                                \
  }
DEF_TILED(orc_dgemm_tiled, double, tile_gemm_f64)
DEF_TILED(orc_sgemm_tiled, float, tile_gemm_f32)

/* ---------------------------------------------------------------------------------------------- BLAS-1 */

static inline const double* first_c(const double* p, long n, long inc) { return inc < 0 ? p + (1 - n) * inc : p; }
static inline double* first_m(double* p, long n, long inc) { return inc < 0 ? p + (1 - n) * inc : p; }

void orc_daxpy(long n, double alpha, const double* x, long incx, double* y, long incy) {
  if (n <= 0 || alpha == 0.0) return;
  const double* xs = first_c(x, n, incx);
  double* ys = first_m(y, n, incy);
  for (long i = 0; i < n; ++i) ys[i * incy] = fma(alpha, xs[i * incx], ys[i * incy]);
}
void orc_daxpy_mul_add(long n, double alpha, const double* x, long incx, double* y, long incy) {
  if (n <= 0 || alpha == 0.0) return;
  const double* xs = first_c(x, n, incx);
  double* ys = first_m(y, n, incy);
  for (long i = 0; i < n; ++i) {
    volatile double p = alpha * xs[i * incx]; /* keep the product rounded on its own */
    ys[i * incy] = p + ys[i * incy];
  }
}
/* daxpy.cpp:35-78: one subkernel per 1-D tile of T elements, x read-only, y read + written back. */
long orc_daxpy_tiled(long T, long n, double alpha, const double* x, long incx, double* y, long incy) {
  if (n <= 0 || T <= 0) return 0;
  long tiles = 0;
  for (long s = 0; s < n; s += T, ++tiles) {
    const long len = (n - s < T) ? n - s : T;
    orc_daxpy(len, alpha, x + s * incx, incx, y + s * incy, incy);
  }
  return tiles;
}
/* ddot.cpp:36-77: one partial per tile; ddot.cpp:431: *result += every partial, in tile order. */
long orc_ddot_tiled(long T, long n, const double* x, long incx, const double* y, long incy, double* result) {
  if (n <= 0 || T <= 0) return 0;
  long tiles = 0;
  for (long s = 0; s < n; s += T, ++tiles) {
    const long len = (n - s < T) ? n - s : T;
    double partial = 0.0;
    for (long i = 0; i < len; ++i) partial += x[(s + i) * incx] * y[(s + i) * incy];
    *result += partial;
  }
  return tiles;
}
long double orc_ddot_longdouble(long n, const double* x, long incx, const double* y, long incy) {
  if (n <= 0) return 0;
  const double* xs = first_c(x, n, incx);
  const double* ys = first_c(y, n, incy);
  long double s = 0, c = 0; /* Kahan on top of long double */
  for (long i = 0; i < n; ++i) {
    long double t = (long double)xs[i * incx] * ys[i * incy] - c;
    long double u = s + t;
    c = (u - s) - t;
    s = u;
  }
  return s;
}

/* ------------------------------------------------------------------------------------- tile heuristic */

#define ORC_TILE_MIN 2048              /* CMakeLists.txt:157 */
#define ORC_TILE_MIN_SLOWDOWN 0.2      /* :158 */
#define ORC_MAX_DESIRED_SK_DEV 512     /* :161 */
#define ORC_MAX_DESIRED_SK_DEV_SLOWDOWN 0.1 /* :162 */
#define ORC_TILE_MAX 4096              /* :164 */
#define ORC_TILE_MAX_SLOWDOWN 0.1      /* :165 */

/* ------------------------------------------------------------------------------------------------ BLAS-2 */
/* y = alpha*op(A)*x + beta*y, long double accumulation, one rounding per element; BLAS conventions: quick return for
 * M == 0 or N == 0, beta == 0 never reads y, negative increments walk the vector backwards. */
void orc_dgemv_bruteforce(char ta, long M, long N, double alpha, const double* A, long lda, const double* x, long incx,
                          double beta, double* y, long incy) {
  if (M <= 0 || N <= 0) return;
  const int t = is_t(ta);
  const long lx = t ? M : N, ly = t ? N : M;
  const double* xs = first_c(x, lx, incx);
  double* ys = first_m(y, ly, incy);
  for (long i = 0; i < ly; ++i) {
    long double acc = 0.0L;
    if (alpha != 0.0) /* BLAS: A and x are not referenced when alpha == 0 */
      for (long j = 0; j < lx; ++j) acc += (long double)(t ? A[j + i * lda] : A[i + j * lda]) * (long double)xs[j * incx];
    const long double prev = beta == 0.0 ? 0.0L : (long double)beta * (long double)ys[i * incy];
    ys[i * incy] = (double)((long double)alpha * acc + prev);
  }
}

/* The reference's schedule (dgemv.cpp:41-118, 121-126): A cut into T x T tiles, subkernel mi*Ng + ni multiplies the x
 * tile of its reduction index into the y tile of its output index, the first subkernel of a y tile applies the
 * caller's beta and later ones accumulate with beta = 1.  Each tile product is an ordinary double-precision gemv
 * (fma accumulation in index order), as one cublasDgemv call per tile would be.  Returns the number of subkernels. */
long orc_dgemv_tiled(long T, char ta, long M, long N, double alpha, const double* A, long lda, const double* x, long incx,
                     double beta, double* y, long incy) {
  if (M <= 0 || N <= 0 || T <= 0) return 0;
  const int t = is_t(ta);
  const long lx = t ? M : N, ly = t ? N : M;
  const double* xs = first_c(x, lx, incx);
  double* ys = first_m(y, ly, incy);
  const long Mg = (M + T - 1) / T, Ng = (N + T - 1) / T;
  for (long mi = 0; mi < Mg; ++mi)
    for (long ni = 0; ni < Ng; ++ni) {
      const long tm = mi == Mg - 1 ? M - mi * T : T, tn = ni == Ng - 1 ? N - ni * T : T;
      const double* At = A + mi * T + ni * T * lda;
      const long xi = t ? mi : ni, yi = t ? ni : mi, xl = t ? tm : tn, yl = t ? tn : tm;
      const int first = (t ? mi : ni) == 0;
      const double b = first ? beta : 1.0;
      for (long i = 0; i < yl; ++i) {
        double acc = 0.0;
        for (long j = 0; j < xl; ++j) acc = fma(t ? At[j + i * lda] : At[i + j * lda], xs[(xi * T + j) * incx], acc);
        double* yp = ys + (yi * T + i) * incy;
        *yp = b == 0.0 ? alpha * acc : fma(alpha, acc, b * *yp);
      }
    }
  return Mg * Ng;
}

static long cdiv(long a, long b) { return a / b + ((a % b) ? 1 : 0); }

long orc_sk_num_blas3(long D1, long D2, long D3, long T) { return cdiv(D1, T) * cdiv(D2, T) * cdiv(D3, T); }

/* Autotuner.cpp:571-603 (integer and floating conversions kept as written there). */
void orc_get_T_slowdowns(long D1in, long D2in, long D3in, int units, long T, double sl[6]) {
  const int D1 = (int)D1in, D2 = (D2in == -1) ? D1 : (int)D2in, D3 = (D3in == -1) ? D1 : (int)D3in;
  const int cT = (int)T;
  for (int i = 0; i < 6; ++i) sl[i] = 0.0;
  int bucket_num = (int)(orc_sk_num_blas3(D1, D2, D3, cT) / (D3 / cT + ((D3 % cT) ? 1 : 0)));
  sl[1] = (bucket_num / units) ? 1.0 * (bucket_num % units) / (bucket_num / units) * units : 1.0 * bucket_num / units;
  if (D1 % cT) sl[2] += 1.0 / (D1 / cT);
  if (D2 % cT) sl[2] += 1.0 / (D2 / cT);
  if (D3 % cT) sl[2] += 1.0 / (D3 / cT);
  if (cT < ORC_TILE_MIN) sl[3] += 1.0 * ORC_TILE_MIN / cT * ORC_TILE_MIN_SLOWDOWN;
  long dev_sks = (long)((1.0 * orc_sk_num_blas3(D1, D2, D3, cT)) / units);
  sl[4] += 2.0 / dev_sks;
  if (dev_sks > ORC_MAX_DESIRED_SK_DEV) sl[4] += (1.0 * dev_sks / ORC_MAX_DESIRED_SK_DEV) * ORC_MAX_DESIRED_SK_DEV_SLOWDOWN;
  if (cT > ORC_TILE_MAX) sl[5] += cT / ORC_TILE_MAX * ORC_TILE_MAX_SLOWDOWN;
  sl[0] = sl[1] + sl[2] + sl[3] + sl[4] + sl[5];
}

/* Autotuner.cpp:605-655: scan T = min(D) ... 1, keep the first strict minimum of the aggregate. */
long orc_optimize_tile(long D1, long D2in, long D3in, int units, double best_sl[6]) {
  const long D2 = (D2in == -1) ? D1 : D2in, D3 = (D3in == -1) ? D1 : D3in;
  long maxT = D1 < D2 ? D1 : D2;
  if (D3 < maxT) maxT = D3;
  long best = -1;
  double cur[6];
  for (int i = 0; i < 6; ++i) best_sl[i] = DBL_MAX;
  for (long T = maxT; T > 0; --T) {
    orc_get_T_slowdowns(D1, D2, D3, units, T, cur);
    if (cur[0] < best_sl[0]) {
      memcpy(best_sl, cur, sizeof(cur));
      best = T;
    }
  }
  return best;
}

long orc_gemm_block_num(long M, long N, long K, long T, int lazy) {
  const long a = cdiv(M, T) * cdiv(K, T), b = cdiv(K, T) * cdiv(N, T), c = cdiv(M, T) * cdiv(N, T);
  return 1 + a + b + c + (lazy ? c : 0);
}

/* ------------------------------------------------------------------------------------------ link model */

double orc_t_com_predict(const orc_link* m, double bytes) { /* CoModel.cpp:108-117 */
  if (bytes < 0) return -1;
  if (bytes == 0) return 0;
  return m->ti + m->tb * bytes;
}
double orc_t_com_sl(const orc_link* m, double bytes) { /* CoModel.cpp:143-148 */
  if (bytes < 0) return -1;
  if (bytes == 0) return 0;
  return m->ti + m->tb * bytes * m->sl;
}
double orc_t_com_bid_predict(const orc_link* m1, const orc_link* m2, double b1, double b2) { /* CoModel.cpp:151-162 */
  if (b1 < 0 || b2 < 0) return -1;
  if (b1 == 0) return orc_t_com_predict(m2, b2);
  if (b2 == 0) return orc_t_com_predict(m1, b1);
  const double t1 = orc_t_com_sl(m1, b1), t2 = orc_t_com_sl(m2, b2);
  if (t1 < t2) return t1 * (1.0 - 1 / m2->sl) + b2 * m2->tb + m2->ti / m2->sl;
  return t2 * (1.0 - 1 / m1->sl) + b1 * m1->tb + m1->ti / m1->sl;
}
double orc_clamp_slowdown(double sl) { /* CoModel.cpp:40-54, NORMALIZE_NEAR_SPLIT_LIMIT = 0.05 */
  if (sl < 1 - 0.05) sl = 1;      /* "faster when shared" is measurement noise */
  else if (sl > 2) sl = 2.0;      /* worse than an even split of the link is capped at 50% sharing */
  if (!(fabs(sl - 1) < 0.05)) return sl;
  return 1.0;                     /* within 5% of 1: the entry keeps its default of 1 */
}

/* ----------------------------------------------------------------------------------------- exec lookup */

long orc_exec_nearest_T(const orc_exec_table* tab, long Tin) { /* GPUexec_lookup.cpp:29-39 */
  if (Tin < tab->T[0]) return tab->T[0];
  long ctr = 0, result = tab->T[ctr++], prev = 0;
  while (result <= Tin) {
    if (result == Tin) return result;
    prev = result;
    if (ctr >= tab->lines) return prev; /* the reference runs off the table here */
    result = tab->T[ctr++];
  }
  return prev;
}
double orc_exec_predict(const orc_exec_table* tab, long T, char ta, char tb) { /* GPUexec_lookup.cpp:103-129 */
  for (int i = 0; i < tab->lines; ++i)
    if (tab->T[i] == T && (!tab->ta || (tab->ta[i] == ta && tab->tb[i] == tb))) return tab->t[i];
  const long nearest = orc_exec_nearest_T(tab, T);
  long double reg_t = 0;
  for (int i = 0; i < tab->lines; ++i)
    if (tab->T[i] == nearest && (!tab->ta || (tab->ta[i] == ta && tab->tb[i] == tb))) {
      reg_t = tab->t[i];
      break;
    }
  if (reg_t == 0) return -1;
  return (double)(reg_t * pow((double)T, 3) / pow((double)nearest, 3)); /* cubic scaling, also for BLAS-1 */
}

/* -------------------------------------------------------------------------------------- overlap models */

static const int gemm_in[3] = {1, 1, 1}, gemm_out[3] = {0, 0, 1}; /* ModelLvl3.cpp CoCoModel_gemm_init */

static void dims_of(const orc_problem* p, int i, double* d1, double* d2) {
  /* A: D1 x D3, B: D3 x D2, C: D1 x D2 */
  *d1 = (i == 1) ? (double)p->D3 : (double)p->D1;
  *d2 = (i == 0) ? (double)p->D3 : (double)p->D2;
}

/* The "most valuable" location whose link prices a tile transfer: the location holding the most operands,
 * host winning ties (ModelLvl3.cpp:306-312).  On one GPU that is the host unless the device holds more. */
static int mv_is_host(const orc_problem* p, int numT) {
  int host = 0;
  for (int i = 0; i < numT; ++i) host += p->remote[i] ? 1 : 0;
  return host >= numT - host;
}

double orc_predict_blas3(int mode, const orc_problem* p, long T) {
  const orc_link local = {0.0, 0.0, 1.0};
  if (mode == ORC_FULL_OVERLAP || mode == ORC_NO_OVERLAP) { /* ModelLvl3.cpp:20-73, 239-284 */
    long maxT = p->exec->T[0];
    for (int i = 0; i < p->exec->lines; ++i)
      if (p->exec->T[i] > maxT) maxT = p->exec->T[i];
    double lim = fmin((double)maxT, fmin(fmin((double)p->D1, (double)p->D2), (double)p->D3));
    const long Tbig = orc_exec_nearest_T(p->exec, (long)lim);
    const double t_exec = (p->D1 * 1.0 / Tbig * p->D2 * 1.0 / Tbig * p->D3 * 1.0 / Tbig) *
                          orc_exec_predict(p->exec, Tbig, p->ta, p->tb);
    if (t_exec < 0) return -1.0;
    double t_recv = 0, t_send = 0;
    for (int i = 0; i < 3; ++i) {
      double d1, d2;
      dims_of(p, i, &d1, &d2);
      /* both directions are priced with the receive-side model there */
      t_recv += gemm_in[i] * orc_t_com_predict(p->remote[i] ? &p->h2d : &local, d1 * d2 * p->dtype_sz);
      t_send += gemm_out[i] * orc_t_com_predict(p->out_remote[i] ? &p->h2d : &local, d1 * d2 * p->dtype_sz);
    }
    return mode == ORC_FULL_OVERLAP ? fmax(t_exec, fmax(t_recv, t_send)) : t_exec + t_recv + t_send;
  }
  const double t_exec = orc_exec_predict(p->exec, T, p->ta, p->tb);
  if (t_exec < 0) return -1.0;
  const int host = mv_is_host(p, 3);
  const double tile_bytes = (double)T * T * p->dtype_sz;
  const double t_recv = orc_t_com_predict(host ? &p->h2d : &local, tile_bytes);
  const double t_send = orc_t_com_predict(host ? &p->d2h : &local, tile_bytes);
  int numTin = 0, numTout = 0;
  const double ker_over = (1.0 * p->D1 / T) * (1.0 * p->D2 / T) * (1.0 * p->D3 / T) - 1;
  if (mode == ORC_BASELINE) { /* ModelLvl3.cpp:287-346: location-blind */
    for (int i = 0; i < 3; ++i) { numTin += gemm_in[i]; numTout += gemm_out[i]; }
    const double t_over = fmax(numTin * t_recv, t_send * numTout);
    return fmax(t_exec, t_over) * ker_over + t_exec + numTin * t_recv + numTout * t_send;
  }
  if (mode == ORC_DATALOC || mode == ORC_BIDIRECTIONAL) { /* :348-408, :410-474 */
    for (int i = 0; i < 3; ++i) { numTin += gemm_in[i] * p->remote[i]; numTout += gemm_out[i] * p->remote[i]; }
    double t_over;
    if (mode == ORC_DATALOC) t_over = fmax(numTin * t_recv, t_send * numTout);
    else t_over = orc_t_com_bid_predict(host ? &p->h2d : &local, host ? &p->d2h : &local, tile_bytes * numTin, tile_bytes * numTout);
    return fmax(t_exec, t_over) * ker_over + t_exec + numTin * t_recv + numTout * t_send;
  }
  if (mode == ORC_REUSE) { /* ModelLvl3.cpp:476-551 */
    double zero_over = ker_over, one_over = 0, two_over = 0;
    for (int i = 0; i < 3; ++i) {
      double d1, d2;
      dims_of(p, i, &d1, &d2);
      numTin += gemm_in[i] * p->remote[i];
      numTout += gemm_out[i] * p->out_remote[i];
      one_over += gemm_in[i] * p->remote[i] * (d1 / T) * (d2 / T);
      if (t_recv > t_exec)
        for (int j = i + 1; j < 3; ++j)
          if ((gemm_in[i] * p->remote[i]) != 0 && (gemm_in[j] * p->remote[j]) != 0) {
            /* the shared dimension of operands i and j: (A,B) share D3 = Dim2 of A; (A,C) share D1 = Dim1 of A;
             * (B,C) share D2 = Dim2 of B.  The reference tests Dim1[i] first, then Dim2[i]. */
            if (i == 0 && j == 2) two_over += d1 / T - 1;
            else two_over += d2 / T - 1;
          }
    }
    if (2 * t_recv > t_exec && t_exec > t_recv) two_over += (1.0 * p->D3 / T);
    one_over -= (2 * two_over + numTin);
    zero_over -= (one_over + two_over);
    return t_exec * (1 + zero_over) + fmax(t_exec, t_recv) * one_over + fmax(t_exec, t_recv * 2) * two_over +
           numTin * t_recv + numTout * t_send;
  }
  return -1.0;
}

double orc_predict_blas1_bidirectional(const orc_problem* p, int numT, const int* in, const int* out, long T) {
  /* ModelLvl1.cpp:262-326 */
  const orc_link local = {0.0, 0.0, 1.0};
  const double t_exec = orc_exec_predict(p->exec, T, 0, 0);
  if (t_exec < 0) return -1.0;
  const int host = mv_is_host(p, numT);
  const double bytes = (double)T * p->dtype_sz;
  const double t_recv = orc_t_com_predict(host ? &p->h2d : &local, bytes);
  const double t_send = orc_t_com_predict(host ? &p->d2h : &local, bytes);
  int numTin = 0, numTout = 0;
  const double ker_over = (1.0 * p->D1 / T) - 1;
  for (int i = 0; i < numT; ++i) { numTin += in[i] * p->remote[i]; numTout += out[i] * p->remote[i]; }
  const double t_over = orc_t_com_bid_predict(host ? &p->h2d : &local, host ? &p->d2h : &local, bytes * numTin, bytes * numTout);
  return fmax(t_exec, t_over) * ker_over + fmax(t_exec, numTout * t_send) + numTin * t_recv + numTout * t_send;
}

double orc_predict_blas2(int mode, const orc_problem* p, long T) {
  /* ModelLvl2.cpp:89-132 (full overlap), :133-176 (zero overlap), :194-259 (bidirectional).  Operand sizes as the
   * reference declares them (CoCoModel_gemv_init, :66-71): A is D1 x D2, x D1 x 1, y D2 x 1; in = {1,1,1}, out = {0,0,1}.
   * The bidirectional model prices one tile transfer as T elements and overlaps D1/T - 1 kernels. */
  static const int in[3] = {1, 1, 1}, out[3] = {0, 0, 1};
  const orc_link local = {0.0, 0.0, 1.0};
  if (mode == ORC_FULL_OVERLAP || mode == ORC_NO_OVERLAP) {
    long maxT = p->exec->T[0];
    for (int i = 0; i < p->exec->lines; ++i) if (p->exec->T[i] > maxT) maxT = p->exec->T[i];
    const long Tbig = orc_exec_nearest_T(p->exec, (long)fmin((double)maxT, fmin((double)p->D1, (double)p->D2)));
    const double t_exec = (p->D1 * 1.0 / Tbig * p->D2 * 1.0 / Tbig) * orc_exec_predict(p->exec, Tbig, p->ta, 'N');
    double t_recv = 0, t_send = 0;
    for (int i = 0; i < 3; ++i) {
      const double d1 = (i == 2) ? (double)p->D2 : (double)p->D1, d2 = (i == 0) ? (double)p->D2 : 1.0;
      t_recv += in[i] * orc_t_com_predict(p->remote[i] ? &p->h2d : &local, d1 * d2 * p->dtype_sz);
      t_send += out[i] * orc_t_com_predict(p->out_remote[i] ? &p->h2d : &local, d1 * d2 * p->dtype_sz);
    }
    return mode == ORC_FULL_OVERLAP ? fmax(t_exec, fmax(t_recv, t_send)) : t_exec + t_recv + t_send;
  }
  if (mode != ORC_BIDIRECTIONAL) return -1.0;
  const double t_exec = orc_exec_predict(p->exec, T, p->ta, 'N');
  if (t_exec < 0) return -1.0;
  const int host = mv_is_host(p, 3);
  const double bytes = (double)T * p->dtype_sz;
  const double t_recv = orc_t_com_predict(host ? &p->h2d : &local, bytes);
  const double t_send = orc_t_com_predict(host ? &p->d2h : &local, bytes);
  int numTin = 0, numTout = 0;
  for (int i = 0; i < 3; ++i) { numTin += in[i] * p->remote[i]; numTout += out[i] * p->remote[i]; }
  const double ker_over = (1.0 * p->D1 / T) - 1;
  const double t_over = orc_t_com_bid_predict(host ? &p->h2d : &local, host ? &p->d2h : &local, bytes * numTin, bytes * numTout);
  return fmax(t_exec, t_over) * ker_over + fmax(t_exec, numTout * t_send) + numTin * t_recv + numTout * t_send;
}

long orc_optimize_tile_model(int mode, const orc_problem* p, double* pred_t) { /* Model_functions.cpp:195-244 */
  long minT = p->exec->T[0];
  for (int i = 0; i < p->exec->lines; ++i)
    if (p->exec->T[i] < minT) minT = p->exec->T[i];
  if (minT < 1024) minT = 1024; /* MinAllowedTBLAS3 */
  const long maxT = (long)fmin(fmin((double)p->D1, (double)p->D2), (double)p->D3);
  if (minT > maxT) { *pred_t = 0; return maxT; }
  double min_t = orc_predict_blas3(mode, p, p->exec->T[0]);
  long best = minT, prev = 0;
  for (int c = 1; c < p->exec->lines; ++c) {
    const long trial = p->exec->T[c];
    if (trial > maxT) break;
    if (trial == prev) continue;
    const double t = orc_predict_blas3(mode, p, trial);
    if (t >= 0 && t < min_t) { min_t = t; best = trial; }
    prev = trial;
  }
  *pred_t = min_t;
  return best;
}

/* -------------------------------------------------------------------------------------------- OpenBLAS */

static void* g_blas = NULL;
static char g_blas_path[1024] = "";
static int g_ilp64 = 0;
static void *g_dgemm, *g_sgemm, *g_dgemv, *g_daxpy, *g_ddot, *g_cfg, *g_setthr, *g_getthr;

static int try_open(const char* path) {
  void* h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!h) return 1;
  static const char* pre[] = {"cblas_", "scipy_cblas_"};
  static const char* suf[] = {"", "64_"};
  for (int s = 0; s < 2; ++s)
    for (int pr = 0; pr < 2; ++pr) {
      char name[128];
      snprintf(name, sizeof name, "%sdgemm%s", pre[pr], suf[s]);
      void* f = dlsym(h, name);
      if (!f) continue;
      g_dgemm = f;
      snprintf(name, sizeof name, "%ssgemm%s", pre[pr], suf[s]); g_sgemm = dlsym(h, name);
      snprintf(name, sizeof name, "%sdgemv%s", pre[pr], suf[s]); g_dgemv = dlsym(h, name);
      snprintf(name, sizeof name, "%sdaxpy%s", pre[pr], suf[s]); g_daxpy = dlsym(h, name);
      snprintf(name, sizeof name, "%sddot%s", pre[pr], suf[s]); g_ddot = dlsym(h, name);
      const char* op = pr ? "scipy_openblas_" : "openblas_";
      snprintf(name, sizeof name, "%sget_config%s", op, suf[s]); g_cfg = dlsym(h, name);
      snprintf(name, sizeof name, "%sset_num_threads%s", op, suf[s]); g_setthr = dlsym(h, name);
      snprintf(name, sizeof name, "%sget_num_threads%s", op, suf[s]); g_getthr = dlsym(h, name);
      g_ilp64 = s;
      g_blas = h;
      snprintf(g_blas_path, sizeof g_blas_path, "%s", path);
      return (g_sgemm && g_daxpy && g_ddot) ? 0 : 1;
    }
  dlclose(h);
  return 1;
}

int orc_openblas_open(const char* path) {
  if (g_blas) return 0;
  if (path && *path) return try_open(path);
  const char* env = getenv("PARALIA_OPENBLAS_LIB");
  if (env && *env && try_open(env) == 0) return 0;
  static const char* sys[] = {"libopenblas.so.0", "libopenblas.so", "libopenblas64_.so.0", NULL};
  for (int i = 0; sys[i]; ++i)
    if (try_open(sys[i]) == 0) return 0;
  static const char* pats[] = {"/usr/local/lib/python3*/dist-packages/numpy.libs/libscipy_openblas*.so",
                               "/usr/local/lib/python3*/dist-packages/scipy.libs/libscipy_openblas*.so",
                               "/usr/lib/python3*/dist-packages/numpy.libs/libscipy_openblas*.so",
                               "/usr/local/lib/python3*/site-packages/numpy.libs/libscipy_openblas*.so",
                               "/opt/conda/lib/python3*/site-packages/numpy.libs/libscipy_openblas*.so",
                               "/opt/conda/lib/libopenblas.so*", NULL};
  for (int i = 0; pats[i]; ++i) {
    glob_t g;
    if (glob(pats[i], 0, NULL, &g) == 0) {
      for (size_t k = 0; k < g.gl_pathc; ++k)
        if (try_open(g.gl_pathv[k]) == 0) { globfree(&g); return 0; }
      globfree(&g);
    }
  }
  return 1;
}
const char* orc_openblas_path(void) { return g_blas_path; }
const char* orc_openblas_config(void) { return g_cfg ? ((const char* (*)(void))g_cfg)() : "unknown"; }
int orc_openblas_threads(int n) {
  if (n > 0 && g_setthr) ((void (*)(int))g_setthr)(n);
  return g_getthr ? ((int (*)(void))g_getthr)() : 0;
}

enum { COL_MAJOR = 102, NO_TRANS = 111, TRANS = 112 };

int orc_openblas_dgemm(char ta, char tb, long M, long N, long K, double alpha, const double* A, long lda,
                       const double* B, long ldb, double beta, double* C, long ldc) {
  if (!g_blas) return 1;
  const int a = is_t(ta) ? TRANS : NO_TRANS, b = is_t(tb) ? TRANS : NO_TRANS;
  if (g_ilp64)
    ((void (*)(int, int, int, int64_t, int64_t, int64_t, double, const double*, int64_t, const double*, int64_t, double,
               double*, int64_t))g_dgemm)(COL_MAJOR, a, b, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
  else
    ((void (*)(int, int, int, int, int, int, double, const double*, int, const double*, int, double, double*, int))
         g_dgemm)(COL_MAJOR, a, b, (int)M, (int)N, (int)K, alpha, A, (int)lda, B, (int)ldb, beta, C, (int)ldc);
  return 0;
}
int orc_openblas_sgemm(char ta, char tb, long M, long N, long K, float alpha, const float* A, long lda, const float* B,
                       long ldb, float beta, float* C, long ldc) {
  if (!g_blas) return 1;
  const int a = is_t(ta) ? TRANS : NO_TRANS, b = is_t(tb) ? TRANS : NO_TRANS;
  if (g_ilp64)
    ((void (*)(int, int, int, int64_t, int64_t, int64_t, float, const float*, int64_t, const float*, int64_t, float,
               float*, int64_t))g_sgemm)(COL_MAJOR, a, b, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
  else
    ((void (*)(int, int, int, int, int, int, float, const float*, int, const float*, int, float, float*, int))g_sgemm)(
        COL_MAJOR, a, b, (int)M, (int)N, (int)K, alpha, A, (int)lda, B, (int)ldb, beta, C, (int)ldc);
  return 0;
}
int orc_openblas_dgemv(char ta, long M, long N, double alpha, const double* A, long lda, const double* x, long incx,
                       double beta, double* y, long incy) {
  if (!g_blas || !g_dgemv) return 1;
  const int a = is_t(ta) ? TRANS : NO_TRANS;
  if (g_ilp64)
    ((void (*)(int, int, int64_t, int64_t, double, const double*, int64_t, const double*, int64_t, double, double*,
               int64_t))g_dgemv)(COL_MAJOR, a, M, N, alpha, A, lda, x, incx, beta, y, incy);
  else
    ((void (*)(int, int, int, int, double, const double*, int, const double*, int, double, double*, int))g_dgemv)(
        COL_MAJOR, a, (int)M, (int)N, alpha, A, (int)lda, x, (int)incx, beta, y, (int)incy);
  return 0;
}
int orc_openblas_daxpy(long n, double alpha, const double* x, long incx, double* y, long incy) {
  if (!g_blas) return 1;
  if (g_ilp64) ((void (*)(int64_t, double, const double*, int64_t, double*, int64_t))g_daxpy)(n, alpha, x, incx, y, incy);
  else ((void (*)(int, double, const double*, int, double*, int))g_daxpy)((int)n, alpha, x, (int)incx, y, (int)incy);
  return 0;
}
int orc_openblas_ddot(long n, const double* x, long incx, const double* y, long incy, double* out) {
  if (!g_blas) return 1;
  if (g_ilp64) *out = ((double (*)(int64_t, const double*, int64_t, const double*, int64_t))g_ddot)(n, x, incx, y, incy);
  else *out = ((double (*)(int, const double*, int, const double*, int))g_ddot)((int)n, x, (int)incx, y, (int)incy);
  return 0;
}
