///
/// Public C++ API of the MI355X PARALiA runtime.  Same routine names, argument order and meaning as the
/// reference's Library_scheduler/include/PARALiA.hpp:33-72: OpenBLAS-style column-major arguments, operands may
/// live in host memory (pinned or pageable) or in device memory, the location of every pointer is detected by
/// the library.  Calls are synchronous: on return the result is in the caller's buffer.  Not re-entrant.
///
/// The returned ATC_p is a fresh heap copy of the tuned controller (T, pred_t, subkernel_num ...) owned by the
/// caller, as in the reference (dgemm.cpp:689-693).  Errors print a message and terminate the process, as the
/// reference's error() does; the PARALiA_* C entry points in paralia_hip.h return status codes instead.
///
#ifndef PARALiA_H
#define PARALiA_H

#include "Autotuner.hpp"

/// C <- alpha * op(A) * op(B) + beta * C  (reference dgemm.cpp:318)
ATC_p PARALiADgemm(char TransA, char TransB, long int M, long int N, long int K, double alpha, double* A, long int ldA,
                   double* B, long int ldB, double beta, double* C, long int ldC);
/// Same with preset control values: T, cache_limit (bytes), active unit list (dgemm.cpp:697)
ATC_p PARALiADgemmControled(char TransA, char TransB, long int M, long int N, long int K, double alpha, double* A,
                            long int ldA, double* B, long int ldB, double beta, double* C, long int ldC,
                            ATC_p predef_control_values);
/// fp32 twin (sgemm.cpp:296)
ATC_p PARALiASgemm(char TransA, char TransB, long int M, long int N, long int K, float alpha, float* A, long int ldA,
                   float* B, long int ldB, float beta, float* C, long int ldC);
ATC_p PARALiASgemmControled(char TransA, char TransB, long int M, long int N, long int K, float alpha, float* A,
                            long int ldA, float* B, long int ldB, float beta, float* C, long int ldC,
                            ATC_p predef_control_values);
/// y <- alpha * x + y  (daxpy.cpp:200)
/// y = alpha * op(A) * x + beta * y with A column-major M x N (PARALiA.hpp:48-53 of the reference, dgemv.cpp:288):
/// x has N elements for TransA = 'N' and M for 'T', y the other count.
ATC_p PARALiADgemv(char TransA, long int M, long int N, double alpha, double* A, long int ldA, double* x, long int incx,
                   double beta, double* y, long int incy);
ATC_p PARALiADgemvControled(char TransA, long int M, long int N, double alpha, double* A, long int ldA, double* x,
                            long int incx, double beta, double* y, long int incy, ATC_p predef_control_values);
ATC_p PARALiADaxpy(long int N, double alpha, double* x, long int incx, double* y, long int incy);
ATC_p PARALiADaxpyControled(long int N, double alpha, double* x, long int incx, double* y, long int incy,
                            ATC_p predef_control_values);
/// *result += x . y  -- the dot product is ADDED to *result, as in the reference (ddot.cpp:431); zero it first.
ATC_p PARALiADdot(long int N, double* x, long int incx, double* y, long int incy, double* result);
ATC_p PARALiADdotControled(long int N, double* x, long int incx, double* y, long int incy, double* result,
                           ATC_p predef_control_values);
/// Frees the device block pool kept between calls (Subkernel.cpp:488)
void PARALiADevCacheFree(short dev_id);

/// Underscore spellings of the same routines.
inline ATC_p PARALiA_dgemm(char TransA, char TransB, long int M, long int N, long int K, double alpha, double* A,
                           long int ldA, double* B, long int ldB, double beta, double* C, long int ldC) {
  return PARALiADgemm(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC);
}
inline ATC_p PARALiA_sgemm(char TransA, char TransB, long int M, long int N, long int K, float alpha, float* A,
                           long int ldA, float* B, long int ldB, float beta, float* C, long int ldC) {
  return PARALiASgemm(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC);
}
inline ATC_p PARALiA_dgemv(char TransA, long int M, long int N, double alpha, double* A, long int ldA, double* x,
                           long int incx, double beta, double* y, long int incy) {
  return PARALiADgemv(TransA, M, N, alpha, A, ldA, x, incx, beta, y, incy);
}
inline ATC_p PARALiA_daxpy(long int N, double alpha, double* x, long int incx, double* y, long int incy) {
  return PARALiADaxpy(N, alpha, x, incx, y, incy);
}
inline ATC_p PARALiA_ddot(long int N, double* x, long int incx, double* y, long int incy, double* result) {
  return PARALiADdot(N, x, incx, y, incy, result);
}

#endif
