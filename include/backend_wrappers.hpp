///
/// Helper surface the PARALiA drivers link against: allocation by location code, copies, seeded fill,
/// equality tests, timers and flop counters.  In the reference these come from its backend wrapper library
/// (un-vendored; call sites Benchmarking/CuCuBLAS/src/PARALia/dgemm_runner.cpp:45-110,146-155 and
/// Benchmarking/CuCuBLAS/src/testing.cpp:273-428).  Location codes: >= 0 device id, -1 page-locked host,
/// -2 pageable host.
///
#ifndef PARALIA_BACKEND_WRAPPERS_HPP
#define PARALIA_BACKEND_WRAPPERS_HPP

#include <cstdio>
#include <stdexcept>
#include <string>

/// Thrown by error(); the C++ routine entry points let it reach the caller's frame, print it and terminate
/// the process (the reference's error() prints and exits); the C entry points turn it into a status code.
struct paralia_error : public std::runtime_error {
  int code;
  paralia_error(int c, const std::string& what) : std::runtime_error(what), code(c) {}
};

[[noreturn]] void error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void warning(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void massert(bool cond, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

double csecond();

void* CoCoMalloc(long long bytes, short loc, short write_flag = 0);
void CoCoFree(void* ptr, short loc);
void CoCoMemcpy(void* dest, void* src, long long bytes, short loc_dest, short loc_src);
void CoCoSyncCheckErr();
short CoCoGetPtrLoc(const void* ptr);
void CoCoPeLiaSelectDevice(short dev_id);
short CoCoPeLiaGetDevice();
void CoCoPeLiaDevGetMemInfo(long long* free_dev_mem, long long* max_dev_mem);

/// Fill with uniform values in [-1, 1).  Element i of a stream is a pure function of (seed, i)
/// (splitmix64 of seed * 0xD1342543DE82EF95 + i * 0x9E3779B97F4A7C15), so the same (seed, n) gives the same
/// data wherever the buffer lives; device buffers are filled through a pinned staging buffer.
template <typename T> void CoCoVecInit(T* vec, long long length, int seed, short loc);

/// Number of matching decimal digits of the worst element, capped at 16 (fp64) / 7 (fp32).
short Dtest_equality(double* C_comp, double* C, long long size);
short Stest_equality(float* C_comp, float* C, long long size);

inline double Gval_per_s(long long value, double time) { return value / (time * 1e9); }
inline long long gemm_flops(long M, long N, long K) { return (long long)M * K * (2 * N + 1); }
inline long long gemm_memory(long M, long N, long K, long A_loc, long B_loc, long C_loc, short dsize) {
  return ((long long)M * K * A_loc + (long long)K * N * B_loc + (long long)M * N * C_loc) * dsize;
}
inline long long gemv_flops(long M, long N) { return (long long)M * (2 * N + 1); }  // by analogy with gemm_flops (the reference's own is un-vendored)
inline long long axpy_flops(long N) { return 2LL * N; }
inline long long dot_flops(long N) { return 2LL * N; }

/// Leading dimension of a stored operand: rows of the matrix as stored.
inline void TransposeTranslate(char TransChar, long* ldim, long dim1, long dim2) {
  *ldim = (TransChar == 'N' || TransChar == 'n') ? dim1 : dim2;
}
/// The call shape of the reference's drivers (dgemm_runner.cpp:44-46, dgemv_runner.cpp:47):
///   TransposeTranslate(TransA, &cpu_op_A, &gpu_op_A, &ldA, M, K);
/// The two operation out-parameters have the types of the host BLAS and of the device BLAS the driver was written
/// for; here they are whatever enum or integer types the driver declares.  They receive the CBLAS codes
/// (111 no-transpose, 112 transpose) and 0 / 1 respectively; nothing in this library reads them back.
template <typename HostOp, typename DeviceOp>
inline void TransposeTranslate(char TransChar, HostOp* host_op, DeviceOp* device_op, long* ldim, long dim1, long dim2) {
  const bool n = (TransChar == 'N' || TransChar == 'n');
  if (!n && TransChar != 'T' && TransChar != 't') error("TransposeTranslate: %c is an invalid Trans parameter\n", TransChar);
  if (host_op) *host_op = static_cast<HostOp>(n ? 111 : 112);
  if (device_op) *device_op = static_cast<DeviceOp>(n ? 0 : 1);
  *ldim = n ? dim1 : dim2;
}

#endif
