// BLAS-1 and tile-epilogue kernels for gfx950 (MI355X): daxpy, ddot, and the "lazy write-back" scale-add.
//
// Reference call sites these replace: cublasDaxpy / cublasDdot behind backend_run_operation
// (Library_scheduler/src/Functions/daxpy.cpp:62-93, ddot.cpp:63-94; direct forms
// Database_builder/CuCuBLAS/src/daxpy_microbench.cu:99,126 and ddot_microbench.cu:97,124) and the
// C_local <- reduce_mult * C_source + C_local step of the ALGO_WR_LAZY output mode
// (Library_scheduler/src/Functions/dgemm.cpp:173-179, CMakeLists.txt:78-88).
//
// All three are HBM-streaming: 16-byte loads, several independent loads in flight per lane, no LDS except
// for the ddot block reduction.  ddot is deterministic: a fixed grid (a function of n only) writes one partial
// per workgroup, a second single-workgroup kernel folds the partials in index order.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace plk {

typedef double dvec2 __attribute__((ext_vector_type(2)));
typedef float fvec4 __attribute__((ext_vector_type(4)));

constexpr int B1_THREADS = 256;
constexpr int B1_UNROLL = 4;                       // independent 16-byte vectors per lane per step (ddot)
constexpr int DOT_MAX_BLOCKS = 4096;               // upper bound on ddot partials

// y <- alpha * x + y, unit stride, both 16-byte aligned.  n2 = number of double pairs.
// One 16-byte vector per lane and one wavefront per workgroup: on MI355X the memory system is fed best by very
// many small workgroups, each touching one contiguous kilobyte of x and of y (measured 6.7 TB/s at N = 2^28, against
// 5.5 TB/s for a grid-stride loop with four vectors per lane).  Streaming (non-temporal) loads and stores keep
// the once-touched data from displacing anything in the caches.
constexpr int AXPY_THREADS = 64;
__global__ __launch_bounds__(AXPY_THREADS) void daxpy_vec_kernel(long n2, double alpha, const dvec2* __restrict__ x,
                                                                dvec2* __restrict__ y) {
  const long i = (long)blockIdx.x * AXPY_THREADS + threadIdx.x;
  if (i < n2) {
    const dvec2 xv = __builtin_nontemporal_load(x + i), yv = __builtin_nontemporal_load(y + i);
    dvec2 r;
    r.x = fma(alpha, xv.x, yv.x);
    r.y = fma(alpha, xv.y, yv.y);
    __builtin_nontemporal_store(r, y + i);
  }
}

// General strides (and the scalar tail / unaligned case): element i of x is x[i * incx], pointers pre-offset
// by the caller for negative increments.
__global__ __launch_bounds__(B1_THREADS) void daxpy_strided_kernel(long n, double alpha, const double* __restrict__ x,
                                                                  long incx, double* __restrict__ y, long incy) {
  const long stride = (long)gridDim.x * B1_THREADS;
  for (long i = (long)blockIdx.x * B1_THREADS + threadIdx.x; i < n; i += stride)
    y[i * incy] = fma(alpha, x[i * incx], y[i * incy]);
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// Sum over the workgroup in a fixed order: lanes by shuffle tree, then the 4 wave totals in wave order.
__device__ __forceinline__ double block_sum(double v) {
  __shared__ double wsum[B1_THREADS / 64];
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = v;
  __syncthreads();
  double t = 0.0;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 0; w < B1_THREADS / 64; ++w) t += wsum[w];
  }
  return t;  // valid on thread 0
}

// Each workgroup owns one contiguous chunk of the vectors and walks it with B1_UNROLL independent 16-byte loads per
// lane in flight (measured 7.1 TB/s at N = 2^28 with 4096 workgroups).
__global__ __launch_bounds__(B1_THREADS) void ddot_vec_kernel(long n2, const dvec2* __restrict__ x,
                                                             const dvec2* __restrict__ y, double* __restrict__ partials) {
  const long per = (n2 + gridDim.x - 1) / gridDim.x;
  const long b0 = (long)blockIdx.x * per, b1 = min(b0 + per, n2);
  long i = b0 + threadIdx.x;
  double acc[2 * B1_UNROLL];
#pragma unroll
  for (int u = 0; u < 2 * B1_UNROLL; ++u) acc[u] = 0.0;
  for (; i + (B1_UNROLL - 1) * B1_THREADS < b1; i += B1_UNROLL * B1_THREADS) {
    dvec2 xv[B1_UNROLL], yv[B1_UNROLL];
#pragma unroll
    for (int u = 0; u < B1_UNROLL; ++u) {
      xv[u] = __builtin_nontemporal_load(x + i + u * B1_THREADS);
      yv[u] = __builtin_nontemporal_load(y + i + u * B1_THREADS);
    }
#pragma unroll
    for (int u = 0; u < B1_UNROLL; ++u) {
      acc[2 * u] = fma(xv[u].x, yv[u].x, acc[2 * u]);
      acc[2 * u + 1] = fma(xv[u].y, yv[u].y, acc[2 * u + 1]);
    }
  }
  for (; i < b1; i += B1_THREADS) {
    dvec2 xv = x[i], yv = y[i];
    acc[0] = fma(xv.x, yv.x, acc[0]);
    acc[1] = fma(xv.y, yv.y, acc[1]);
  }
  double s = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
  s = block_sum(s);
  if (threadIdx.x == 0) partials[blockIdx.x] = s;
}

__global__ __launch_bounds__(B1_THREADS) void ddot_strided_kernel(long n, const double* __restrict__ x, long incx,
                                                                 const double* __restrict__ y, long incy,
                                                                 double* __restrict__ partials) {
  const long stride = (long)gridDim.x * B1_THREADS;
  double acc = 0.0;
  for (long i = (long)blockIdx.x * B1_THREADS + threadIdx.x; i < n; i += stride) acc = fma(x[i * incx], y[i * incy], acc);
  acc = block_sum(acc);
  if (threadIdx.x == 0) partials[blockIdx.x] = acc;
}

// result <- (accumulate ? *result : 0) + sum_{b < nparts} partials[b] (+ the products of the elements the 16-byte pairs
// of the vector kernel left out: the first nh, in front of the cache line the pairs start on, and an odd last one,
// xt / yt, null when there is none)
__global__ __launch_bounds__(B1_THREADS) void ddot_final_kernel(int nparts, const double* __restrict__ partials,
                                                               const double* __restrict__ xh, const double* __restrict__ yh, int nh,
                                                               const double* __restrict__ xt, const double* __restrict__ yt,
                                                               double* __restrict__ result, int accumulate) {
  double acc = 0.0;
  for (int i = threadIdx.x; i < nparts; i += B1_THREADS) acc += partials[i];
  acc = block_sum(acc);
  if (threadIdx.x == 0) {
    for (int i = 0; i < nh; ++i) acc = fma(xh[i], yh[i], acc);
    if (xt) acc = fma(*xt, *yt, acc);
    *result = accumulate ? *result + acc : acc;
  }
}

// out(m, n) <- beta * src(m, n) + acc(m, n) on an M x N column-major view; out may alias acc.
template <typename T, typename V, int VEC>
__global__ __launch_bounds__(B1_THREADS) void geadd_kernel(int M, int N, T beta, const T* __restrict__ src, long lds,
                                                          const T* acc, long lda, T* out, long ldo, int vec_ok) {
  const int n = blockIdx.y;
  const T* s = src + (long)n * lds;
  const T* a = acc + (long)n * lda;
  T* o = out + (long)n * ldo;
  const int m0 = (blockIdx.x * B1_THREADS + threadIdx.x) * VEC;
  if (m0 >= M) return;
  if (vec_ok && m0 + VEC <= M) {
    V sv = *reinterpret_cast<const V*>(s + m0), av = *reinterpret_cast<const V*>(a + m0), r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) r[e] = fma(beta, sv[e], av[e]);
    *reinterpret_cast<V*>(o + m0) = r;
  } else {
    for (int e = 0; e < VEC && m0 + e < M; ++e) o[m0 + e] = fma(beta, s[m0 + e], a[m0 + e]);
  }
}

inline int grid_for(long work_items, int per_block, int cap) {
  long b = (work_items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > cap) b = cap;
  return (int)b;
}

template <typename T, typename V, int VEC>
int launch_geadd(long M, long N, T beta, const T* src, long lds, const T* acc, long lda, T* out, long ldo,
                 hipStream_t stream) {
  if (M < 0 || N < 0) return 2;
  if (M == 0 || N == 0) return 0;
  if (!src || !acc || !out) return 5;
  if (lds < M || lda < M || ldo < M) return 3;
  if (N > 65535 * 1024L || M > INT32_MAX) return 2;
  const int vec_ok = (((uintptr_t)src | (uintptr_t)acc | (uintptr_t)out) & 15) == 0 && lds % VEC == 0 && lda % VEC == 0 &&
                     ldo % VEC == 0;
  // blockIdx.y is limited to 65535: walk N in slabs
  for (long n0 = 0; n0 < N; n0 += 65535) {
    const long nn = (N - n0 < 65535) ? N - n0 : 65535;
    dim3 grid((unsigned)((M + (long)B1_THREADS * VEC - 1) / ((long)B1_THREADS * VEC)), (unsigned)nn);
    hipLaunchKernelGGL((geadd_kernel<T, V, VEC>), grid, dim3(B1_THREADS), 0, stream, (int)M, (int)nn, beta,
                       src + n0 * lds, lds, acc + n0 * lda, lda, out + n0 * ldo, ldo, vec_ok);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

}  // namespace plk

extern "C" int pl_daxpy(long n, double alpha, const double* x, long incx, double* y, long incy, void* stream) {
  using namespace plk;
  if (n <= 0 || alpha == 0.0) return 0;  // BLAS: quick return, y untouched
  if (!x || !y) return 5;
  if (incx == 0 || incy == 0) return 3;
  hipStream_t s = (hipStream_t)stream;
  // 16-byte pairs when x and y sit at the same place in their 16 bytes (both on a boundary, or both 8 bytes past one):
  // the elements in front of y's next cache line are updated on their own and the pairs start on that line (x and y at
  // an odd element of an aligned array: 5.0 -> 6.7 TB/s)
  const bool pairs = incx == 1 && incy == 1 && ((((uintptr_t)x) ^ ((uintptr_t)y)) & 15) == 0 && (((uintptr_t)x) & 7) == 0;
  if (pairs) {
    long head = (long)(((128 - ((uintptr_t)y & 127)) & 127) / 8);
    if (head > n) head = n;
    if (head) hipLaunchKernelGGL(daxpy_strided_kernel, dim3(1), dim3(B1_THREADS), 0, s, head, alpha, x, 1L, y, 1L);
    const double* xv = x + head;
    double* yv = y + head;
    const long n2 = (n - head) / 2;
    if (n2 > 0) {
      // the grid's x extent caps one launch at 2^31 - 1 workgroups of 64 pairs: split longer vectors
      const long per_launch = (long)AXPY_THREADS * 0x7fffffffL;
      for (long off = 0; off < n2; off += per_launch) {
        const long m = (n2 - off < per_launch) ? n2 - off : per_launch;
        const unsigned blocks = (unsigned)((m + AXPY_THREADS - 1) / AXPY_THREADS);
        hipLaunchKernelGGL(daxpy_vec_kernel, dim3(blocks), dim3(AXPY_THREADS), 0, s, m, alpha, (const dvec2*)xv + off, (dvec2*)yv + off);
      }
    }
    if ((n - head) & 1) hipLaunchKernelGGL(daxpy_strided_kernel, dim3(1), dim3(B1_THREADS), 0, s, 1L, alpha, x + n - 1, 1L, y + n - 1, 1L);
  } else {
    // BLAS convention for negative increments: element 0 sits at the far end
    const double* xs = incx < 0 ? x + (1 - n) * incx : x;
    double* ys = incy < 0 ? y + (1 - n) * incy : y;
    const int blocks = grid_for(n, B1_THREADS * 4, 1 << 16);
    hipLaunchKernelGGL(daxpy_strided_kernel, dim3(blocks), dim3(B1_THREADS), 0, s, n, alpha, xs, incx, ys, incy);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

extern "C" long pl_ddot_workspace_doubles(void) { return plk::DOT_MAX_BLOCKS; }

// result (device pointer) <- [*result +] x . y ; workspace: device buffer of pl_ddot_workspace_doubles() doubles.
extern "C" int pl_ddot(long n, const double* x, long incx, const double* y, long incy, double* result, int accumulate,
                       double* workspace, void* stream) {
  using namespace plk;
  if (!result || !workspace) return 5;
  hipStream_t s = (hipStream_t)stream;
  if (n <= 0) {
    hipLaunchKernelGGL(ddot_final_kernel, dim3(1), dim3(B1_THREADS), 0, s, 0, workspace, (const double*)nullptr,
                       (const double*)nullptr, 0, (const double*)nullptr, (const double*)nullptr, result, accumulate);
    return hipGetLastError() == hipSuccess ? 0 : 4;
  }
  if (!x || !y) return 5;
  if (incx == 0 || incy == 0) return 3;
  // 16-byte pairs when x and y sit at the same place in their 16 bytes (both on a boundary, or both 8 bytes past one):
  // the elements in front of y's next cache line go to the final kernel and the pairs start on that line (x and y at an
  // odd element of an aligned array: 6.1 -> 7.0 TB/s)
  const bool pairs = incx == 1 && incy == 1 && ((((uintptr_t)x) ^ ((uintptr_t)y)) & 15) == 0 && (((uintptr_t)x) & 7) == 0;
  int blocks = 0;
  const double *xh = nullptr, *yh = nullptr, *xt = nullptr, *yt = nullptr;
  long head = 0;
  if (pairs) {
    head = (long)(((128 - ((uintptr_t)y & 127)) & 127) / 8);
    if (head > n) head = n;
    if (head) { xh = x; yh = y; }
    const long n2 = (n - head) / 2;
    if (n2 > 0) {
      blocks = grid_for(n2, B1_THREADS * B1_UNROLL * 4, DOT_MAX_BLOCKS);
      hipLaunchKernelGGL(ddot_vec_kernel, dim3(blocks), dim3(B1_THREADS), 0, s, n2, (const dvec2*)(x + head), (const dvec2*)(y + head), workspace);
    }
    if ((n - head) & 1) { xt = x + n - 1; yt = y + n - 1; }
  } else {
    const double* xs = incx < 0 ? x + (1 - n) * incx : x;
    const double* ys = incy < 0 ? y + (1 - n) * incy : y;
    blocks = grid_for(n, B1_THREADS * 8, DOT_MAX_BLOCKS);
    hipLaunchKernelGGL(ddot_strided_kernel, dim3(blocks), dim3(B1_THREADS), 0, s, n, xs, incx, ys, incy, workspace);
  }
  hipLaunchKernelGGL(ddot_final_kernel, dim3(1), dim3(B1_THREADS), 0, s, blocks, workspace, xh, yh, (int)head, xt, yt, result, accumulate);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

extern "C" int pl_dgeadd_tile(long M, long N, double beta, const double* src, long ld_src, const double* acc, long ld_acc,
                              double* out, long ld_out, void* stream) {
  return plk::launch_geadd<double, plk::dvec2, 2>(M, N, beta, src, ld_src, acc, ld_acc, out, ld_out, (hipStream_t)stream);
}

extern "C" int pl_sgeadd_tile(long M, long N, float beta, const float* src, long ld_src, const float* acc, long ld_acc,
                              float* out, long ld_out, void* stream) {
  return plk::launch_geadd<float, plk::fvec4, 4>(M, N, beta, src, ld_src, acc, ld_acc, out, ld_out, (hipStream_t)stream);
}
