// fp64 matrix-vector product for gfx950:  y = alpha * op(A) * x + beta * y,  A column-major M x N, leading dimension lda.
//
// Stands where the reference calls cublasDgemv on one tile (gemv_backend_in<double>, Library_scheduler
// dgemv.cpp:41-118; cuBLASDgemvWrap in Benchmarking/CuCuBLAS/src/PARALia/dgemv_runner.cpp).  The routine streams A
// once (8*M*N bytes) and is bound by HBM, so both kernels are laid out for coalesced 16-byte loads and enough
// independent loads in flight, not for the matrix cores:
//   op = N  lanes run down the rows (a wave reads 1 KiB of one column per load), the four waves of a workgroup take
//           every fourth column of a column chunk and are combined through LDS;
//   op = T  four adjacent columns at a time, walked down their rows with each x load shared between the four dot
//           products and reduced with wavefront shuffles: by one wave (a workgroup takes sixteen columns) for short
//           columns, by the four waves of a workgroup together (every fourth block of rows each, combined through LDS)
//           from 2048 rows on.
// Long reductions are split into chunks (grid.y) so that about GEMV_TARGET_WGS workgroups are in flight whatever the
// shape; every chunk writes its partial sums to a workspace and a small second kernel adds them in chunk order and
// applies alpha and beta.  The summation order therefore depends only on (op, M, N), never on timing.
#include <hip/hip_runtime.h>

#include <mutex>

#include "backend/pl_internal.h"
#include "paralia_hip.h"

namespace plk {

typedef double dvec2 __attribute__((ext_vector_type(2)));

constexpr int GEMV_WG = 256;
constexpr long GEMV_TARGET_WGS = 2048;
constexpr long GEMV_N_MIN_COLS = 64;    // columns per chunk at least (16 per wave)
constexpr long GEMV_T_MIN_ROWS = 2048;  // rows per chunk at least
constexpr long GEMV_T_ROWSPLIT_FROM = 2048;  // op = T: from this many rows on the waves of a workgroup share their columns

struct GemvShape {
  long blocks_x;  // row blocks (N) or column groups (T)
  long chunks;    // grid.y
  long per_chunk; // columns (N) or rows (T) per chunk
  int vec;        // rows per lane in one load: 2 when 16-byte loads are possible, else 1
  bool rowsplit;  // op = T: the four waves of a workgroup share four columns and split the rows
  long len_y;
};

// Pure function of the arguments: the workspace size and the summation order follow from it.
__host__ inline GemvShape gemv_shape(bool trans, long M, long N, long lda, const void* A) {
  GemvShape s;
  // 16-byte loads: every column must start on a 16-byte boundary; op = T also walks the rows in pairs against x, so it
  // wants an even M, op = N gives the one lane that holds an odd last row an 8-byte load (16383 x 16383 with lda =
  // 16384: 5.4 -> 6.7 TB/s)
  s.vec = (lda % 2 == 0 && ((unsigned long long)A % 16) == 0 && (!trans || M % 2 == 0)) ? 2 : 1;
  s.rowsplit = false;
  if (!trans) {
    s.len_y = M;
    s.blocks_x = (M + 64 * s.vec - 1) / (64 * s.vec);
    long want = (GEMV_TARGET_WGS + s.blocks_x - 1) / s.blocks_x;
    long most = N / GEMV_N_MIN_COLS > 0 ? N / GEMV_N_MIN_COLS : 1;
    s.chunks = want < most ? want : most;
    if (s.chunks < 1) s.chunks = 1;
    s.per_chunk = (N + s.chunks - 1) / s.chunks;
    s.per_chunk = (s.per_chunk + 3) / 4 * 4;
    s.chunks = (N + s.per_chunk - 1) / s.per_chunk;
  } else {
    s.len_y = N;
    // long columns: a workgroup takes four columns and reads 4 KiB of each at a time (its waves take every fourth block
    // of rows) instead of sixteen columns 1 KiB at a time -- 4 GiB matrices, 16384 x 32768: 6.47 -> 6.81 TB/s, 4096 x
    // 131072: 6.25 -> 6.73, 2048 x 262144: 6.56 -> 7.05, 1048576 x 512: 6.38 -> 6.75; short columns leave waves without
    // rows (256 x 2097152: 6.47 -> 3.92) and keep a wave per four columns
    s.rowsplit = M >= GEMV_T_ROWSPLIT_FROM;
    s.blocks_x = s.rowsplit ? (N + 3) / 4 : (N + 15) / 16;
    long want = (GEMV_TARGET_WGS + s.blocks_x - 1) / s.blocks_x;
    long most = M / GEMV_T_MIN_ROWS > 0 ? M / GEMV_T_MIN_ROWS : 1;
    s.chunks = want < most ? want : most;
    if (s.chunks < 1) s.chunks = 1;
    s.per_chunk = (M + s.chunks - 1) / s.chunks;
    s.per_chunk = (s.per_chunk + 127) / 128 * 128;
    s.chunks = (M + s.per_chunk - 1) / s.per_chunk;
  }
  if (s.chunks < 1) s.chunks = 1;
  return s;
}

template <int VEC> struct RowVec;
template <> struct RowVec<2> {
  typedef dvec2 type;
  static __device__ __forceinline__ dvec2 load(const double* p) { return __builtin_nontemporal_load((const dvec2*)p); }
  // the first of the two rows only (the second one lies beyond the matrix)
  static __device__ __forceinline__ dvec2 load_first(const double* p) { dvec2 v; v.x = __builtin_nontemporal_load(p); v.y = 0.0; return v; }
  static __device__ __forceinline__ void fma_into(double* acc, dvec2 a, double xv) { acc[0] = fma(a.x, xv, acc[0]); acc[1] = fma(a.y, xv, acc[1]); }
  static __device__ __forceinline__ double dot_into(double acc, dvec2 a, const double* xv) { return fma(a.y, xv[1], fma(a.x, xv[0], acc)); }
};
template <> struct RowVec<1> {
  typedef double type;
  static __device__ __forceinline__ double load(const double* p) { return __builtin_nontemporal_load(p); }
  static __device__ __forceinline__ double load_first(const double* p) { return __builtin_nontemporal_load(p); }
  static __device__ __forceinline__ void fma_into(double* acc, double a, double xv) { acc[0] = fma(a, xv, acc[0]); }
  static __device__ __forceinline__ double dot_into(double acc, double a, const double* xv) { return fma(a, xv[0], acc); }
};

// partial[chunk * M + m] = sum over the chunk's columns n of A[m, n] * x[n]
template <int VEC>
__global__ __launch_bounds__(GEMV_WG) void gemv_n_kernel(long M, long N, const double* __restrict__ A, long lda,
                                                         const double* __restrict__ x, long incx, double* __restrict__ partial,
                                                         long cols_per_chunk) {
  __shared__ double red[4][64 * VEC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long row0 = ((long)blockIdx.x * 64 + lane) * VEC;
  const long c0 = (long)blockIdx.y * cols_per_chunk;
  const long c1 = c0 + cols_per_chunk < N ? c0 + cols_per_chunk : N;
  double acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.0;
  if (row0 < M) {
    // VEC == 2 and M odd: one lane of the launch's last row block holds the last row alone.  The row it reads along
    // with it is the padding between two columns (lda is even, so there is some) and its sum is never stored -- except in
    // the matrix's last column, where that element may lie beyond the caller's allocation: there the lane loads 8 bytes.
    const bool last_row_alone = VEC == 2 && row0 + 1 == M;
    auto rows = [&](const double* p, long n) { return (last_row_alone && n == N - 1) ? RowVec<VEC>::load_first(p) : RowVec<VEC>::load(p); };
    const double* col = A + row0;
    long n = c0 + wave;
    for (; n + 12 < c1; n += 16) {
      typename RowVec<VEC>::type a0 = rows(col + n * lda, n);
      typename RowVec<VEC>::type a1 = rows(col + (n + 4) * lda, n + 4);
      typename RowVec<VEC>::type a2 = rows(col + (n + 8) * lda, n + 8);
      typename RowVec<VEC>::type a3 = rows(col + (n + 12) * lda, n + 12);
      const double x0 = x[n * incx], x1 = x[(n + 4) * incx], x2 = x[(n + 8) * incx], x3 = x[(n + 12) * incx];
      RowVec<VEC>::fma_into(acc, a0, x0);
      RowVec<VEC>::fma_into(acc, a1, x1);
      RowVec<VEC>::fma_into(acc, a2, x2);
      RowVec<VEC>::fma_into(acc, a3, x3);
    }
    for (; n < c1; n += 4) RowVec<VEC>::fma_into(acc, rows(col + n * lda, n), x[n * incx]);
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) red[wave][lane * VEC + v] = acc[v];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const int i = lane * VEC + v;
      if (row0 + v < M) partial[(long)blockIdx.y * M + row0 + v] = ((red[0][i] + red[1][i]) + red[2][i]) + red[3][i];
    }
  }
}

// partial[chunk * N + n] = sum over the chunk's rows m of A[m, n] * x[m]
template <int VEC>
__global__ __launch_bounds__(GEMV_WG) void gemv_t_kernel(long M, long N, const double* __restrict__ A, long lda,
                                                         const double* __restrict__ x, long incx, double* __restrict__ partial,
                                                         long rows_per_chunk, int rowsplit) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (rowsplit) {
    // the four waves share four columns and take every fourth block of 64 * VEC rows: the workgroup reads 4 KiB of each
    // column at a time
    __shared__ double red[4][4];
    const long col0 = (long)blockIdx.x * 4;
    const int ncols = N - col0 < 4 ? (int)(N - col0) : 4;
    const long r0 = (long)blockIdx.y * rows_per_chunk;
    const long r1 = r0 + rows_per_chunk < M ? r0 + rows_per_chunk : M;
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    const double* base = A + col0 * lda;
    if (ncols == 4) {
      for (long m = r0 + ((long)wave * 64 + lane) * VEC; m < r1; m += 4 * 64 * VEC) {
        double xv[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) xv[v] = x[(m + v) * incx];
        typename RowVec<VEC>::type a[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c] = RowVec<VEC>::load(base + c * lda + m);
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] = RowVec<VEC>::dot_into(acc[c], a[c], xv);
      }
    } else {
      for (long m = r0 + wave * 64 + lane; m < r1; m += 256) {
        const double xv = x[m * incx];
        for (int c = 0; c < ncols; ++c) acc[c] = fma(base[c * lda + m], xv, acc[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c)
      for (int off = 32; off > 0; off >>= 1) acc[c] += __shfl_down(acc[c], off, 64);
    if (lane == 0)
      for (int c = 0; c < 4; ++c) red[wave][c] = acc[c];
    __syncthreads();
    if (threadIdx.x < ncols) partial[(long)blockIdx.y * N + col0 + threadIdx.x] = ((red[0][threadIdx.x] + red[1][threadIdx.x]) + red[2][threadIdx.x]) + red[3][threadIdx.x];
    return;
  }
  const long col0 = ((long)blockIdx.x * 4 + wave) * 4;
  if (col0 >= N) return;
  const int ncols = N - col0 < 4 ? (int)(N - col0) : 4;
  const long r0 = (long)blockIdx.y * rows_per_chunk;
  const long r1 = r0 + rows_per_chunk < M ? r0 + rows_per_chunk : M;
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  const double* base = A + col0 * lda;
  if (ncols == 4) {
    for (long m = r0 + (long)lane * VEC; m < r1; m += 64 * VEC) {  // VEC == 2: M and the chunk size are even
      double xv[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) xv[v] = x[(m + v) * incx];
      typename RowVec<VEC>::type a[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) a[c] = RowVec<VEC>::load(base + c * lda + m);
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = RowVec<VEC>::dot_into(acc[c], a[c], xv);
    }
  } else {
    for (long m = r0 + lane; m < r1; m += 64) {
      const double xv = x[m * incx];
      for (int c = 0; c < ncols; ++c) acc[c] = fma(base[c * lda + m], xv, acc[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c)
    for (int off = 32; off > 0; off >>= 1) acc[c] += __shfl_down(acc[c], off, 64);
  if (lane == 0)
    for (int c = 0; c < ncols; ++c) partial[(long)blockIdx.y * N + col0 + c] = acc[c];
}

// y[i] = alpha * (partial[0][i] + partial[1][i] + ...) + beta * y[i]; beta == 0 never reads y (NaN-safe, as in BLAS)
__global__ __launch_bounds__(GEMV_WG) void gemv_final_kernel(long len, long chunks, const double* __restrict__ partial, double alpha,
                                                             double beta, double* __restrict__ y, long incy) {
  const long i = (long)blockIdx.x * GEMV_WG + threadIdx.x;
  if (i >= len) return;
  double s = 0.0;
  for (long c = 0; c < chunks; ++c) s += partial[c * len + i];
  double* yp = y + i * incy;
  *yp = beta == 0.0 ? alpha * s : fma(alpha, s, beta * *yp);
}

// The same for a short y with many chunks (a wide op = N or a tall op = T matrix: 128 x 4194304 has 2064 chunks of
// 128 sums, and one thread per element of y adding them one after the other took 490 us of a 1100 us call).  A workgroup
// takes 16 elements of y and cuts the chunks into 16 runs, one per thread of an element; a thread adds its run in four
// interleaved sums, the sixteen runs are combined in LDS in run order.  The order depends on the shape only.
constexpr int GEMV_FIN_ROWS = 16, GEMV_FIN_RUNS = GEMV_WG / GEMV_FIN_ROWS, GEMV_FIN_WIDE_FROM = 64;
__global__ __launch_bounds__(GEMV_WG) void gemv_final_wide_kernel(long len, long chunks, const double* __restrict__ partial, double alpha,
                                                                  double beta, double* __restrict__ y, long incy) {
  __shared__ double red[GEMV_FIN_RUNS][GEMV_FIN_ROWS];
  const int r = threadIdx.x % GEMV_FIN_ROWS, run = threadIdx.x / GEMV_FIN_ROWS;
  const long i = (long)blockIdx.x * GEMV_FIN_ROWS + r;
  double s = 0.0;
  if (i < len) {
    const long per = (chunks + GEMV_FIN_RUNS - 1) / GEMV_FIN_RUNS;
    const long c0 = run * per, c1 = c0 + per < chunks ? c0 + per : chunks;
    double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
    long c = c0;
    for (; c + 3 < c1; c += 4) {
      a0 += partial[c * len + i];
      a1 += partial[(c + 1) * len + i];
      a2 += partial[(c + 2) * len + i];
      a3 += partial[(c + 3) * len + i];
    }
    for (; c < c1; ++c) a0 += partial[c * len + i];
    s = (a0 + a1) + (a2 + a3);
  }
  red[run][r] = s;
  __syncthreads();
  if (run == 0 && i < len) {
    s = red[0][r];
#pragma unroll
    for (int k = 1; k < GEMV_FIN_RUNS; ++k) s += red[k][r];
    double* yp = y + i * incy;
    *yp = beta == 0.0 ? alpha * s : fma(alpha, s, beta * *yp);
  }
}

// Launches the chunk kernel and the final kernel on `stream`; `workspace` receives the chunks' partial sums.
static int launch_gemv(char trans, long M, long N, double alpha, const double* A, long lda, const double* x, long incx, double beta,
                       double* y, long incy, double* workspace, void* stream) {
  const bool is_n = trans == 'N' || trans == 'n';
  const bool is_t = trans == 'T' || trans == 't' || trans == 'C' || trans == 'c';
  if (!is_n && !is_t) return PL_ERR_TRANS;
  if (M < 0 || N < 0) return PL_ERR_DIM;
  if (lda < (M > 1 ? M : 1)) return PL_ERR_LD;
  if (incx == 0 || incy == 0) return PL_ERR_LD;
  if (M == 0 || N == 0 || (alpha == 0.0 && beta == 1.0)) return 0;  // BLAS quick return: y untouched
  if (!A || !x || !y) return PL_ERR_NULL;
  hipStream_t st = (hipStream_t)stream;
  const long len_x = is_n ? N : M, len_y = is_n ? M : N;
  // BLAS: with a negative increment the vector runs backwards from the far end of its span
  const double* xs = incx > 0 ? x : x - (len_x - 1) * incx;
  double* ys = incy > 0 ? y : y - (len_y - 1) * incy;
  const unsigned fin_blocks = (unsigned)((len_y + GEMV_WG - 1) / GEMV_WG);
  if (alpha == 0.0) {
    hipLaunchKernelGGL(gemv_final_kernel, dim3(fin_blocks), dim3(GEMV_WG), 0, st, len_y, 0L, (const double*)nullptr, 0.0, beta, ys, incy);
    return hipGetLastError() == hipSuccess ? 0 : PL_ERR_HIP;
  }
  if (!workspace) return PL_ERR_NULL;
  const GemvShape s = gemv_shape(is_t, M, N, lda, A);
  if (s.blocks_x > 0x7fffffffL || s.chunks > 65535) return PL_ERR_DIM;
  const dim3 grid((unsigned)s.blocks_x, (unsigned)s.chunks);
  if (is_n) {
    if (s.vec == 2) hipLaunchKernelGGL(gemv_n_kernel<2>, grid, dim3(GEMV_WG), 0, st, M, N, A, lda, xs, incx, workspace, s.per_chunk);
    else hipLaunchKernelGGL(gemv_n_kernel<1>, grid, dim3(GEMV_WG), 0, st, M, N, A, lda, xs, incx, workspace, s.per_chunk);
  } else {
    const int rs = s.rowsplit ? 1 : 0;
    if (s.vec == 2) hipLaunchKernelGGL(gemv_t_kernel<2>, grid, dim3(GEMV_WG), 0, st, M, N, A, lda, xs, incx, workspace, s.per_chunk, rs);
    else hipLaunchKernelGGL(gemv_t_kernel<1>, grid, dim3(GEMV_WG), 0, st, M, N, A, lda, xs, incx, workspace, s.per_chunk, rs);
  }
  if (s.chunks >= GEMV_FIN_WIDE_FROM)
    hipLaunchKernelGGL(gemv_final_wide_kernel, dim3((unsigned)((len_y + GEMV_FIN_ROWS - 1) / GEMV_FIN_ROWS)), dim3(GEMV_WG), 0, st, len_y, s.chunks,
                       (const double*)workspace, alpha, beta, ys, incy);
  else
    hipLaunchKernelGGL(gemv_final_kernel, dim3(fin_blocks), dim3(GEMV_WG), 0, st, len_y, s.chunks, (const double*)workspace, alpha, beta, ys, incy);
  return hipGetLastError() == hipSuccess ? 0 : PL_ERR_HIP;
}

// ---- scratch of the allocation-free entry point ----
// The partial sums of pl_dgemv_noalloc go to this array instead of a caller-provided workspace.  Every GPU holds its
// own copy, at its own address, from the moment the code object is loaded there until the process ends.  In host
// code the name is only a handle for hipGetSymbolAddress; kernels get the address that call returned.
static __device__ __align__(256) double scratch[PL_DGEMV_NOALLOC_MAX_DOUBLES];

constexpr int NOALLOC_MAX_DEVICES = 64;
static std::mutex scratch_mu;
static double* scratch_ptr[NOALLOC_MAX_DEVICES];  // address of `scratch` on device d; null until the first call there

// Address of the current device's copy of `scratch`, looked up once per device.
static int noalloc_scratch(double** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return pl_fail_hip((int)e, "pl_dgemv_noalloc: hipGetDevice");
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return pl_fail_msg(PL_ERR_ARG, "pl_dgemv_noalloc: device index beyond the per-device table");
  std::lock_guard<std::mutex> lk(scratch_mu);
  if (!scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return pl_fail_hip((int)e, "pl_dgemv_noalloc: hipGetSymbolAddress(scratch)");
    if (!p) return pl_fail_msg(PL_ERR_HIP, "pl_dgemv_noalloc: hipGetSymbolAddress(scratch) returned a null address");
    scratch_ptr[dev] = (double*)p;
  }
  *out = scratch_ptr[dev];
  return 0;
}

}  // namespace plk

// Set-up half of pl_dgemv_noalloc: looks the scratch address of the current device up, which may make the runtime load
// the code object there.  pl_set_device and pl_stream_create call it, so that a caller who holds a stream from this
// library never pays for it inside pl_dgemv_noalloc (under graph capture, say).
int pl_noalloc_setup_current_device(void) {
  double* unused = nullptr;
  return plk::noalloc_scratch(&unused);
}

extern "C" {

long long pl_dgemv_workspace_doubles(char trans, long M, long N) {
  if (M <= 0 || N <= 0) return 0;
  const bool t = !(trans == 'N' || trans == 'n');
  // the chunk count depends on which load width the launch will pick (parity of M and lda, alignment of A):
  // take the larger of the two
  const plk::GemvShape wide = plk::gemv_shape(t, M + (M & 1), N, 2, nullptr);
  const plk::GemvShape narrow = plk::gemv_shape(t, M, N, 1, nullptr);
  const long chunks = wide.chunks > narrow.chunks ? wide.chunks : narrow.chunks;
  return (long long)chunks * (wide.len_y + 1);
}

int pl_dgemv(char trans, long M, long N, double alpha, const double* A, long lda, const double* x, long incx, double beta,
             double* y, long incy, double* workspace, void* stream) {
  return plk::launch_gemv(trans, M, N, alpha, A, lda, x, incx, beta, y, incy, workspace, stream);
}

long long pl_dgemv_noalloc_max_doubles(void) { return PL_DGEMV_NOALLOC_MAX_DOUBLES; }

// pl_dgemv without a workspace argument and without any allocation: same kernels, same chunking, same summation
// order, partial sums in the per-device static array above.  Every chunk writes its whole slice before the final
// kernel reads it, so nothing has to be cleared between calls.
int pl_dgemv_noalloc(char trans, long M, long N, double alpha, const double* A, long lda, const double* x, long incx, double beta,
                     double* y, long incy, void* stream) {
  if (M > 0 && N > 0 && pl_dgemv_workspace_doubles(trans, M, N) > PL_DGEMV_NOALLOC_MAX_DOUBLES)
    return pl_fail_msg(PL_ERR_DIM, "pl_dgemv_noalloc: this shape needs more partial sums than the fixed scratch holds "
                                   "(pl_dgemv_workspace_doubles > pl_dgemv_noalloc_max_doubles); use pl_dgemv with a workspace");
  double* ws = nullptr;
  const int rc = plk::noalloc_scratch(&ws);
  if (rc != 0) return rc;
  return plk::launch_gemv(trans, M, N, alpha, A, lda, x, incx, beta, y, incy, ws, stream);
}

}  // extern "C"
