/*
 * paralia_hip.h -- C ABI of libparalia.so, the MI355X (gfx950) backend of the PARALiA tiled BLAS runtime.
 *
 * Two groups of entry points:
 *   1. pl_*       device layer: memory, streams, events, strided copies and the hand-written kernels.  This is
 *                 what the reference's backend wrapper library (headers backend_wrappers.hpp / linkmap.hpp,
 *                 included at Library_scheduler/src/Functions/dgemm.cpp:7-13) provides over CUDA + cuBLAS.
 *   2. PARALiA_*  the routines of Library_scheduler/include/PARALiA.hpp:33-72 with plain-C signatures
 *                 (declared further down); the C++ spellings PARALiADgemm ... live in PARALiA.hpp.
 *
 * Conventions: matrices are column-major, "ld" counts elements between columns, every function returns 0 on
 * success and a PL_ERR_* code otherwise, streams and events are opaque pointers (a null stream is the
 * default HIP stream), pointers passed to kernels are device pointers unless stated otherwise.
 */
#ifndef PARALIA_HIP_H
#define PARALIA_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

enum {
  PL_OK = 0,
  PL_ERR_TRANS = 1,   /* transpose flag is not 'N' or 'T' (dgemm.cpp:188-192 accepts only these) */
  PL_ERR_DIM = 2,     /* negative or oversized dimension */
  PL_ERR_LD = 3,      /* leading dimension / increment invalid */
  PL_ERR_LAUNCH = 4,  /* kernel launch failed */
  PL_ERR_NULL = 5,    /* null operand */
  PL_ERR_HIP = 6,     /* HIP runtime call failed, see pl_last_error() */
  PL_ERR_ARG = 7,     /* other invalid argument */
  PL_ERR_NOMEM = 8,   /* device block pool cannot hold the minimum working set */
  PL_ERR_DB = 9       /* autotuner database file missing or malformed */
};

/* Location codes (Benchmarking/CuCuBLAS/src/testing.cpp:296-321): device id, or one of these. */
#define PL_LOC_HOST_PINNED (-1)
#define PL_LOC_HOST_PAGEABLE (-2)

/* ---- device, memory (CoCoMalloc / CoCoFree / CoCoGetPtrLoc / CoCoPeLiaDevGetMemInfo:
 *      dgemm_runner.cpp:55-57,153-155; ModelLvl3.cpp:729-731; dgemm.cpp:50,73) ---- */
const char* pl_last_error(void);
int pl_device_count(int* count);
int pl_set_device(int dev);
int pl_get_device(int* dev);
int pl_device_sync(void);
int pl_device_name(int dev, char* buf, int len);
int pl_mem_info(long long* free_bytes, long long* total_bytes);
int pl_malloc_device(void** ptr, long long bytes);
int pl_free_device(void* ptr);
int pl_malloc_pinned(void** ptr, long long bytes);
int pl_free_pinned(void* ptr);
int pl_ptr_location(const void* ptr, int* loc);

/* ---- streams and events (CommandQueue / Event: Subkernel.cpp:162,200,249-306) ---- */
int pl_stream_create(void** stream);
int pl_stream_destroy(void* stream);
int pl_stream_sync(void* stream);
int pl_stream_query(void* stream, int* done);
int pl_event_create(void** event, int timing);
int pl_event_destroy(void* event);
int pl_event_record(void* event, void* stream);
int pl_stream_wait_event(void* stream, void* event);
int pl_event_sync(void* event);
int pl_event_query(void* event, int* done);
int pl_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---- copies (CoCoMemcpy2DAsync: Subkernel_backup.cpp:526-529,1229-1232; CoCoMemcpyAsync: :468-470;
 *      CoCoMemcpy: dgemm_runner.cpp:77; CoCoSyncCheckErr: dgemm.cpp:597) ---- */
int pl_copy2d_async(void* dst, long ld_dst, const void* src, long ld_src, long rows, long cols, int elem_size,
                    void* stream);
int pl_copy_async(void* dst, const void* src, long long bytes, void* stream);
int pl_copy(void* dst, const void* src, long long bytes);
int pl_memset_async(void* dst, int value, long long bytes, void* stream);
int pl_sync_check(void);

/* ---- kernels ---- */

/* C <- alpha*op(A)*op(B) + beta*C on one tile; replaces the cublasDgemm / cublasSgemm behind
 * backend_run_operation (Subkernel.cpp:168,228; argument set of gemm_backend_in, dgemm.cpp:382-395).
 * beta == 0 never reads C. */
int pl_dgemm_tile(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                  const double* B, long ldb, double beta, double* C, long ldc, void* stream);
int pl_sgemm_tile(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                  const float* B, long ldb, float beta, float* C, long ldc, void* stream);

/* out <- beta*src + acc on an M x N tile (out may alias acc): the ALGO_WR_LAZY reduce of a finished C tile
 * with the caller's original C (dgemm.cpp:173-179; CMakeLists.txt:78-88). */
int pl_dgeadd_tile(long M, long N, double beta, const double* src, long ld_src, const double* acc, long ld_acc,
                   double* out, long ld_out, void* stream);
int pl_sgeadd_tile(long M, long N, float beta, const float* src, long ld_src, const float* acc, long ld_acc,
                   float* out, long ld_out, void* stream);

/* y <- alpha*x + y; replaces cublasDaxpy (daxpy.cpp:62-93).  Negative increments follow BLAS. */
int pl_daxpy(long n, double alpha, const double* x, long incx, double* y, long incy, void* stream);

/* *result <- (accumulate ? *result : 0) + x.y; replaces cublasDdot (ddot.cpp:63-94).  result and workspace
 * are device pointers; workspace holds pl_ddot_workspace_doubles() doubles.  The summation order depends
 * only on n and the increments. */
long pl_ddot_workspace_doubles(void);
int pl_ddot(long n, const double* x, long incx, const double* y, long incy, double* result, int accumulate,
            double* workspace, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PARALIA_HIP_H */
