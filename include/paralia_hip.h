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
/* *shares <- 1 when `candidate` executes in order with at least one of others[0 .. n-1] (n <= PL_MAX_PROBE_STREAMS),
 * i.e. HIP placed it on the same hardware queue; 0 when its work can overlap theirs.  Launches two tiny kernels per
 * stream and waits for them (about half a millisecond).  The reference creates its queues per link and per backend
 * worker (Subkernel.cpp:249-306) and relies on CUDA streams being independent; HIP streams are only independent when
 * they sit on different hardware queues. */
#define PL_MAX_PROBE_STREAMS 8
int pl_stream_shares_queue(void* candidate, void* const* others, int n, int* shares);

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

/* The same product with a device workspace: when the 128 x 128 tiles of C are too few to occupy the compute units
 * (small or skinny products), K is split over several workgroups per tile, their partial products go to the
 * workspace and a second kernel adds them in a fixed order (the result is reproducible).  cuBLAS makes the same
 * choice internally behind the call sites above.  pl_gemm_tile_workspace_bytes returns what a given shape can
 * use (0: it would not be split); a null or smaller workspace falls back to the unsplit kernel.  The workspace
 * must not be shared by launches that may overlap (one per stream). */
long pl_gemm_tile_workspace_bytes(long M, long N, long K, int elem_size);
int pl_dgemm_tile_ws(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                     const double* B, long ldb, double beta, double* C, long ldc, void* workspace, long workspace_bytes,
                     void* stream);
int pl_sgemm_tile_ws(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                     const float* B, long ldb, float beta, float* C, long ldc, void* workspace, long workspace_bytes,
                     void* stream);

/* The same again with the caller's split count instead of the model's: K goes to `splits` workgroups per tile of C (in
 * whole panels, so the count used may be lower; 1, or a workspace under splits * M * N elements, launches the unsplit
 * kernel; a count below 1 is PL_ERR_ARG).  For a scheduler that knows a product will have the device to itself, where the model above assumes a
 * second product running beside it (the end of a call: the reference's last subkernels of Subkernel.cpp:168 run alone
 * on their queue). */
int pl_dgemm_tile_split(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                        const double* B, long ldb, double beta, double* C, long ldc, void* workspace, long workspace_bytes,
                        int splits, void* stream);
int pl_sgemm_tile_split(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                        const float* B, long ldb, float beta, float* C, long ldc, void* workspace, long workspace_bytes,
                        int splits, void* stream);

/* The product on operands that live in larger blocks (the scheduler's tiles in its device pool: the reference's tiles
 * in CBlocks, DataCaching.hpp).  m_readable >= M rows of op(A) and n_readable >= N columns of op(B) may be READ -- the
 * memory is there, its content beyond M and N is anything -- so the workgroups on the ragged edge of C load whole
 * 128-wide tiles without guards like the interior ones (what they read from beyond only reaches elements of C that
 * are not stored).  0 stands for M or N.  splits: 0 the launcher's choice as in pl_dgemm_tile_ws, >= 1 as in
 * pl_dgemm_tile_split, -1 its choice for a product alone on the device as in pl_dgemm_tile_alone (declared below). */
int pl_dgemm_tile_padded(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                         const double* B, long ldb, double beta, double* C, long ldc, void* workspace, long workspace_bytes,
                         int splits, long m_readable, long n_readable, void* stream);
int pl_sgemm_tile_padded(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                         const float* B, long ldb, float beta, float* C, long ldc, void* workspace, long workspace_bytes,
                         int splits, long m_readable, long n_readable, void* stream);

/* The product for a caller who knows it has the device to itself (every operand already in HBM and nothing else
 * running: the reference's call with all data on the GPU is one cublasDgemm, dgemm.cpp:382-395 with a single
 * subkernel).  The launcher then counts whole rounds of two workgroups per compute unit instead of assuming a second
 * product beside this one, and splits K where that fills the last round (a 3072 x 3072 x 16384 product: 576 tiles, 52.7
 * TFLOP/s unsplit, 73.7 split four ways).  pl_gemm_tile_alone_workspace_bytes: what that choice can use (at most 1 GiB;
 * 0: not split); pl_gemm_tile_choice_alone reports the choice like pl_gemm_tile_choice.  Where the tiles do not fill
 * whole rounds and K is too short for the slices of all of C to pay, the product is cut along N instead: the first
 * n_head columns of C (whole tile columns) in one unsplit launch, the rest in a second one that splits K tail_splits
 * ways (3072^3 fp64: 21 of 24 tile columns, the last three split seven ways).  pl_gemm_tile_cut_alone reports that:
 * *n_head == N and *tail_splits == 0 when the product stays one launch; PARALIA_GEMM_TAIL=0 switches the cut off. */
long pl_gemm_tile_alone_workspace_bytes(char transA, char transB, long M, long N, long K, int beta_is_zero, int elem_size);
int pl_dgemm_tile_alone(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                        const double* B, long ldb, double beta, double* C, long ldc, void* workspace, long workspace_bytes,
                        void* stream);
int pl_sgemm_tile_alone(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                        const float* B, long ldb, float beta, float* C, long ldc, void* workspace, long workspace_bytes,
                        void* stream);
int pl_gemm_tile_choice_alone(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero,
                              long workspace_bytes, int* tile_m, int* tile_n, int* splits);
int pl_gemm_tile_cut_alone(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero,
                           long workspace_bytes, long* n_head, int* tail_splits);
/* the launcher's own estimate of that product's time on the device in microseconds, kernels only (< 0: bad arguments) */
double pl_gemm_tile_alone_us(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero,
                             long workspace_bytes);

/* Fitted constants of the tile-GEMM launcher's cost model: how it chooses between its macro tiles (fp32: 128 x 128,
 * 256 x 128 "wide", 256 x 256 "large") and how many ways it splits K for products with few tiles.  They describe one
 * device and one build of the kernels; the deploy tool measures them and writes Processed/Kernel-fit_dev-<id>.log, the
 * autotuner's database loader hands them over with pl_gemm_set_fit (the role of the reference's deploy-time kernel
 * tables, Deploy.in:14-18, Database_builder/CuCuBLAS/src/dgemm_microbench.cu:125-160, for a library that owns its
 * kernels).  Without a call the built-in values (measured on an MI355X) apply.  Times in microseconds.
 * Transpose index: 0 NN, 1 NT, 2 TN, 3 TT. */
typedef struct pl_gemm_fit {
  double lone_us_per_k[2];          /* [0] fp64, [1] fp32: one 128 x 128 workgroup per compute unit, per unit of k */
  double lone_fixed_k;              /* its prologue and epilogue, in units of k */
  double splitk_launch_us;          /* the second launch of a split product */
  double pass_bytes_per_us;         /* rate of the pass that adds the split-K slices */
  double f32_small_us_per_k;        /* a round of 512 small fp32 tiles (two per compute unit), per unit of k */
  double f32_small_fixed_us;        /* ... and its fixed part */
  double f32_wide_gain;             /* wide tile: 2 * f32_small_us_per_k * K / gain per round of 512 */
  double f32_wide_fixed_us[2];      /* beta == 0, beta != 0 */
  double f32_large_gain[4];         /* large tile: 2 * f32_small_us_per_k * K / (1 + gain) per round of 256, per transpose */
  double f32_large_fixed_us[4][2];  /* per transpose; beta == 0, beta != 0 */
  double edge_rounds[2];            /* what the guarded edge workgroups of a grid with a ragged last row or column add to a
                                       product alone on the device, in rounds: [0] 128 x 128 tiles, [1] 256-wide tiles */
} pl_gemm_fit;
void pl_gemm_fit_defaults(pl_gemm_fit* fit);
int pl_gemm_set_fit(const pl_gemm_fit* fit);   /* null: back to the built-in values */
int pl_gemm_get_fit(pl_gemm_fit* fit);
/* What the launcher would do for a product (no GPU call): macro tile rows and columns, and the split count it would use
 * given a workspace of workspace_bytes (0: none).  elem_size 8 or 4. */
int pl_gemm_tile_choice(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero, long workspace_bytes,
                        int* tile_m, int* tile_n, int* splits);

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

/* y <- alpha*op(A)*x + beta*y, A column-major M x N; replaces cublasDgemv on a tile or on a whole device-resident
 * matrix (gemv_backend_in<double>, dgemv.cpp:41-118).  All pointers are device pointers; workspace holds
 * pl_dgemv_workspace_doubles(trans, M, N) doubles (partial sums of the reduction chunks; the chunking, and with it the
 * summation order, depends only on the shape, the parity of M and lda, and the 16-byte alignment of A).  BLAS quick returns: M == 0, N == 0, or alpha == 0 with
 * beta == 1 leave y untouched; beta == 0 never reads y. */
long long pl_dgemv_workspace_doubles(char trans, long M, long N);
int pl_dgemv(char trans, long M, long N, double alpha, const double* A, long lda, const double* x, long incx, double beta,
             double* y, long incy, double* workspace, void* stream);

/* pl_dgemv for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): no workspace argument and no allocation of any kind inside the call.  It has no counterpart in the
 * reference.  The partial sums go to a fixed array of PL_DGEMV_NOALLOC_MAX_DOUBLES doubles (4 MiB) that every GPU
 * the library runs on holds until the process ends; kernels, chunking and summation order are those of pl_dgemv,
 * so the results are bitwise the same.  A shape with pl_dgemv_workspace_doubles(trans, M, N) above that size is
 * refused with PL_ERR_DIM (pl_last_error() says why).  All calls on one GPU share the array and nothing in the call
 * checks for a call still in flight (a check would need an event query, which graph capture forbids): the caller must
 * serialise them -- calls on one stream are safe, calls that may overlap on different streams or threads race.  The
 * array's address on a device is resolved by pl_set_device and pl_stream_create on that device (the look-up may make
 * the HIP runtime load the code object, which is not something to do under capture); only a caller who has used
 * neither pays for it in its first pl_dgemv_noalloc call there. */
#define PL_DGEMV_NOALLOC_MAX_DOUBLES 524288
long long pl_dgemv_noalloc_max_doubles(void);
int pl_dgemv_noalloc(char trans, long M, long N, double alpha, const double* A, long lda, const double* x, long incx,
                     double beta, double* y, long incy, void* stream);

/* ---- routines: plain-C faces of Library_scheduler/include/PARALiA.hpp:33-72 ----
 * Operands may be host (pinned or pageable) or device pointers; the library detects which.  Calls return
 * after the result has reached the caller's buffer.  T > 0 / cache_limit > 0 preset the tile size and the
 * device block-pool limit in bytes (the ...Controled variants, PARALiA.hpp:37-38; unset: T <= 0, limit 0,
 * Autotuner.cpp:27-31).  info, when not null, receives what the returned ATC_p carries in C++. */
typedef struct pl_atc_info {
  long T;                 /* tile size used */
  double pred_t;          /* predicted seconds */
  long subkernel_num;
  int order_id;           /* subkernel order family picked by the pipeline model */
  int exec_queues;
  long long cache_limit;
  int has_db;             /* autotuner database found */
  char selected_by[32];   /* user | resident | pipeline-model | cocopelia-reuse | cocopelia-bidirectional | heuristic */
  double slowdowns[6];    /* T_aggregate, imbalance, remainder, small, sknum, big (Autotuner.cpp:561-569) */
  double pipe_total, pipe_h2d, pipe_exec, pipe_d2h;
} pl_atc_info;

const char* PARALiA_last_error(void);
/* PARALiADgemm / PARALiADgemmControled (dgemm.cpp:318,697) */
int PARALiA_dgemm(char TransA, char TransB, long M, long N, long K, double alpha, double* A, long ldA, double* B, long ldB,
                  double beta, double* C, long ldC, long T, long long cache_limit, pl_atc_info* info);
/* PARALiASgemm / PARALiASgemmControled (sgemm.cpp:296) */
int PARALiA_sgemm(char TransA, char TransB, long M, long N, long K, float alpha, float* A, long ldA, float* B, long ldB,
                  float beta, float* C, long ldC, long T, long long cache_limit, pl_atc_info* info);
/* PARALiADaxpy / PARALiADaxpyControled (daxpy.cpp:200) */
int PARALiA_daxpy(long N, double alpha, double* x, long incx, double* y, long incy, long T, pl_atc_info* info);
/* PARALiADdot / PARALiADdotControled (ddot.cpp:201): the dot product is ADDED to *result (ddot.cpp:431) */
int PARALiA_ddot(long N, double* x, long incx, double* y, long incy, double* result, long T, pl_atc_info* info);
/* PARALiADgemv / PARALiADgemvControled (dgemv.cpp:288,720, PARALiA.hpp:48-53): y <- alpha*op(A)*x + beta*y; x has N
 * ('N') or M ('T') elements, y the other count */
int PARALiA_dgemv(char TransA, long M, long N, double alpha, double* A, long ldA, double* x, long incx, double beta, double* y,
                  long incy, long T, long long cache_limit, pl_atc_info* info);
/* PARALiADevCacheFree (Subkernel.cpp:488): device 0 gives back the block pool, the split-K workspaces and the
 * aligned copies of unaligned device-resident GEMM operands; streams, events and the cached problems stay */
int PARALiA_dev_cache_free(int dev_id);
/* metadata-cache and pool counters (PMD_cache, dgemm.cpp:342-368); reset drops the cached problems */
int PARALiA_runtime_stats(long* pmd_hits, long* pmd_misses, long long* pool_bytes, long* pmd_entries);
int PARALiA_runtime_reset(void);
/* releases everything the library holds: device block pool, streams, events, workspaces, pinned bounce buffers and
 * the cached problems (CoCoPeLiaFreeResources, Subkernel.cpp:330, together with PARALiADevCacheFree); the next call
 * creates what it needs again */
int PARALiA_runtime_shutdown(void);
/* per-command timeline of the streamed GEMM calls (what the reference's STEST / TTEST builds print per subkernel,
 * Subkernel.cpp:498, dgemm.cpp:612-615).  While enabled, every command of a call's plan is bracketed by two timing
 * events on its stream; PARALiA_trace_read copies the rows of the most recent such call, PL_TRACE_ROW doubles each:
 * kind (0 fetch A, 1 fetch B, 2 fetch C, 3 tile GEMM, 4 lazy reduce, 5 write-back), mi, ni, ki, stream (0 H2D, 1 D2H,
 * 2.. compute), start and end in milliseconds since the call's first command.  Returns the number of rows the call
 * had (rows may be null to ask for the count).  Tracing costs a few percent; leave it off when timing. */
#define PL_TRACE_ROW 7
int PARALiA_trace_enable(int on);
long PARALiA_trace_read(double* rows, long max_rows);
/* host-side phases of the most recent PARALiA_dgemm / PARALiA_sgemm call, in seconds: [0] autotune (database lookups,
 * tile and order search), [1] plan (static plan of the chosen order), [2] device block pool (allocation or growth),
 * [3] streams (creation and placement test), [4] execution (enqueue, device work, final sync), [5] whole call.  [0] and
 * [1] are 0 when the problem came from the metadata cache.  What the reference's TEST build prints per call
 * (dgemm.cpp:330-333,430-445,497-511,598-604). */
int PARALiA_last_call_phases(double seconds[6]);
/* the scheduler's stream inventory: *independent <- how many of its four busy streams (H2D, D2H, two compute) were
 * found to sit on hardware queues of their own (4 unless the process has fewer than four hardware queues), *created <-
 * how many streams it created to find them; both 0 before the first call that needs streams.  No counterpart in the
 * reference. */
int PARALiA_stream_queues(int* independent, int* created);
/* directory holding Processed/ lookup tables and link models (DEPLOYDB, CMakeLists.txt:376) */
int PARALiA_set_db_dir(const char* dir);

/* cols runs of width_bytes, run c at dst + c*dst_pitch <- src + c*src_pitch, split over `threads` host threads.  The
 * gather / scatter step of the pinned bounce buffers that stand in for the reference's pinning of pageable operands
 * (prepareAsync, dgemm.cpp:413-416). */
int PARALiA_host_copy2d(void* dst, long dst_pitch, const void* src, long src_pitch, long width_bytes, long cols, int threads);

/* ---- driver helper surface (CoCoMalloc / CoCoFree / CoCoVecInit / Dtest_equality, dgemm_runner.cpp:55-99) ---- */
int PARALiA_malloc(void** ptr, long long bytes, int loc);
int PARALiA_free(void* ptr, int loc);
int PARALiA_vec_init_f64(double* p, long long n, int seed, int loc);
int PARALiA_vec_init_f32(float* p, long long n, int seed, int loc);
int PARALiA_test_equality_f64(double* ref, double* x, long long n);
int PARALiA_test_equality_f32(float* ref, float* x, long long n);

/* ---- host-logic probes: no GPU call is made by any of these ---- */
/* ATC::optimize_tile / get_T_slowdowns for one unit (Autotuner.cpp:571-655); returns T */
long PARALiA_heuristic_tile(long D1, long D2, long D3, double slowdowns[6]);
int PARALiA_T_slowdowns(long D1, long D2, long D3, long T, double slowdowns[6]);
/* Modeler::predict (ModelLvl3.cpp:287-551, ModelLvl1.cpp:262): mode = ModelType value, loc[i] = -1 host / 0 device */
double PARALiA_model_predict(const char* db_dir, const char* func, int mode, long D1, long D2, long D3, char ta, char tb,
                             const int loc[3], long T);
/* ATC::autotune_problem (Autotuner.cpp:279) without touching the GPU */
int PARALiA_autotune(const char* db_dir, const char* func, long D1, long D2, long D3, char ta, char tb, const int loc[3],
                     int beta_zero, long T_in, long long pool_budget_bytes, pl_atc_info* info);
/* static GEMM plan (CreateSubkernelsDgemm + request_data + run_operation, dgemm.cpp:123-205, Subkernel.cpp:90-247) */
#define PL_PLAN_MAX_WAITS 12
#define PL_PLAN_ROW (14 + PL_PLAN_MAX_WAITS)
long PARALiA_gemm_plan(long M, long N, long K, long T, int a_remote, int b_remote, int c_remote, int beta_zero, int elem,
                       int exec_queues, long pool_blocks, int order_id, int* rows, long max_rows, long stats[6]);
/* makespan of one order (order_id >= 0) or of the best candidate (< 0) on the simulated H2D / compute / D2H pipeline;
   h2d_sl, d2h_sl >= 1: how much slower a copy runs while the opposite direction is busy (the link model's sl,
   CoModel.cpp:143-162) */
double PARALiA_gemm_plan_simulate(long M, long N, long K, long T, int a_remote, int b_remote, int c_remote, int beta_zero,
                                  int elem, int exec_queues, long pool_blocks, int order_id, double t_exec, double h2d_ti,
                                  double h2d_tb, double d2h_ti, double d2h_tb, double t_reduce, double h2d_sl, double d2h_sl, int* picked,
                                  double busy[3]);

#ifdef __cplusplus
}
#endif
#endif /* PARALIA_HIP_H */
