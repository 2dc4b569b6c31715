// Thin C-ABI over the HIP runtime: the only place (besides the kernel files) that includes HIP headers.
// It stands where the reference's un-vendored backend wrappers stand (CoCoMalloc / CoCoFree / CoCoMemcpy /
// CoCoMemcpy2DAsync / CommandQueue / Event / CoCoGetPtrLoc / CoCoPeLiaDevGetMemInfo / CoCoSyncCheckErr, used
// from Library_scheduler/src/Subkernel.cpp:249-306, Subkernel_backup.cpp:526-529,1229-1232 and
// Benchmarking/CuCuBLAS/src/PARALia/dgemm_runner.cpp:55-77).  Every call returns 0 on success and a non-zero
// code otherwise; pl_last_error() gives the HIP error text of the most recent failure on the calling thread.
#include <hip/hip_runtime.h>
#include <stdlib.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "paralia_hip.h"
#include "backend/pl_internal.h"

namespace {
thread_local char g_err[256] = "no error";

int fail(hipError_t e, const char* what) {
  snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
  return PL_ERR_HIP;
}
#define PL_TRY(call)                      \
  do {                                    \
    hipError_t e_ = (call);               \
    if (e_ != hipSuccess) return fail(e_, #call); \
  } while (0)

// One wave that stays on the device for `ticks` of the constant-rate wall clock; the loop count bounds it whatever
// the clock reads.
__global__ void hold_kernel(long long ticks) {
  const long long t0 = (long long)wall_clock64();
  for (int i = 0; i < 4096; ++i) {
    if ((long long)wall_clock64() - t0 >= ticks) break;
    __builtin_amdgcn_s_sleep(64);
  }
}
__global__ void noop_kernel() {}
}  // namespace

int pl_fail_hip(int hip_error, const char* what) { return fail((hipError_t)hip_error, what); }
int pl_fail_msg(int code, const char* message) {
  snprintf(g_err, sizeof(g_err), "%s", message);
  return code;
}

extern "C" {

const char* pl_last_error(void) { return g_err; }

int pl_device_count(int* count) {
  int c = 0;
  hipError_t e = hipGetDeviceCount(&c);
  if (e != hipSuccess) { *count = 0; return fail(e, "hipGetDeviceCount"); }
  *count = c;
  return 0;
}
int pl_set_device(int dev) {
  PL_TRY(hipSetDevice(dev));
  return pl_noalloc_setup_current_device();
}
int pl_get_device(int* dev) { PL_TRY(hipGetDevice(dev)); return 0; }
int pl_device_sync(void) { PL_TRY(hipDeviceSynchronize()); return 0; }

int pl_device_name(int dev, char* buf, int len) {
  hipDeviceProp_t p;
  PL_TRY(hipGetDeviceProperties(&p, dev));
  snprintf(buf, len, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
  return 0;
}

int pl_mem_info(long long* free_bytes, long long* total_bytes) {
  size_t f = 0, t = 0;
  PL_TRY(hipMemGetInfo(&f, &t));
  *free_bytes = (long long)f;
  *total_bytes = (long long)t;
  return 0;
}

int pl_malloc_device(void** ptr, long long bytes) {
  *ptr = nullptr;
  if (bytes <= 0) return 0;
  PL_TRY(hipMalloc(ptr, (size_t)bytes));
  return 0;
}
int pl_free_device(void* ptr) {
  if (ptr) PL_TRY(hipFree(ptr));
  return 0;
}
// Page-locked host memory.  Existing allocations are never registered after the fact (hipHostRegister):
// pinned operands have to be born pinned.
int pl_malloc_pinned(void** ptr, long long bytes) {
  *ptr = nullptr;
  if (bytes <= 0) return 0;
  PL_TRY(hipHostMalloc(ptr, (size_t)bytes, hipHostMallocDefault));
  return 0;
}
int pl_free_pinned(void* ptr) {
  if (ptr) PL_TRY(hipHostFree(ptr));
  return 0;
}

// Location code of a pointer, in the reference's convention (dgemm_runner.cpp:55-57, testing.cpp:296-321):
// >= 0 device id, -1 page-locked host memory, -2 pageable host memory.
int pl_ptr_location(const void* ptr, int* loc) {
  hipPointerAttribute_t attr;
  memset(&attr, 0, sizeof(attr));
  hipError_t e = hipPointerGetAttributes(&attr, ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // unknown pointers are ordinary pageable memory, not an error
    *loc = PL_LOC_HOST_PAGEABLE;
    return 0;
  }
  switch (attr.type) {
    case hipMemoryTypeDevice: *loc = attr.device; break;
    case hipMemoryTypeHost: *loc = PL_LOC_HOST_PINNED; break;
    case hipMemoryTypeManaged: *loc = attr.device; break;
    default: *loc = PL_LOC_HOST_PAGEABLE; break;
  }
  return 0;
}

int pl_stream_create(void** stream) {
  hipStream_t s;
  PL_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = (void*)s;
  return pl_noalloc_setup_current_device();   // so that pl_dgemv_noalloc on this stream finds its scratch resolved
}
int pl_stream_destroy(void* stream) { PL_TRY(hipStreamDestroy((hipStream_t)stream)); return 0; }
int pl_stream_sync(void* stream) { PL_TRY(hipStreamSynchronize((hipStream_t)stream)); return 0; }
int pl_stream_query(void* stream, int* done) {
  hipError_t e = hipStreamQuery((hipStream_t)stream);
  if (e == hipSuccess) { *done = 1; return 0; }
  if (e == hipErrorNotReady) { (void)hipGetLastError(); *done = 0; return 0; }
  return fail(e, "hipStreamQuery");
}

int pl_event_create(void** event, int timing) {
  hipEvent_t ev;
  PL_TRY(hipEventCreateWithFlags(&ev, timing ? hipEventDefault : hipEventDisableTiming));
  *event = (void*)ev;
  return 0;
}
int pl_event_destroy(void* event) { PL_TRY(hipEventDestroy((hipEvent_t)event)); return 0; }
int pl_event_record(void* event, void* stream) { PL_TRY(hipEventRecord((hipEvent_t)event, (hipStream_t)stream)); return 0; }
int pl_stream_wait_event(void* stream, void* event) {
  PL_TRY(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0));
  return 0;
}
int pl_event_sync(void* event) { PL_TRY(hipEventSynchronize((hipEvent_t)event)); return 0; }
int pl_event_query(void* event, int* done) {
  hipError_t e = hipEventQuery((hipEvent_t)event);
  if (e == hipSuccess) { *done = 1; return 0; }
  if (e == hipErrorNotReady) { (void)hipGetLastError(); *done = 0; return 0; }
  return fail(e, "hipEventQuery");
}
int pl_event_elapsed_ms(void* start, void* stop, float* ms) {
  PL_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}

// Does `candidate` run in order with one of others[0 .. n-1]?  HIP places the streams of a process on a few hardware
// queues (GPU_MAX_HW_QUEUES, 4 by default): a new stream goes to the queue with the fewest streams, ties broken in an
// order that is not creation order, so which streams end up together cannot be told from how many were created.
// Streams on one queue execute strictly one after the other, as if they were one stream.  The test is functional: a
// one-wave kernel that stays resident for half a millisecond goes to each of the others, an empty kernel to the
// candidate; if the empty kernel has completed while all the holders are still running, the candidate's queue is its
// own.  A candidate that shares a queue cannot pass (its kernel is behind a holder); one that does not share can only
// fail when the calling thread loses the processor for the rest of the half millisecond, and the caller then simply
// tries another stream.
int pl_stream_shares_queue(void* candidate, void* const* others, int n, int* shares) {
  *shares = 0;
  if (n <= 0) return 0;
  if (n > PL_MAX_PROBE_STREAMS || !candidate) return pl_fail_msg(PL_ERR_ARG, "pl_stream_shares_queue: 1 to 8 streams to compare with");
  int dev = 0, khz = 0;
  PL_TRY(hipGetDevice(&dev));
  PL_TRY(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
  if (khz <= 0) khz = 100000;
  const long long hold_ticks = (long long)khz / 2;  // 0.5 ms of the constant-rate clock
  static bool warmed = false;  // the first launch of a kernel loads its code: not inside the measured window
  if (!warmed) {
    hipLaunchKernelGGL(hold_kernel, dim3(1), dim3(64), 0, (hipStream_t)candidate, 0LL);
    hipLaunchKernelGGL(noop_kernel, dim3(1), dim3(64), 0, (hipStream_t)candidate);
    PL_TRY(hipGetLastError());
    PL_TRY(hipStreamSynchronize((hipStream_t)candidate));
    warmed = true;
  }
  hipEvent_t held[PL_MAX_PROBE_STREAMS], done;
  for (int i = 0; i < n; ++i) PL_TRY(hipEventCreateWithFlags(&held[i], hipEventDisableTiming));
  PL_TRY(hipEventCreateWithFlags(&done, hipEventDisableTiming));
  for (int i = 0; i < n; ++i) {
    hipLaunchKernelGGL(hold_kernel, dim3(1), dim3(64), 0, (hipStream_t)others[i], hold_ticks);
    PL_TRY(hipEventRecord(held[i], (hipStream_t)others[i]));
  }
  hipLaunchKernelGGL(noop_kernel, dim3(1), dim3(64), 0, (hipStream_t)candidate);
  PL_TRY(hipGetLastError());
  PL_TRY(hipEventRecord(done, (hipStream_t)candidate));
  PL_TRY(hipEventSynchronize(done));
  for (int i = 0; i < n; ++i) {
    hipError_t e = hipEventQuery(held[i]);
    if (e == hipSuccess) *shares = 1;                       // a holder had finished before the candidate's kernel ran
    else if (e == hipErrorNotReady) (void)hipGetLastError();
    else return fail(e, "hipEventQuery");
  }
  for (int i = 0; i < n; ++i) {
    PL_TRY(hipEventSynchronize(held[i]));
    PL_TRY(hipEventDestroy(held[i]));
  }
  PL_TRY(hipEventDestroy(done));
  return 0;
}

// rows x cols elements of elem_size bytes, column-major on both sides: "rows" is the contiguous extent,
// ld_* the distance between columns in elements (the argument order of CoCoMemcpy2DAsync,
// Subkernel_backup.cpp:526-529).  Direction is inferred from the pointers.
int pl_copy2d_async(void* dst, long ld_dst, const void* src, long ld_src, long rows, long cols, int elem_size,
                    void* stream) {
  if (rows <= 0 || cols <= 0) return 0;
  if (ld_dst < rows || ld_src < rows) { snprintf(g_err, sizeof(g_err), "pl_copy2d_async: ld < rows"); return PL_ERR_ARG; }
  const size_t width = (size_t)rows * elem_size;
  // Always the 2-D call, also for a dense view (ld == rows on both sides): a plain 1-D copy between pinned host
  // memory and the device takes another path through the runtime, and on a stream that otherwise carries 2-D copies
  // it was seen to start only after the copy running on the opposite-direction stream had finished (ten such tiles
  // cost dgemm 40000 x 40000 x 2048 with host operands 26 ms of 300).
  PL_TRY(hipMemcpy2DAsync(dst, (size_t)ld_dst * elem_size, src, (size_t)ld_src * elem_size, width, (size_t)cols,
                          hipMemcpyDefault, (hipStream_t)stream));
  return 0;
}

int pl_copy_async(void* dst, const void* src, long long bytes, void* stream) {
  if (bytes <= 0) return 0;
  PL_TRY(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDefault, (hipStream_t)stream));
  return 0;
}

int pl_copy(void* dst, const void* src, long long bytes) {
  if (bytes <= 0) return 0;
  PL_TRY(hipMemcpy(dst, src, (size_t)bytes, hipMemcpyDefault));
  return 0;
}

int pl_memset_async(void* dst, int value, long long bytes, void* stream) {
  if (bytes <= 0) return 0;
  PL_TRY(hipMemsetAsync(dst, value, (size_t)bytes, (hipStream_t)stream));
  return 0;
}

// Deferred errors from asynchronous work surface here (CoCoSyncCheckErr, dgemm.cpp:597).
int pl_sync_check(void) {
  PL_TRY(hipDeviceSynchronize());
  PL_TRY(hipGetLastError());
  return 0;
}

}  // extern "C"
