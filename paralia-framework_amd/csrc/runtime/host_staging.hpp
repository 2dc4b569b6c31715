// Staging of pageable (not pinned) host operands.
//
// The reference pins whatever host memory it is given (cudaHostRegister in the operands' prepareAsync,
// Library_scheduler/src/Functions/dgemm.cpp:413-416) so that every tile copy runs at the pinned rate.  Registering
// existing memory is not available to this runtime, and a strided 2-D copy straight from pageable memory runs at
// about 1 GB/s.  So tiles of pageable operands travel through a small ring of pinned bounce buffers: worker threads
// gather a tile (strided rows -> dense) into a pinned slot, one contiguous asynchronous copy moves it to the device,
// and the reverse for results.  Pure host logic apart from the C ABI calls; no HIP header.
#ifndef PARALIA_HOST_STAGING_HPP
#define PARALIA_HOST_STAGING_HPP

#include <atomic>
#include <condition_variable>
#include <cstddef>
#include <deque>
#include <exception>
#include <mutex>
#include <thread>
#include <vector>

namespace paralia {

// Fixed pool of worker threads running one strided 2-D memcpy at a time, split by columns.
class CopyThreads {
 public:
  explicit CopyThreads(int nthreads);
  ~CopyThreads();
  CopyThreads(const CopyThreads&) = delete;
  CopyThreads& operator=(const CopyThreads&) = delete;
  // cols runs of width_bytes each, run c at dst + c*dst_pitch  <-  src + c*src_pitch.  Returns when all are copied.
  void copy2d(void* dst, size_t dst_pitch, const void* src, size_t src_pitch, size_t width_bytes, long cols);
  int threads() const { return (int)workers_.size() + 1; }

 private:
  struct Job {
    char* dst = nullptr;
    const char* src = nullptr;
    size_t dst_pitch = 0, src_pitch = 0, width = 0;
    long cols = 0, chunk = 1;
  };
  void worker();
  void run_chunks();
  std::vector<std::thread> workers_;
  std::mutex mu_;
  std::condition_variable cv_start_, cv_done_;
  Job job_;
  std::atomic<long> next_{0};
  long generation_ = 0;
  int running_ = 0;
  bool stop_ = false;
};

// Ring of pinned slots for tiles on their way to the device, and a second ring for tiles coming back.
class HostStager {
 public:
  static constexpr int MAX_DEFERRED_WAITS = 12;   // events a deferred write-back may wait for (the plan's MAX_WAITS)
  HostStager() = default;
  ~HostStager();
  HostStager(const HostStager&) = delete;
  HostStager& operator=(const HostStager&) = delete;
  // dst (device, leading dimension ld_dst; 0 = dense, i.e. rows)  <-  src (pageable host, leading dimension ld_src), on
  // `stream`.
  void fetch(void* dst, const void* src, long ld_src, long rows, long cols, int elem, void* stream, long ld_dst = 0);
  // dst (pageable host, leading dimension ld_dst)  <-  src (device, leading dimension ld_src; 0 = dense, i.e. rows) on
  // `stream`; the host-side scatter happens when the slot is needed again or in finish().
  void write_back(void* dst, long ld_dst, const void* src, long rows, long cols, int elem, void* stream, long ld_src = 0);
  // The same, handed to a background thread: it makes `stream` wait for the n_after events (the tile's last kernels),
  // copies the tile into a pinned slot as slots come free, waits for the copy and scatters it.  The caller does not
  // wait for a slot, so the thread that enqueues a plan keeps going when many C tiles complete close together (with
  // the blocking call it fell back to the pace of the write-backs there, the kernels behind them were launched late and
  // a call with a pageable C took 148 ms instead of 125 ms at 16384^3).  Nothing else may use `stream` or the slots
  // until finish(); the device memory at src must stay untouched until then.
  void write_back_deferred(void* dst, long ld_dst, const void* src, long rows, long cols, int elem, void* stream,
                           void* const* after, int n_after, long ld_src = 0);
  // Completes every pending scatter, deferred ones included (those need not have been waited for: their copies are
  // synchronised here); rethrows what the background thread ran into.  The blocking ones need the streams synchronised.
  void finish();
  // Forgets pending scatters without performing them: after a failed call their destinations may no longer be valid.
  void abandon();
  // Sizes the slots for tiles of up to tile_bytes (waits for tiles in flight and reallocates when they must grow).
  void reserve(long long tile_bytes);
  void release();

 private:
  static constexpr int SLOTS = 4;
  struct Pending { void* dst = nullptr; long ld = 0, rows = 0, cols = 0; int elem = 0; bool active = false; };
  void flush(int slot);
  CopyThreads* threads();
  char* in_[SLOTS] = {nullptr};
  char* out_[SLOTS] = {nullptr};
  void* in_ev_[SLOTS] = {nullptr};
  void* out_ev_[SLOTS] = {nullptr};
  bool in_used_[SLOTS] = {false};
  Pending pending_[SLOTS];
  long long slot_bytes_ = 0;
  long in_next_ = 0, out_next_ = 0;
  CopyThreads* pool_ = nullptr;
  // deferred write-backs: requests in call order; the background thread owns the out_ slots while any are open
  struct Request {
    void* dst; long ld; const void* src; long rows, cols; int elem; void* stream;
    void* after[MAX_DEFERRED_WAITS]; int n_after; long ld_src;
  };
  int device_ = 0;             // device that was current when the background thread was started; the thread makes it its own
  void deferred_loop();
  std::thread deferred_;
  CopyThreads* deferred_pool_ = nullptr;
  std::mutex dmu_;
  std::condition_variable dcv_;
  std::deque<Request> requests_;
  long open_ = 0;              // requests accepted and not yet scattered (or dropped)
  bool stop_ = false, dropping_ = false;
  std::exception_ptr error_;
};

// Completes the staged write-backs on the normal path, drops them when the call unwinds with an error.
struct StagerScope {
  HostStager& stager;
  bool finished = false;
  explicit StagerScope(HostStager& s) : stager(s) {}
  void finish() { stager.finish(); finished = true; }
  ~StagerScope() { if (!finished) stager.abandon(); }
};

}  // namespace paralia
#endif
