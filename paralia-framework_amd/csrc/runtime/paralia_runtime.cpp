// PARALiA routines on one MI355X: argument checks, operand location detection, problem-metadata cache, device
// block pool, stream/event inventory and the executor that turns a static GEMM plan into HIP stream work.
//
// Reference counterparts: Library_scheduler/src/Functions/dgemm.cpp:318-705 (PARALiADgemm: metadata cache
// :342-368, decomposition :409-440, cache sizing :23-121, fire loop :512-546, sync :596-597, reuse :627-649),
// sgemm.cpp:296, daxpy.cpp:200, ddot.cpp:201, Subkernel.cpp:249-306 (queue inventory), :488 (cache free).
// All device work goes through the C ABI in paralia_hip.h; this file includes no HIP header.
#include <algorithm>
#include <array>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "PARALiA.hpp"
#include "backend_wrappers.hpp"
#include "gemm_plan.hpp"
#include "host_staging.hpp"
#include "paralia_hip.h"

namespace paralia {

static void chk(int rc, const char* what) {
  if (rc != 0) throw paralia_error(rc, std::string(what) + " failed: " + (rc == PL_ERR_HIP ? pl_last_error() : "invalid argument"));
}

// ------------------------------------------------------------------------------------------ block pool
// Equal-size device blocks carved from one allocation that is kept between calls (the reference's Buffer with
// BUFFER_REUSE_ENABLE, dgemm.cpp:95-117).  The allocation is only replaced when a call needs more bytes than it
// holds: a call with another block size re-partitions the memory it already has.  Freeing and re-allocating tens of
// gigabytes between calls is not free on this device: for a few seconds after such a hipFree the host link runs
// about 4 % slower (the link-bound 40000 x 40000 x 2048 product: 284 ms instead of 273 ms for its first ten calls).
struct DevicePool {
  void* base = nullptr;
  long long capacity = 0;  // bytes held
  long long block_sz = 0;
  long blocks = 0;
  long long bytes() const { return capacity; }
  void* at(long b) const { return (char*)base + block_sz * b; }
  // limit > 0: the caller's cache_limit; memory kept from an earlier, larger call is given back rather than held
  void ensure(long need_blocks, long long need_block_sz, long long limit = 0) {
    const long long need = need_block_sz * need_blocks;
    if (!base || capacity < need || (limit > 0 && capacity > std::max(limit, need))) {
      release();
      chk(pl_malloc_device(&base, need), "device block pool allocation");
      capacity = need;
    }
    block_sz = need_block_sz;
    blocks = need_block_sz > 0 ? (long)(capacity / need_block_sz) : 0;
  }
  void release() {
    if (base) chk(pl_free_device(base), "device block pool free");
    base = nullptr;
    capacity = block_sz = 0;
    blocks = 0;
  }
};

// ------------------------------------------------------------------------------- streams, events, scratch
// One H2D stream, one D2H stream, up to MAX_BACKEND_L compute streams (Subkernel.cpp:249-306 keeps
// recv/wb queues per link and 8 exec queues per device); created once and reused (BACKEND_RES_REUSE_ENABLE).
struct Resources {
  void* h2d = nullptr;
  void* d2h = nullptr;
  void* exec[MAX_EXEC_QUEUES] = {nullptr};
  int nexec = 0;
  std::vector<void*> events;
  std::unique_ptr<HostStager> stager_;  // pinned bounce buffers for pageable host operands, created on first use
  HostStager& stager() { if (!stager_) stager_.reset(new HostStager()); return *stager_; }
  double* dot_ws = nullptr;      // ddot partials
  double* dot_result = nullptr;  // device scalar
  double* dot_host = nullptr;    // pinned scalar
  // HIP places the streams of a process on GPU_MAX_HW_QUEUES hardware queues (4 by default), and streams that share
  // a queue run strictly one after the other.  A new stream goes to the queue with the fewest streams, ties broken in
  // a fixed order that is not creation order (seven streams created back to back land on queues 1 2 3 4 4 3 2), and
  // streams the application created earlier shift everything.  What sharing costs the streamed 16384^3 fp64 GEMM:
  // both compute streams on one queue 138 ms (no two tile kernels ever overlap), each copy stream sharing with a
  // compute stream 150 ms (a tile kernel waits for every fetch enqueued before it), both copy streams on one queue
  // 160 ms, four queues of their own 122 ms.  So the four busy streams are not taken as they come: streams are
  // created one at a time and each is kept only if a functional test (pl_stream_shares_queue) shows that it does not
  // run in order with the ones already kept; the others are destroyed again.  A few milliseconds, once.
  std::vector<void*> owned;   // every stream this inventory created and still holds
  int independent = 0;        // how many of (h2d, d2h, exec0, exec1) sit on a hardware queue of their own
  int created = 0;            // streams created while looking for them
  void* new_stream() {
    void* s = nullptr;
    chk(pl_stream_create(&s), "stream create");
    ++created;
    return s;
  }
  bool shares_queue(void* cand, const std::vector<void*>& with) {
    if (with.empty()) return false;
    int shares = 0;
    chk(pl_stream_shares_queue(cand, with.data(), (int)with.size(), &shares), "stream placement test");
    if (shares) chk(pl_stream_shares_queue(cand, with.data(), (int)with.size(), &shares), "stream placement test");  // confirm
    return shares != 0;
  }
  void ensure_streams(int nq) {
    if (!h2d) {
      std::vector<void*> kept, sharing;
      // at most 4 hardware queues are expected to matter; 16 candidates cover an application that already holds a
      // dozen streams on them
      for (int tries = 0; kept.size() < 4 && tries < 16; ++tries) {
        void* s = new_stream();
        (shares_queue(s, kept) ? sharing : kept).push_back(s);
      }
      independent = (int)kept.size();
      // Fewer than four queues to be had (GPU_MAX_HW_QUEUES below 4): the copy streams keep queues of their own first,
      // and a compute stream rather shares with the other compute stream than with a copy stream.
      while (kept.size() < 4) {
        const std::vector<void*> copies(kept.begin(), kept.begin() + std::min<size_t>(2, kept.size()));
        size_t pick = sharing.size();
        for (size_t i = 0; i < sharing.size() && pick == sharing.size(); ++i)
          if (kept.size() >= 2 && !shares_queue(sharing[i], copies)) pick = i;
        if (pick == sharing.size()) {
          if (sharing.empty()) sharing.push_back(new_stream());
          pick = 0;
        }
        kept.push_back(sharing[pick]);
        sharing.erase(sharing.begin() + pick);
      }
      for (void* s : sharing) chk(pl_stream_destroy(s), "stream destroy");
      owned = kept;
      h2d = kept[0];
      d2h = kept[1];
      exec[0] = kept[2];
      exec[1] = kept[3];
      nexec = 2;
    }
    // further compute streams (PARALIA_EXEC_QUEUES above 2) have to share a queue with somebody: not with a copy stream
    for (; nexec < nq; ++nexec) {
      const std::vector<void*> copies = {h2d, d2h};
      std::vector<void*> sharing;
      void* pick = nullptr;
      for (int tries = 0; !pick && tries < 8; ++tries) {
        void* s = new_stream();
        if (shares_queue(s, copies)) sharing.push_back(s);
        else pick = s;
      }
      if (!pick) { pick = sharing.back(); sharing.pop_back(); }
      for (void* s : sharing) chk(pl_stream_destroy(s), "stream destroy");
      owned.push_back(pick);
      exec[nexec] = pick;
    }
  }
  void ensure_events(size_t n) {
    while (events.size() < n) {
      void* e = nullptr;
      chk(pl_event_create(&e, 0), "event create");
      events.push_back(e);
    }
  }
  void ensure_dot() {
    if (dot_ws) return;
    void* p = nullptr;
    chk(pl_malloc_device(&p, (pl_ddot_workspace_doubles() + 8) * (long long)sizeof(double)), "ddot workspace");
    dot_ws = (double*)p;
    dot_result = dot_ws + pl_ddot_workspace_doubles();
    chk(pl_malloc_pinned(&p, 64), "ddot host scalar");
    dot_host = (double*)p;
  }
  // growable device scratch of dgemv: staged copies of host-resident x and y, and the kernels' partial sums
  struct Scratch {
    void* p = nullptr;
    long long cap = 0;
    void* ensure(long long bytes) {
      if (bytes <= cap) return p;
      if (p) chk(pl_free_device(p), "scratch free");
      p = nullptr; cap = 0;
      chk(pl_malloc_device(&p, bytes), "scratch allocation");
      cap = bytes;
      return p;
    }
    // The same for memory the caller can do without: nullptr, and nothing attempted, unless the device has twice the
    // room to spare (a caller whose matrices fill the device keeps what is left of it).
    void* ensure_if_room(long long bytes) {
      if (bytes <= cap) return p;
      long long free_b = 0, total_b = 0;
      chk(pl_mem_info(&free_b, &total_b), "mem info");
      if (2 * (bytes - cap) > free_b) return nullptr;
      return ensure(bytes);
    }
    void release() { if (p) pl_free_device(p); p = nullptr; cap = 0; }
  } gemv_x, gemv_y, gemv_ws;
  // split-K workspaces of the tile GEMM, one per exec stream (launches on different streams may overlap)
  Scratch gemm_ws[MAX_EXEC_QUEUES];
  // 16-byte aligned copies of device-resident GEMM operands whose own address or leading dimension is not (A, B)
  Scratch gemm_realigned[2];
  void* stream(int id) const { return id == STREAM_H2D ? h2d : id == STREAM_D2H ? d2h : exec[id - STREAM_EXEC0]; }
  void sync_all() {
    if (h2d) chk(pl_stream_sync(h2d), "stream sync");
    for (int q = 0; q < nexec; ++q) chk(pl_stream_sync(exec[q]), "stream sync");
    if (d2h) chk(pl_stream_sync(d2h), "stream sync");
  }
  // Best effort, for error paths: whatever was enqueued before the failure must not outlive the call (it reads
  // and writes the caller's operands and the pool blocks).
  void drain() noexcept {
    if (h2d) pl_stream_sync(h2d);
    for (int q = 0; q < nexec; ++q) if (exec[q]) pl_stream_sync(exec[q]);
    if (d2h) pl_stream_sync(d2h);
  }
  // Per-command timeline of a GEMM call (the reference's STEST / TTEST builds print one per subkernel,
  // Subkernel.cpp:498, dgemm.cpp:612-615): when switched on, every command of the plan is bracketed by two timing
  // events on its stream and the rows of the last call are kept for PARALiA_trace_read.
  bool trace_on = false;
  std::vector<void*> timing_events;
  struct TraceRow { int kind, mi, ni, ki, stream; double t0_ms, t1_ms; };
  std::vector<TraceRow> trace;
  void ensure_timing_events(size_t n) {
    while (timing_events.size() < n) {
      void* e = nullptr;
      chk(pl_event_create(&e, 1), "event create");
      timing_events.push_back(e);
    }
  }
  // The counterpart of CoCoPeLiaFreeResources (Subkernel.cpp:330): streams, events, workspaces and bounce buffers
  // go; the next call creates them again (and places its streams anew).
  void destroy() {
    drain();
    for (void* s : owned) pl_stream_destroy(s);
    for (void* e : events) pl_event_destroy(e);
    for (void* e : timing_events) pl_event_destroy(e);
    if (dot_ws) pl_free_device(dot_ws);
    if (dot_host) pl_free_pinned(dot_host);
    gemv_x.release(); gemv_y.release(); gemv_ws.release();
    for (Scratch& w : gemm_ws) w.release();
    for (Scratch& w : gemm_realigned) w.release();
    stager_.reset();
    const bool keep_trace = trace_on;
    *this = Resources();
    trace_on = keep_trace;
  }
};
// Armed while a routine enqueues work; if the routine leaves by an exception the streams are drained first.
struct DrainOnError {
  Resources& res;
  bool armed = true;
  explicit DrainOnError(Resources& r) : res(r) {}
  ~DrainOnError() { if (armed) res.drain(); }
};

// ------------------------------------------------------------------------------------ metadata cache
struct PMDKey {
  std::string routine;
  char ta = 'N', tb = 'N';
  long D1 = 0, D2 = 0, D3 = 0;
  int loc[3] = {0, 0, 0};
  bool beta_zero = false;
  long predef_T = -1;
  long long cache_limit = 0;
  bool operator==(const PMDKey& o) const {
    return routine == o.routine && ta == o.ta && tb == o.tb && D1 == o.D1 && D2 == o.D2 && D3 == o.D3 && loc[0] == o.loc[0] &&
           loc[1] == o.loc[1] && loc[2] == o.loc[2] && beta_zero == o.beta_zero && predef_T == o.predef_T &&
           cache_limit == o.cache_limit;
  }
};
struct PMDEntry {
  PMDKey key;
  std::unique_ptr<ATC> atc;
  GemmPlan plan;
  long calls = 0;  // calls served from this entry
};

struct Runtime {
  std::mutex mu;  // serialises calls: the routines are not re-entrant (file-scope state in the reference too)
  DevicePool pool;
  Resources res;
  std::vector<std::unique_ptr<PMDEntry>> pmd;  // at most PROBLEM_MD_CACHE entries, oldest dropped first
  long pmd_hits = 0, pmd_misses = 0;
  // Host-side phases of the most recent GEMM call, in seconds (the reference's TEST build prints the same split:
  // dgemm.cpp:330-333 autotune, :430-445 decomposition and tile maps, :497-511 cache allocation and queues, :598-604
  // execution).  autotune and plan are 0 on a call served from the metadata cache.
  struct Phases { double autotune = 0, plan = 0, pool = 0, streams = 0, execute = 0, total = 0; } phases;
};
static Runtime& rt() {
  // never destroyed: at process exit the HIP runtime may already be gone, and freeing pinned buffers, events or
  // streams from a static destructor would call into it
  static Runtime* r = new Runtime();
  return *r;
}

static int host_or_dev(int loc) { return loc >= 0 ? 0 : -1; }  // the scheduler routes by "on device 0" vs "host"

static long long pool_budget(long long cache_limit, long long prev_pool_bytes) {
  long long free_b = 0, total_b = 0;
  chk(pl_mem_info(&free_b, &total_b), "mem info");
  // dgemm.cpp:73-78: leave (100 - PROBLEM_GPU_PERCENTAGE)% of the device alone; the old pool is reusable
  long long budget = free_b - (long long)(total_b * (1 - PROBLEM_GPU_PERCENTAGE / 100.0)) + prev_pool_bytes;
  if (cache_limit > 0) budget = std::min(budget, cache_limit);
  return std::max(budget, 0LL);
}

static ATC_p atc_copy(ATC* src) {
  ATC_p out = new ATC();
  out->mimic_ATC(src);
  return out;
}

// ------------------------------------------------------------------------------------------- GEMM
template <typename T> struct GemmFns;
template <> struct GemmFns<double> {
  static constexpr const char* name = "Dgemm";
  static int tile(char ta, char tb, long M, long N, long K, double al, const double* A, long lda, const double* B, long ldb,
                  double be, double* C, long ldc, void* ws, long ws_bytes, void* s) {
    return pl_dgemm_tile_ws(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ws, ws_bytes, s);
  }
  static int tile_padded(char ta, char tb, long M, long N, long K, double al, const double* A, long lda, const double* B, long ldb,
                         double be, double* C, long ldc, void* ws, long ws_bytes, int splits, long m_read, long n_read, void* s) {
    return pl_dgemm_tile_padded(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ws, ws_bytes, splits, m_read, n_read, s);
  }
  static int tile_split(char ta, char tb, long M, long N, long K, double al, const double* A, long lda, const double* B, long ldb,
                        double be, double* C, long ldc, void* ws, long ws_bytes, int splits, void* s) {
    return pl_dgemm_tile_split(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ws, ws_bytes, splits, s);
  }
  static int geadd(long M, long N, double be, const double* s, long lds, const double* a, long lda, double* o, long ldo, void* st) {
    return pl_dgeadd_tile(M, N, be, s, lds, a, lda, o, ldo, st);
  }
};
template <> struct GemmFns<float> {
  static constexpr const char* name = "Sgemm";
  static int tile(char ta, char tb, long M, long N, long K, float al, const float* A, long lda, const float* B, long ldb,
                  float be, float* C, long ldc, void* ws, long ws_bytes, void* s) {
    return pl_sgemm_tile_ws(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ws, ws_bytes, s);
  }
  static int tile_padded(char ta, char tb, long M, long N, long K, float al, const float* A, long lda, const float* B, long ldb,
                         float be, float* C, long ldc, void* ws, long ws_bytes, int splits, long m_read, long n_read, void* s) {
    return pl_sgemm_tile_padded(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ws, ws_bytes, splits, m_read, n_read, s);
  }
  static int tile_split(char ta, char tb, long M, long N, long K, float al, const float* A, long lda, const float* B, long ldb,
                        float be, float* C, long ldc, void* ws, long ws_bytes, int splits, void* s) {
    return pl_sgemm_tile_split(ta, tb, M, N, K, al, A, lda, B, ldb, be, C, ldc, ws, ws_bytes, splits, s);
  }
  static int geadd(long M, long N, float be, const float* s, long lds, const float* a, long lda, float* o, long ldo, void* st) {
    return pl_sgeadd_tile(M, N, be, s, lds, a, lda, o, ldo, st);
  }
};

template <typename T>
static void execute_gemm_plan(Runtime& R, const GemmPlan& plan, char ta, char tb, T alpha, const T* A, long lda, const T* B,
                              long ldb, T beta, T* C, long ldc, const bool pageable[3]) {
  const GemmProblem& p = plan.p;
  const bool at = (ta == 'T'), bt = (tb == 'T');
  const long Tt = p.T;
  R.res.ensure_streams(std::max(1, std::min(p.exec_queues, MAX_EXEC_QUEUES)));
  size_t nsig = 0;
  for (const Cmd& c : plan.cmds) nsig += c.signals ? 1 : 0;
  R.res.ensure_events(nsig);
  std::vector<void*> ev(plan.cmds.size(), nullptr);
  size_t next_ev = 0;
  // tiles of pageable operands go through pinned bounce buffers (a strided copy straight from pageable memory
  // runs at about 1 GB/s)
  HostStager& stager = R.res.stager();
  if (pageable[0] || pageable[1] || pageable[2]) stager.reserve((long long)Tt * Tt * (long long)sizeof(T));
  StagerScope staged(stager);
  // what the tile kernel can use to split K when a tile product has too few workgroups (small T): the largest need
  // over the launches of the plan -- full and ragged tile extents, slabs of a thin start, merged chains, whose one
  // launch covers the summed k of their tiles, and row strips, which come with their own split count
  long ws_bytes = 0;
  {
    std::vector<std::array<long, 3>> seen;
    for (const Cmd& c : plan.cmds) {
      if (c.kind != CMD_GEMM) continue;
      long k = 0;
      for (int kt = c.ki; kt < c.ki + c.kn; ++kt) k += p.tk(kt);
      const std::array<long, 3> shape = {c.rows > 0 ? (long)c.rows : p.tm(c.mi), p.tn(c.ni), k};
      if (c.splits > 1) ws_bytes = std::max(ws_bytes, (long)c.splits * shape[0] * shape[1] * (long)sizeof(T));
      if (std::find(seen.begin(), seen.end(), shape) != seen.end()) continue;
      seen.push_back(shape);
      ws_bytes = std::max(ws_bytes, pl_gemm_tile_workspace_bytes(shape[0], shape[1], shape[2], (int)sizeof(T)));
    }
  }
  void* ws[MAX_EXEC_QUEUES] = {nullptr};
  if (ws_bytes > 0)
    for (int q = 0; q < std::max(1, std::min(p.exec_queues, MAX_EXEC_QUEUES)); ++q) ws[q] = R.res.gemm_ws[q].ensure(ws_bytes);
  const bool trace = R.res.trace_on;
  if (trace) {
    R.res.ensure_timing_events(2 * plan.cmds.size() + 1);
    chk(pl_event_record(R.res.timing_events[0], R.res.h2d), "event record");  // time zero of the timeline
  }

  // Where a fetched tile of A / B lives on the device and with which leading dimension.  Without panels: its own
  // block, dense.  With panels (GemmPlan::panels) the Kg blocks of a row panel of op(A) / column panel of op(B) hold one
  // matrix: tiles one after the other when the operand is contiguous along m / n (leading dimension = tile rows), or a
  // K x tile matrix with leading dimension K when it is contiguous along k.
  // The leading dimension of a ragged tile (or of a panel over a ragged K) is rounded up to 16 elements, so that the
  // kernel can read every tile in 16-byte pieces whatever the problem's dimensions: with the tile's own extent as its
  // leading dimension an odd M, N or K left the tiles of the last block row / column / k-step -- with merged chains
  // every K-major panel -- to the element loads (dgemm 16383^3 from the host: 152 ms against 120 ms at 16384^3).  The
  // padded tile still fits its block of T x T elements when T is a multiple of 16; other tile sizes keep dense tiles.
  // With T a multiple of 128 the m / n extent of a tile is rounded up to whole 128-wide kernel tiles instead: the rows
  // of op(A) and the columns of op(B) up to there lie inside the tile's block (or panel) whichever way the operand is
  // stored, so the kernel may read them (pl_dgemm_tile_padded) and the workgroups on a ragged edge of C need no guarded
  // loads either.
  const int Kg = p.Kg();
  // (whole 256-wide tiles where T allows it: the fp32 kernel's larger macro tiles are 256 wide)
  const bool pad_ld = Tt % 16 == 0;
  const long tile_w = Tt % 256 == 0 ? 256 : Tt % 128 == 0 ? 128 : 0;
  auto padded = [&](long rows) { return pad_ld ? (rows + 15) / 16 * 16 : rows; };
  auto readable = [&](long mn) { return tile_w ? (mn + tile_w - 1) / tile_w * tile_w : mn; };   // <= T
  auto a_tile = [&](int block, int mi, int ki, long* ld) -> T* {
    if (!plan.panels) { *ld = at ? padded(p.tk(ki)) : padded(readable(p.tm(mi))); return (T*)R.pool.at(block); }
    T* base = (T*)R.pool.at(plan.a_first + (long)mi * Kg);
    if (at) { *ld = padded(std::max(1L, p.K)); return base + p.k0(ki); }
    *ld = padded(readable(p.tm(mi)));
    return base + p.k0(ki) * *ld;
  };
  auto b_tile = [&](int block, int ni, int ki, long* ld) -> T* {
    if (!plan.panels) { *ld = bt ? padded(readable(p.tn(ni))) : padded(p.tk(ki)); return (T*)R.pool.at(block); }
    T* base = (T*)R.pool.at(plan.b_first + (long)ni * Kg);
    if (!bt) { *ld = padded(std::max(1L, p.K)); return base + p.k0(ki); }
    *ld = padded(readable(p.tn(ni)));
    return base + p.k0(ki) * *ld;
  };

  // Write-backs into a pageable C are handed to the stager's background thread (it waits for the tile's kernels, copies
  // and scatters at the pace of the link while this thread goes on enqueuing), unless a later command waits for a
  // write-back (a pool smaller than the working set recycles accumulator blocks) or the call is being traced.
  bool defer_wb = pageable[2] && !trace;
  for (const Cmd& c : plan.cmds) defer_wb = defer_wb && !(c.kind == CMD_WRITEBACK && c.signals);

  DrainOnError guard(R.res);
  for (size_t i = 0; i < plan.cmds.size(); ++i) {
    const Cmd& c = plan.cmds[i];
    void* s = R.res.stream(c.stream);
    const bool deferred = defer_wb && c.kind == CMD_WRITEBACK;  // its waits are enqueued with its copy, by the other thread
    for (int w = 0; w < c.nwait && !deferred; ++w) chk(pl_stream_wait_event(s, ev[c.wait[w]]), "stream wait event");
    if (trace) chk(pl_event_record(R.res.timing_events[1 + 2 * i], s), "event record");
    switch (c.kind) {
      case CMD_FETCH_A: {
        const long rows = at ? p.tk(c.ki) : p.tm(c.mi), cols = at ? p.tm(c.mi) : p.tk(c.ki);
        const T* src = at ? A + p.k0(c.ki) + (long)c.mi * Tt * lda : A + (long)c.mi * Tt + p.k0(c.ki) * lda;
        long ld_dst;
        T* dst = a_tile(c.block, c.mi, c.ki, &ld_dst);
        if (pageable[0]) stager.fetch(dst, src, lda, rows, cols, sizeof(T), s, ld_dst);
        else chk(pl_copy2d_async(dst, ld_dst, src, lda, rows, cols, sizeof(T), s), "fetch A tile");
      } break;
      case CMD_FETCH_B: {
        const long rows = bt ? p.tn(c.ni) : p.tk(c.ki), cols = bt ? p.tk(c.ki) : p.tn(c.ni);
        const T* src = bt ? B + (long)c.ni * Tt + p.k0(c.ki) * ldb : B + p.k0(c.ki) + (long)c.ni * Tt * ldb;
        long ld_dst;
        T* dst = b_tile(c.block, c.ni, c.ki, &ld_dst);
        if (pageable[1]) stager.fetch(dst, src, ldb, rows, cols, sizeof(T), s, ld_dst);
        else chk(pl_copy2d_async(dst, ld_dst, src, ldb, rows, cols, sizeof(T), s), "fetch B tile");
      } break;
      case CMD_FETCH_C: {
        // the tile, or the row strip of it the command names, into those rows of the block (which holds the whole tile)
        const long m = p.tm(c.mi), rows = c.rows > 0 ? c.rows : m, cols = p.tn(c.ni);
        const T* src = C + (long)c.mi * Tt + (long)c.ni * Tt * ldc + c.row0;
        T* dst = (T*)R.pool.at(c.block) + c.row0;
        if (pageable[2]) stager.fetch(dst, src, ldc, rows, cols, sizeof(T), s, m);
        else chk(pl_copy2d_async(dst, m, src, ldc, rows, cols, sizeof(T), s), "fetch C tile");
      } break;
      case CMD_GEMM: {
        const long m = p.tm(c.mi), n = p.tn(c.ni);
        long k = 0;  // one launch over the k tiles ki .. ki + kn - 1 (kn > 1 only with the panel layout)
        for (int kt = c.ki; kt < c.ki + c.kn; ++kt) k += p.tk(kt);
        const T* a;
        long la;
        if (c.a_block >= 0) a = a_tile(c.a_block, c.mi, c.ki, &la);
        else { a = at ? A + p.k0(c.ki) + (long)c.mi * Tt * lda : A + (long)c.mi * Tt + p.k0(c.ki) * lda; la = lda; }
        const T* b;
        long lb;
        if (c.b_block >= 0) b = b_tile(c.b_block, c.ni, c.ki, &lb);
        else { b = bt ? B + (long)c.ni * Tt + p.k0(c.ki) * ldb : B + p.k0(c.ki) + (long)c.ni * Tt * ldb; lb = ldb; }
        T* cc;
        long lc;
        if (c.block >= 0) { cc = (T*)R.pool.at(c.block); lc = m; }
        else { cc = C + (long)c.mi * Tt + (long)c.ni * Tt * ldc; lc = ldc; }
        const T bp = c.beta_mode == BETA_ZERO ? T(0) : c.beta_mode == BETA_ONE ? T(1) : beta;
        if (la < 1) la = 1;
        if (lb < 1) lb = 1;
        // what of the operands may be read beyond the tile's ragged edge: tiles in pool blocks, see a_tile / b_tile
        const long m_read = c.a_block >= 0 ? readable(m) : m, n_read = c.b_block >= 0 ? readable(n) : n;
        if (c.rows > 0) {
          // a row strip of the tile: those rows of op(A) and of C, the launch splitting K as the plan says
          a += at ? (long)c.row0 * la : (long)c.row0;
          cc += c.row0;
          chk(GemmFns<T>::tile_padded(ta, tb, c.rows, n, k, alpha, a, la, b, lb, bp, cc, lc, ws[c.stream - STREAM_EXEC0], ws_bytes,
                                      std::max(1, c.splits), std::max<long>(c.rows, m_read - c.row0), n_read, s),
              "tile gemm launch");
        } else {
          chk(GemmFns<T>::tile_padded(ta, tb, m, n, k, alpha, a, la, b, lb, bp, cc, lc, ws[c.stream - STREAM_EXEC0], ws_bytes, 0, m_read, n_read, s),
              "tile gemm launch");
        }
      } break;
      case CMD_REDUCE: {
        const long m = p.tm(c.mi), n = p.tn(c.ni), rows = c.rows > 0 ? c.rows : m;
        T* acc = (T*)R.pool.at(c.block) + c.row0;
        chk(GemmFns<T>::geadd(rows, n, beta, (const T*)R.pool.at(c.a_block) + c.row0, m, acc, m, acc, m, s), "lazy reduce launch");
      } break;
      case CMD_WRITEBACK: {
        // the tile, or the row strip of it the command names (the accumulator block holds the whole tile, m rows)
        const long m = p.tm(c.mi), n = p.tn(c.ni), rows = c.rows > 0 ? c.rows : m;
        T* dst = C + (long)c.mi * Tt + (long)c.ni * Tt * ldc + c.row0;
        const T* src = (const T*)R.pool.at(c.block) + c.row0;
        if (deferred) {
          static_assert(MAX_WAITS <= HostStager::MAX_DEFERRED_WAITS, "a deferred write-back must be able to carry every wait of a command");
          void* after[MAX_WAITS];
          for (int w = 0; w < c.nwait; ++w) after[w] = ev[c.wait[w]];
          stager.write_back_deferred(dst, ldc, src, rows, n, sizeof(T), s, after, c.nwait, m);
        } else if (pageable[2]) stager.write_back(dst, ldc, src, rows, n, sizeof(T), s, m);
        else chk(pl_copy2d_async(dst, ldc, src, m, rows, n, sizeof(T), s), "write back C tile");
      } break;
    }
    if (trace) chk(pl_event_record(R.res.timing_events[2 + 2 * i], s), "event record");
    if (c.signals) {
      ev[i] = R.res.events[next_ev++];
      chk(pl_event_record(ev[i], s), "event record");
    }
  }
  if (defer_wb) stager.finish();  // the background thread is done with the write-back stream and the pinned slots
  R.res.sync_all();
  guard.armed = false;
  staged.finish();
  if (trace) {
    R.res.trace.clear();
    R.res.trace.reserve(plan.cmds.size());
    for (size_t i = 0; i < plan.cmds.size(); ++i) {
      const Cmd& c = plan.cmds[i];
      float t0 = 0, t1 = 0;
      chk(pl_event_elapsed_ms(R.res.timing_events[0], R.res.timing_events[1 + 2 * i], &t0), "event elapsed");
      chk(pl_event_elapsed_ms(R.res.timing_events[0], R.res.timing_events[2 + 2 * i], &t1), "event elapsed");
      R.res.trace.push_back({c.kind, c.mi, c.ni, c.ki, c.stream, (double)t0, (double)t1});
    }
  }
}

template <typename T>
static ATC_p gemm_entry(char TransA, char TransB, long M, long N, long K, T alpha, T* A, long ldA, T* B, long ldB, T beta,
                        T* C, long ldC, ATC_p predef) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  const char ta = (char)toupper(TransA), tb = (char)toupper(TransB);
  if ((ta != 'N' && ta != 'T') || (tb != 'N' && tb != 'T'))
    error("PARALiA%s: invalid transpose flags '%c','%c' (only N and T)\n", GemmFns<T>::name, TransA, TransB);
  if (M < 0 || N < 0 || K < 0) error("PARALiA%s: negative dimension (M=%ld N=%ld K=%ld)\n", GemmFns<T>::name, M, N, K);
  const long rowsA = ta == 'N' ? M : K, rowsB = tb == 'N' ? K : N;
  if (ldA < std::max(1L, rowsA) || ldB < std::max(1L, rowsB) || ldC < std::max(1L, M))
    error("PARALiA%s: leading dimension too small (ldA=%ld ldB=%ld ldC=%ld)\n", GemmFns<T>::name, ldA, ldB, ldC);

  int prev_dev = 0;
  chk(pl_get_device(&prev_dev), "get device");
  if (prev_dev != 0) chk(pl_set_device(0), "set device");
  struct Restore { int d; ~Restore() { if (d != 0) pl_set_device(d); } } restore{prev_dev};

  if (M == 0 || N == 0) {
    ATC_p out = new ATC();
    out->T = 0; out->active_unit_num = 1; out->active_unit_id_list[0] = 0; out->subkernel_num = 0; out->pred_t = 0;
    return out;
  }
  if (!C) error("PARALiA%s: C is null\n", GemmFns<T>::name);
  const bool no_ab = (K == 0 || alpha == T(0));
  if (!no_ab && (!A || !B)) error("PARALiA%s: A or B is null\n", GemmFns<T>::name);

  int locA = 0, locB = 0, locC = 0;
  chk(pl_ptr_location(C, &locC), "pointer location");
  if (no_ab) locA = locB = 0;  // not referenced: treat as resident so nothing is fetched
  else { chk(pl_ptr_location(A, &locA), "pointer location"); chk(pl_ptr_location(B, &locB), "pointer location"); }
  if (locA > 0 || locB > 0 || locC > 0) error("PARALiA%s: operand on device %d; only device 0 is driven\n", GemmFns<T>::name, std::max(locA, std::max(locB, locC)));

  PMDKey key;
  key.routine = GemmFns<T>::name; key.ta = ta; key.tb = tb; key.D1 = M; key.D2 = N; key.D3 = no_ab ? 0 : K;
  key.loc[0] = host_or_dev(locA); key.loc[1] = host_or_dev(locB); key.loc[2] = host_or_dev(locC);
  key.beta_zero = (beta == T(0));
  key.predef_T = predef ? predef->T : -1;
  key.cache_limit = predef ? predef->cache_limit : 0;

  const double t_call = csecond();
  R.phases = Runtime::Phases();
  PMDEntry* entry = nullptr;
  for (auto& e : R.pmd)
    if (e->key == key) { entry = e.get(); break; }
  if (entry) ++R.pmd_hits;
  else {
    ++R.pmd_misses;
    std::unique_ptr<PMDEntry> ne(new PMDEntry());
    ne->key = key;
    ne->atc.reset(new ATC());
    ATC* atc = ne->atc.get();
    if (predef) {
      atc->T = predef->T;
      atc->cache_limit = predef->cache_limit;
      atc->active_unit_num = predef->active_unit_num;
      for (int i = 0; i < std::min(LOC_NUM, std::max(0, predef->active_unit_num)); ++i)
        atc->active_unit_id_list[i] = predef->active_unit_id_list[i];
    }
    ProblemDesc d;
    d.func = GemmFns<T>::name; d.problem = BLAS3;
    d.D1 = M; d.D2 = N; d.D3 = no_ab ? 0 : K;
    d.TransA = ta; d.TransB = tb; d.dtype_sz = sizeof(T); d.numT = 3;
    d.loc[0] = d.out_loc[0] = key.loc[0]; d.loc[1] = d.out_loc[1] = key.loc[1]; d.loc[2] = d.out_loc[2] = key.loc[2];
    d.beta_is_zero = key.beta_zero;
    const bool any_remote = key.loc[0] < 0 || key.loc[1] < 0 || key.loc[2] < 0;
    d.pool_budget_bytes = any_remote ? pool_budget(atc->cache_limit, R.pool.bytes()) : 0;
    // a preset tile larger than every dimension is the whole problem: the limit is judged on the tile that will be used
    const long long t_eff = std::min<long long>(atc->T, std::max(M, std::max(N, K)));
    if (any_remote && atc->cache_limit > 0 && atc->T > 0 && atc->cache_limit < 3LL * t_eff * t_eff * (long long)sizeof(T))
      error("PARALiA%s: Problem cannot run with less memory than %lld\n", GemmFns<T>::name, 3LL * t_eff * t_eff * (long long)sizeof(T));
    // alpha == 0 or K == 0: C <- beta*C only, one "subkernel" per C tile with an empty K; K must not
    // constrain the tile choice then
    if (d.D3 == 0) d.D3 = std::min(M, N);
    double t_phase = csecond();
    atc->autotune_problem(GemmFns<T>::name, d);
    R.phases.autotune = csecond() - t_phase;
    t_phase = csecond();
    if (any_remote) {
      GemmProblem gp;
      gp.M = M; gp.N = N; gp.K = no_ab ? 0 : K; gp.T = atc->T;
      gp.a_remote = key.loc[0] < 0; gp.b_remote = key.loc[1] < 0; gp.c_remote = key.loc[2] < 0;
      gp.beta_zero = key.beta_zero; gp.elem = sizeof(T); gp.exec_queues = atc->exec_queues;
      const long long blk = (long long)atc->T * atc->T * (long long)sizeof(T);
      gp.pool_blocks = (long)std::min<long long>(gemm_max_block_num(gp), d.pool_budget_bytes / blk);
      try {
        ne->plan = build_gemm_plan(gp, atc->order_id);
      } catch (const std::runtime_error&) {
        // the order chosen for the model's K does not fit (K == 0 path): the reference order always does
        try { ne->plan = build_gemm_plan(gp, order_id_of(1, 0)); }
        catch (const std::runtime_error& e2) { error("%s\n", e2.what()); }
        atc->order_id = order_id_of(1, 0);
      }
      atc->update_sk_num(ne->plan.p.subkernels());  // the plan's own problem: a thin start adds k tiles
      atc->distribute_subkernels(ne->plan.p.Mg(), ne->plan.p.Ng(), ne->plan.p.Kg());
    }
    R.phases.plan = csecond() - t_phase;
    if ((int)R.pmd.size() >= PROBLEM_MD_CACHE) R.pmd.erase(R.pmd.begin());
    R.pmd.push_back(std::move(ne));
    entry = R.pmd.back().get();
  }

  ATC* atc = entry->atc.get();
  const bool any_remote = key.loc[0] < 0 || key.loc[1] < 0 || key.loc[2] < 0;
  if (!any_remote) {
    // Every operand already in HBM: one launch over the caller's matrices, alone on the device.
    R.res.ensure_streams(1);
    // (the split-K slices are worth having, not needed: without room for them the launch is unsplit)
    const long ws_bytes = no_ab ? 0 : pl_gemm_tile_alone_workspace_bytes(ta, tb, M, N, K, beta == T(0) ? 1 : 0, (int)sizeof(T));
    void* ws = ws_bytes > 0 ? R.res.gemm_ws[0].ensure_if_room(ws_bytes) : nullptr;
    // An operand the kernel cannot read in 16-byte pieces (its address or its leading dimension is not a multiple of
    // 16 bytes) sends every workgroup to the element loads: 8191^3 with ld = 8191 runs at 57 TFLOP/s (fp32: 103) against
    // 75 (152).  A copy with a padded leading dimension costs two passes over the operand at 3 TB/s, a tenth of that
    // difference once the product's other dimension reaches 2048; taken when the device has the room.
    // The copy is laid out in whole 256-wide kernel tiles along m (or n), like the tiles of the streamed path, so its
    // edge may be read too (m_read, n_read).
    const T* a_use = A;
    const T* b_use = B;
    long lda_use = ldA, ldb_use = ldB, m_read = M, n_read = N;
    if (!no_ab) {
      constexpr long VEC = 16 / (long)sizeof(T);
      // mn_major: the operand's rows run along m (or n); else they run along k and its columns along m (or n)
      auto realigned = [&](int which, const T* p, long ld, long rows, long cols, bool mn_major, long other_dim, long* ld_out, long* read_out) -> const T* {
        const bool unaligned = (reinterpret_cast<uintptr_t>(p) & 15) != 0 || ld % VEC != 0;
        if (!unaligned || other_dim < 2048 || rows < VEC) return p;
        const long mn = mn_major ? rows : cols, mn_tiles = (mn + 255) / 256 * 256;
        const long ld2 = mn_major ? mn_tiles : (rows + 15) / 16 * 16, cols2 = mn_major ? cols : mn_tiles;
        void* copy = R.res.gemm_realigned[which].ensure_if_room((long long)ld2 * cols2 * (long long)sizeof(T));
        if (!copy) return p;
        chk(pl_copy2d_async(copy, ld2, p, ld, rows, cols, sizeof(T), R.res.exec[0]), "operand copy");
        *ld_out = ld2;
        *read_out = mn_tiles;
        return (const T*)copy;
      };
      a_use = realigned(0, A, ldA, ta == 'N' ? M : K, ta == 'N' ? K : M, ta == 'N', N, &lda_use, &m_read);
      b_use = realigned(1, B, ldB, tb == 'N' ? K : N, tb == 'N' ? N : K, tb != 'N', M, &ldb_use, &n_read);
    }
    chk(GemmFns<T>::tile_padded(ta, tb, M, N, no_ab ? 0 : K, alpha, a_use, lda_use, b_use, ldb_use, beta, C, ldC, ws, ws ? ws_bytes : 0, -1, m_read, n_read,
                                R.res.exec[0]), "gemm launch");
    chk(pl_stream_sync(R.res.exec[0]), "stream sync");
  } else {
    const GemmPlan& plan = entry->plan;
    double t_phase = csecond();
    R.pool.ensure(plan.blocks_used, (long long)plan.p.T * plan.p.T * (long long)sizeof(T), atc->cache_limit);
    R.phases.pool = csecond() - t_phase;
    t_phase = csecond();
    R.res.ensure_streams(std::max(1, std::min(plan.p.exec_queues, MAX_EXEC_QUEUES)));
    R.phases.streams = csecond() - t_phase;
    t_phase = csecond();
    const bool pageable[3] = {locA == -2, locB == -2, locC == -2};
    execute_gemm_plan<T>(R, plan, ta, tb, alpha, A, ldA, B, ldB, beta, C, ldC, pageable);
    R.phases.execute = csecond() - t_phase;
  }
  R.phases.total = csecond() - t_call;
  ++entry->calls;
  return atc_copy(atc);
}

// ------------------------------------------------------------------------------------------ BLAS-1
struct Blas1Key { long N; int locx, locy; long T; };

static ATC* blas1_tune(Runtime& R, const char* routine, long N, int locx, int locy, bool y_out, ATC_p predef, size_t elem_span_bytes) {
  PMDKey key;
  key.routine = routine; key.D1 = N; key.D2 = 1; key.D3 = 1;
  key.loc[0] = host_or_dev(locx); key.loc[1] = host_or_dev(locy); key.loc[2] = 0;
  key.predef_T = predef ? predef->T : -1;
  key.cache_limit = predef ? predef->cache_limit : 0;
  for (auto& e : R.pmd)
    if (e->key == key) { ++R.pmd_hits; return e->atc.get(); }
  ++R.pmd_misses;
  std::unique_ptr<PMDEntry> ne(new PMDEntry());
  ne->key = key;
  ne->atc.reset(new ATC());
  ATC* atc = ne->atc.get();
  if (predef) { atc->T = predef->T; atc->cache_limit = predef->cache_limit; }
  ProblemDesc d;
  d.func = routine; d.problem = BLAS1; d.D1 = N; d.D2 = 1; d.D3 = 1; d.dtype_sz = 8; d.numT = 2;
  d.in[0] = 1; d.in[1] = 1; d.in[2] = 0;
  d.out[0] = 0; d.out[1] = y_out ? 1 : 0; d.out[2] = 0;
  d.loc[0] = d.out_loc[0] = key.loc[0]; d.loc[1] = d.out_loc[1] = key.loc[1]; d.loc[2] = d.out_loc[2] = 0;
  atc->autotune_problem(routine, d);
  if (atc->cache_limit > 0) {
    // daxpy.cpp:282-321 sizes the pool as 1 + 2*tiles blocks; under a limit keep at least a 2-deep ring per vector
    const long long need = 4LL * atc->T * (long long)elem_span_bytes;
    if (atc->cache_limit < need) error("PARALiA%s: Problem cannot run with less memory than %lld\n", routine, need);
  }
  if ((int)R.pmd.size() >= PROBLEM_MD_CACHE) R.pmd.erase(R.pmd.begin());
  R.pmd.push_back(std::move(ne));
  return R.pmd.back()->atc.get();
}

// A contiguous span between pinned host memory and the device, through the 2-D copy call: the span is cut into
// columns of 64 KiB (plus a short tail).  The plain 1-D call takes another path through the HIP runtime, on which a
// copy was seen to start only after the copy running on the opposite-direction stream had finished; for the daxpy of
// two host vectors, whose tiles go in on one stream and out on another, that cost 6 ms of 82.
static void copy_span_async(void* dst, const void* src, long long bytes, void* stream, const char* what) {
  const long long col = 65536;
  const long long cols = bytes / col;
  if (cols > 0) chk(pl_copy2d_async(dst, col, src, col, col, cols, 1, stream), what);
  const long long done = cols * col;
  if (bytes > done) chk(pl_copy2d_async((char*)dst + done, bytes - done, (const char*)src + done, bytes - done, bytes - done, 1, 1, stream), what);
}

// Streams 1-D tiles of x and y through a ring of device blocks.  op(tile, xdev, ydev, len, stream) enqueues
// the kernel; write_y sends every y tile back.  Strided vectors move as their contiguous span.
template <typename Op>
static void blas1_stream(Runtime& R, long N, long T, double* x, long incx, int locx, double* y, long incy, int locy, bool write_y, Op op) {
  const long tiles = (N + T - 1) / T;
  const long ax = std::labs(incx), ay = std::labs(incy);
  const bool rx = locx < 0, ry = locy < 0;
  const int ring = (int)std::min<long>(tiles, 3);
  const long long span_x = ((long long)(T - 1) * ax + 1) * 8, span_y = ((long long)(T - 1) * ay + 1) * 8;
  const long long blk = std::max(span_x, span_y);
  R.pool.ensure(2L * ring, blk);
  R.res.ensure_streams(1);
  R.res.ensure_events(3 * (size_t)ring);
  void* s_in = R.res.h2d; void* s_ex = R.res.exec[0]; void* s_out = R.res.d2h;
  HostStager& stager = R.res.stager();
  if (locx == -2 || locy == -2) stager.reserve(blk);
  StagerScope staged(stager);
  std::vector<void*> ev_in(ring), ev_ex(ring), ev_out(ring);
  for (int r = 0; r < ring; ++r) { ev_in[r] = R.res.events[3 * r]; ev_ex[r] = R.res.events[3 * r + 1]; ev_out[r] = R.res.events[3 * r + 2]; }
  DrainOnError guard(R.res);
  for (long t = 0; t < tiles; ++t) {
    const long len = std::min(T, N - t * T);
    const int r = (int)(t % ring);
    // BLAS: with a negative increment the vector runs backwards from the far end of its span
    const long xoff = incx >= 0 ? t * T * ax : (N - t * T - len) * ax;
    const long yoff = incy >= 0 ? t * T * ay : (N - t * T - len) * ay;
    double* xs = x + xoff;
    double* ys = y + yoff;
    double* xd = rx ? (double*)R.pool.at(2 * r) : xs;
    double* yd = ry ? (double*)R.pool.at(2 * r + 1) : ys;
    const long long bx = ((long long)(len - 1) * ax + 1) * 8, by = ((long long)(len - 1) * ay + 1) * 8;
    if (t >= ring) {  // the ring slot is free once its previous tenant has been consumed / written back
      chk(pl_stream_wait_event(s_in, (write_y && ry) ? ev_out[r] : ev_ex[r]), "stream wait event");
    }
    // pageable vectors go through the pinned bounce buffers like matrix tiles do (a span is one long column)
    if (rx) { if (locx == -2) stager.fetch(xd, xs, bx / 8, bx / 8, 1, 8, s_in); else copy_span_async(xd, xs, bx, s_in, "fetch x tile"); }
    if (ry) { if (locy == -2) stager.fetch(yd, ys, by / 8, by / 8, 1, 8, s_in); else copy_span_async(yd, ys, by, s_in, "fetch y tile"); }
    if (rx || ry) {
      chk(pl_event_record(ev_in[r], s_in), "event record");
      chk(pl_stream_wait_event(s_ex, ev_in[r]), "stream wait event");
    }
    op(t, xd, yd, len, s_ex);
    chk(pl_event_record(ev_ex[r], s_ex), "event record");
    if (write_y && ry) {
      chk(pl_stream_wait_event(s_out, ev_ex[r]), "stream wait event");
      if (locy == -2) stager.write_back(ys, by / 8, yd, by / 8, 1, 8, s_out);
      else copy_span_async(ys, yd, by, s_out, "write back y tile");
      chk(pl_event_record(ev_out[r], s_out), "event record");
    }
  }
  R.res.sync_all();
  guard.armed = false;
  staged.finish();
}

static void blas1_common_checks(const char* routine, long N, double* x, long incx, double* y, long incy, int* locx, int* locy) {
  if (N < 0) error("PARALiA%s: negative N\n", routine);
  if (N > 0 && (!x || !y)) error("PARALiA%s: null vector\n", routine);
  if (incx == 0 || incy == 0) error("PARALiA%s: zero increment\n", routine);
  *locx = *locy = 0;
  if (N > 0) { chk(pl_ptr_location(x, locx), "pointer location"); chk(pl_ptr_location(y, locy), "pointer location"); }
  if (*locx > 0 || *locy > 0) error("PARALiA%s: operand on device %d; only device 0 is driven\n", routine, std::max(*locx, *locy));
}

}  // namespace paralia

using namespace paralia;

// The C++ API keeps the reference's error behaviour: print and terminate (its error() never returns).
#define PARALIA_TERMINATE_ON_ERROR(expr)                       \
  try {                                                        \
    return (expr);                                             \
  } catch (const paralia_error& e) {                           \
    fprintf(stderr, "ERROR -> %s", e.what());                  \
    exit(1);                                                   \
  }

namespace paralia {
ATC_p dgemm_impl(char TransA, char TransB, long M, long N, long K, double alpha, double* A, long ldA, double* B, long ldB,
                 double beta, double* C, long ldC, ATC_p predef) {
  return gemm_entry<double>(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef);
}
ATC_p sgemm_impl(char TransA, char TransB, long M, long N, long K, float alpha, float* A, long ldA, float* B, long ldB,
                 float beta, float* C, long ldC, ATC_p predef) {
  return gemm_entry<float>(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef);
}

ATC_p daxpy_impl(long N, double alpha, double* x, long incx, double* y, long incy, ATC_p predef) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  int locx, locy;
  blas1_common_checks("Daxpy", N, x, incx, y, incy, &locx, &locy);
  int prev_dev = 0;
  chk(pl_get_device(&prev_dev), "get device");
  if (prev_dev != 0) chk(pl_set_device(0), "set device");
  struct Restore { int d; ~Restore() { if (d != 0) pl_set_device(d); } } restore{prev_dev};
  if (N == 0) { ATC_p out = new ATC(); out->T = 0; out->active_unit_num = 1; out->active_unit_id_list[0] = 0; out->subkernel_num = 0; return out; }
  ATC* atc = blas1_tune(R, "Daxpy", N, locx, locy, true, predef, 8 * (size_t)std::max(std::labs(incx), std::labs(incy)));
  if (locx >= 0 && locy >= 0) {
    R.res.ensure_streams(1);
    chk(pl_daxpy(N, alpha, x, incx, y, incy, R.res.exec[0]), "daxpy launch");
    chk(pl_stream_sync(R.res.exec[0]), "stream sync");
  } else if (alpha != 0.0) {
    const long T = atc->T;
    blas1_stream(R, N, T, x, incx, locx, y, incy, locy, true, [&](long, double* xd, double* yd, long len, void* s) {
      // inside a tile the span is walked forwards or backwards according to the sign of the increment
      chk(pl_daxpy(len, alpha, xd, incx, yd, incy, s), "daxpy launch");
    });
  }
  return atc_copy(atc);
}

ATC_p ddot_impl(long N, double* x, long incx, double* y, long incy, double* result, ATC_p predef) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  if (!result) error("PARALiADdot: result is null\n");
  int locx, locy;
  blas1_common_checks("Ddot", N, x, incx, y, incy, &locx, &locy);
  int prev_dev = 0;
  chk(pl_get_device(&prev_dev), "get device");
  if (prev_dev != 0) chk(pl_set_device(0), "set device");
  struct Restore { int d; ~Restore() { if (d != 0) pl_set_device(d); } } restore{prev_dev};
  if (N == 0) { ATC_p out = new ATC(); out->T = 0; out->active_unit_num = 1; out->active_unit_id_list[0] = 0; out->subkernel_num = 0; return out; }
  ATC* atc = blas1_tune(R, "Ddot", N, locx, locy, false, predef, 8 * (size_t)std::max(std::labs(incx), std::labs(incy)));
  R.res.ensure_streams(1);
  R.res.ensure_dot();
  if (locx >= 0 && locy >= 0) {
    chk(pl_ddot(N, x, incx, y, incy, R.res.dot_result, 0, R.res.dot_ws, R.res.exec[0]), "ddot launch");
  } else {
    const long T = atc->T;
    // per-tile partials are folded into one device scalar in tile order (ddot.cpp:70,431 sums them on the host)
    blas1_stream(R, N, T, x, incx, locx, y, incy, locy, false, [&](long t, double* xd, double* yd, long len, void* s) {
      chk(pl_ddot(len, xd, incx, yd, incy, R.res.dot_result, t == 0 ? 0 : 1, R.res.dot_ws, s), "ddot launch");
    });
  }
  chk(pl_copy_async(R.res.dot_host, R.res.dot_result, 8, R.res.exec[0]), "ddot result copy");
  chk(pl_stream_sync(R.res.exec[0]), "stream sync");
  *result += *R.res.dot_host;  // the reference accumulates into the caller's scalar (ddot.cpp:431)
  return atc_copy(atc);
}

// ------------------------------------------------------------------------------------------ BLAS-2
// PARALiADgemv (dgemv.cpp:288-718).  One GPU: a device-resident A is one launch; a host-resident A is cut into
// T x T tiles (subkernel mi * Ng + ni, dgemv.cpp:57-60) that cross the link once each through a small ring of device
// blocks while the kernel of the previous tile runs; x and y are staged whole (they are M + N elements against
// M * N of A).  The first subkernel of a y tile applies the caller's beta, later ones accumulate (WR_first /
// DgemvUpdateDevice, dgemv.cpp:121-126).
ATC_p dgemv_impl(char TransA, long M, long N, double alpha, double* A, long ldA, double* x, long incx, double beta, double* y,
                 long incy, ATC_p predef) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  const char ta = (char)toupper(TransA);
  if (ta != 'N' && ta != 'T') error("PARALiADgemv: invalid transpose flag '%c' (only N and T)\n", TransA);
  if (M < 0 || N < 0) error("PARALiADgemv: negative dimension (%ld, %ld)\n", M, N);
  if (ldA < std::max(1L, M)) error("PARALiADgemv: leading dimension %ld smaller than %ld rows\n", ldA, M);
  if (incx == 0 || incy == 0) error("PARALiADgemv: zero increment\n");
  auto empty = [] { ATC_p out = new ATC(); out->T = 0; out->active_unit_num = 1; out->active_unit_id_list[0] = 0; out->subkernel_num = 0; return out; };
  if (M == 0 || N == 0) return empty();  // BLAS quick return: y is not touched
  if (!A || !x || !y) error("PARALiADgemv: null operand\n");
  int locA = 0, locx = 0, locy = 0;
  chk(pl_ptr_location(A, &locA), "pointer location");
  chk(pl_ptr_location(x, &locx), "pointer location");
  chk(pl_ptr_location(y, &locy), "pointer location");
  if (locA > 0 || locx > 0 || locy > 0) error("PARALiADgemv: operand on device %d; only device 0 is driven\n", std::max(locA, std::max(locx, locy)));
  int prev_dev = 0;
  chk(pl_get_device(&prev_dev), "get device");
  if (prev_dev != 0) chk(pl_set_device(0), "set device");
  struct Restore { int d; ~Restore() { if (d != 0) pl_set_device(d); } } restore{prev_dev};

  const long len_x = ta == 'N' ? N : M, len_y = ta == 'N' ? M : N;
  const long ax = std::labs(incx), ay = std::labs(incy);
  const bool beta_zero = beta == 0.0;

  // ---- tuned problem (metadata cache)
  PMDKey key;
  key.routine = "Dgemv"; key.ta = ta; key.D1 = M; key.D2 = N; key.D3 = 1;
  key.loc[0] = host_or_dev(locA); key.loc[1] = host_or_dev(locx); key.loc[2] = host_or_dev(locy);
  key.beta_zero = beta_zero;
  key.predef_T = predef ? predef->T : -1;
  key.cache_limit = predef ? predef->cache_limit : 0;
  ATC* atc = nullptr;
  for (auto& e : R.pmd)
    if (e->key == key) { ++R.pmd_hits; atc = e->atc.get(); break; }
  if (!atc) {
    ++R.pmd_misses;
    std::unique_ptr<PMDEntry> ne(new PMDEntry());
    ne->key = key;
    ne->atc.reset(new ATC());
    atc = ne->atc.get();
    if (predef) {
      atc->T = predef->T; atc->cache_limit = predef->cache_limit; atc->active_unit_num = predef->active_unit_num;
      for (int d = 0; d < LOC_NUM; d++) atc->active_unit_id_list[d] = predef->active_unit_id_list[d];
    }
    ProblemDesc d;
    d.func = "Dgemv"; d.problem = BLAS2; d.D1 = M; d.D2 = N; d.D3 = 1; d.TransA = ta; d.dtype_sz = 8; d.numT = 3;
    d.in[0] = d.in[1] = d.in[2] = 1;
    d.out[0] = d.out[1] = 0; d.out[2] = 1;
    for (int i = 0; i < 3; ++i) d.loc[i] = d.out_loc[i] = key.loc[i];
    d.beta_is_zero = beta_zero;
    d.pool_budget_bytes = key.loc[0] < 0 ? pool_budget(key.cache_limit, R.pool.bytes()) : 0;
    atc->autotune_problem("Dgemv", d);
    if (key.loc[0] < 0) {
      // dgemv.cpp:389-390: one 2-D block (and two 1-D blocks) is the least the routine can run with
      const long long tile = (long long)std::min(atc->T, M) * std::min(atc->T, N) * 8 + 256;
      if (d.pool_budget_bytes < tile) error("PARALiADgemv: Problem cannot run with less memory than %lld\n", tile);
    }
    if ((int)R.pmd.size() >= PROBLEM_MD_CACHE) R.pmd.erase(R.pmd.begin());
    R.pmd.push_back(std::move(ne));
    atc = R.pmd.back()->atc.get();
  }
  if (alpha == 0.0 && beta == 1.0) return atc_copy(atc);  // BLAS quick return

  R.res.ensure_streams(1);
  void* s_in = R.res.h2d; void* s_ex = R.res.exec[0]; void* s_out = R.res.d2h;
  R.res.ensure_events(16);

  // ---- vectors: staged whole; a strided vector moves as its contiguous span (gaps included, so that the
  // write-back of y restores what lies between its elements)
  const long long span_x = ((long long)(len_x - 1) * ax + 1) * 8, span_y = ((long long)(len_y - 1) * ay + 1) * 8;
  double* xd = x;
  double* yd = y;
  void* ev_vec = R.res.events[0];
  bool staged = false;
  DrainOnError guard(R.res);
  if (locx < 0 && alpha != 0.0) {
    xd = (double*)R.res.gemv_x.ensure(span_x);
    chk(pl_copy_async(xd, x, span_x, s_in), "fetch x");
    staged = true;
  }
  if (locy < 0) {
    yd = (double*)R.res.gemv_y.ensure(span_y);
    if (!beta_zero || ay != 1) { chk(pl_copy_async(yd, y, span_y, s_in), "fetch y"); staged = true; }
  }
  if (staged) {
    chk(pl_event_record(ev_vec, s_in), "event record");
    chk(pl_stream_wait_event(s_ex, ev_vec), "stream wait event");
  }

  const long T = atc->T;
  if (locA >= 0 || alpha == 0.0) {
    double* ws = nullptr;
    if (alpha != 0.0) ws = (double*)R.res.gemv_ws.ensure(std::max(8LL, pl_dgemv_workspace_doubles(ta, M, N) * 8));
    chk(pl_dgemv(ta, M, N, alpha, A, ldA, xd, incx, beta, yd, incy, ws, s_ex), "dgemv launch");
  } else {
    const long Mg = (M + T - 1) / T, Ng = (N + T - 1) / T;
    const long tiles = Mg * Ng;
    const long long blk = ((long long)std::min(T, M) * std::min(T, N) * 8 + 255) / 256 * 256;  // slots keep A's alignment
    long long budget = pool_budget(atc->cache_limit, R.pool.bytes());
    const int ring = (int)std::max<long long>(1, std::min<long long>(std::min<long>(tiles, 4), budget / blk));
    R.pool.ensure(ring, blk, atc->cache_limit);
    // every tile has at most max(T, ...) outputs per chunk: size the workspace for the largest tile shape
    long long ws_doubles = 8;
    for (long mi : {0L, Mg - 1})
      for (long ni : {0L, Ng - 1}) {
        const long tm = std::min(T, M - mi * T), tn = std::min(T, N - ni * T);
        ws_doubles = std::max(ws_doubles, pl_dgemv_workspace_doubles(ta, tm, tn));
      }
    double* ws = (double*)R.res.gemv_ws.ensure(ws_doubles * 8);
    for (long t = 0; t < tiles; ++t) {
      const long mi = t / Ng, ni = t % Ng;
      const long tm = std::min(T, M - mi * T), tn = std::min(T, N - ni * T);
      const int r = (int)(t % ring);
      void* ev_in = R.res.events[1 + 2 * r];
      void* ev_ex = R.res.events[2 + 2 * r];
      double* Ad = (double*)R.pool.at(r);
      if (t >= ring) chk(pl_stream_wait_event(s_in, ev_ex), "stream wait event");  // the slot's previous tile was consumed
      if (locA == -2) R.res.stager().fetch(Ad, A + mi * T + ni * T * ldA, ldA, tm, tn, 8, s_in);
      else chk(pl_copy2d_async(Ad, tm, A + mi * T + ni * T * ldA, ldA, tm, tn, 8, s_in), "fetch A tile");
      chk(pl_event_record(ev_in, s_in), "event record");
      chk(pl_stream_wait_event(s_ex, ev_in), "stream wait event");
      // tile (mi, ni) multiplies the x tile of its reduction index into the y tile of its output index
      const long xi = ta == 'N' ? ni : mi, yi = ta == 'N' ? mi : ni;
      const long xlen = ta == 'N' ? tn : tm, ylen = ta == 'N' ? tm : tn;
      const long xoff = incx >= 0 ? xi * T * ax : (len_x - xi * T - xlen) * ax;
      const long yoff = incy >= 0 ? yi * T * ay : (len_y - yi * T - ylen) * ay;
      const bool first = (ta == 'N' ? ni : mi) == 0;
      chk(pl_dgemv(ta, tm, tn, alpha, Ad, tm, xd + xoff, incx, first ? beta : 1.0, yd + yoff, incy, ws, s_ex), "dgemv tile launch");
      chk(pl_event_record(ev_ex, s_ex), "event record");
    }
  }
  if (locy < 0) {
    void* ev_done = R.res.events[15];
    chk(pl_event_record(ev_done, s_ex), "event record");
    chk(pl_stream_wait_event(s_out, ev_done), "stream wait event");
    chk(pl_copy_async(y, yd, span_y, s_out), "write back y");
  }
  R.res.sync_all();
  guard.armed = false;
  return atc_copy(atc);
}

void cache_free_impl(short dev_id) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  if (dev_id != 0) return;  // the host "cache" of the reference (dev -1) holds nothing here
  R.res.sync_all();
  R.pool.release();
  // the device memory that grows with the operands goes with the pool: the split-K workspaces and the aligned copies
  // of unaligned device-resident operands (each is allocated again by the next call that needs it)
  for (auto& w : R.res.gemm_ws) w.release();
  for (auto& w : R.res.gemm_realigned) w.release();
}

void runtime_stats(long* pmd_hits, long* pmd_misses, long long* pool_bytes, long* pmd_entries) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  if (pmd_hits) *pmd_hits = R.pmd_hits;
  if (pmd_misses) *pmd_misses = R.pmd_misses;
  if (pool_bytes) *pool_bytes = R.pool.bytes();
  if (pmd_entries) *pmd_entries = (long)R.pmd.size();
}

void last_call_phases(double seconds[6]) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  const Runtime::Phases& ph = R.phases;
  seconds[0] = ph.autotune; seconds[1] = ph.plan; seconds[2] = ph.pool; seconds[3] = ph.streams; seconds[4] = ph.execute; seconds[5] = ph.total;
}

void stream_queues(int* independent, int* created) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  if (independent) *independent = R.res.independent;
  if (created) *created = R.res.created;
}

void runtime_reset() {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  R.pmd.clear();
  R.pmd_hits = R.pmd_misses = 0;
}

// Everything the library holds on the device goes: block pool, streams, events, workspaces, pinned bounce buffers,
// cached problems (CoCoPeLiaFreeResources + PARALiADevCacheFree, Subkernel.cpp:330,488).  The next call starts cold.
void runtime_shutdown() {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  R.res.drain();
  R.pool.release();
  R.res.destroy();
  R.pmd.clear();
}

void trace_enable(int on) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  R.res.trace_on = on != 0;
  if (!on) R.res.trace.clear();
}

long trace_read(double* rows, long max_rows) {
  Runtime& R = rt();
  std::lock_guard<std::mutex> lk(R.mu);
  const long n = (long)R.res.trace.size();
  for (long i = 0; rows && i < n && i < max_rows; ++i) {
    const Resources::TraceRow& t = R.res.trace[i];
    double* r = rows + i * 7;
    r[0] = t.kind; r[1] = t.mi; r[2] = t.ni; r[3] = t.ki; r[4] = t.stream; r[5] = t.t0_ms; r[6] = t.t1_ms;
  }
  return n;
}
}  // namespace paralia

ATC_p PARALiADgemm(char TransA, char TransB, long int M, long int N, long int K, double alpha, double* A, long int ldA,
                   double* B, long int ldB, double beta, double* C, long int ldC) {
  PARALIA_TERMINATE_ON_ERROR(dgemm_impl(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, nullptr));
}
ATC_p PARALiADgemmControled(char TransA, char TransB, long int M, long int N, long int K, double alpha, double* A,
                            long int ldA, double* B, long int ldB, double beta, double* C, long int ldC, ATC_p predef) {
  PARALIA_TERMINATE_ON_ERROR(dgemm_impl(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef));
}
ATC_p PARALiASgemm(char TransA, char TransB, long int M, long int N, long int K, float alpha, float* A, long int ldA,
                   float* B, long int ldB, float beta, float* C, long int ldC) {
  PARALIA_TERMINATE_ON_ERROR(sgemm_impl(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, nullptr));
}
ATC_p PARALiASgemmControled(char TransA, char TransB, long int M, long int N, long int K, float alpha, float* A,
                            long int ldA, float* B, long int ldB, float beta, float* C, long int ldC, ATC_p predef) {
  PARALIA_TERMINATE_ON_ERROR(sgemm_impl(TransA, TransB, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, predef));
}
ATC_p PARALiADgemv(char TransA, long int M, long int N, double alpha, double* A, long int ldA, double* x, long int incx,
                   double beta, double* y, long int incy) {
  PARALIA_TERMINATE_ON_ERROR(dgemv_impl(TransA, M, N, alpha, A, ldA, x, incx, beta, y, incy, nullptr));
}
ATC_p PARALiADgemvControled(char TransA, long int M, long int N, double alpha, double* A, long int ldA, double* x,
                            long int incx, double beta, double* y, long int incy, ATC_p predef) {
  PARALIA_TERMINATE_ON_ERROR(dgemv_impl(TransA, M, N, alpha, A, ldA, x, incx, beta, y, incy, predef));
}
ATC_p PARALiADaxpy(long int N, double alpha, double* x, long int incx, double* y, long int incy) {
  PARALIA_TERMINATE_ON_ERROR(daxpy_impl(N, alpha, x, incx, y, incy, nullptr));
}
ATC_p PARALiADaxpyControled(long int N, double alpha, double* x, long int incx, double* y, long int incy, ATC_p predef) {
  PARALIA_TERMINATE_ON_ERROR(daxpy_impl(N, alpha, x, incx, y, incy, predef));
}
ATC_p PARALiADdot(long int N, double* x, long int incx, double* y, long int incy, double* result) {
  PARALIA_TERMINATE_ON_ERROR(ddot_impl(N, x, incx, y, incy, result, nullptr));
}
ATC_p PARALiADdotControled(long int N, double* x, long int incx, double* y, long int incy, double* result, ATC_p predef) {
  PARALIA_TERMINATE_ON_ERROR(ddot_impl(N, x, incx, y, incy, result, predef));
}
void PARALiADevCacheFree(short dev_id) {
  try {
    cache_free_impl(dev_id);
  } catch (const paralia_error& e) {
    fprintf(stderr, "ERROR -> %s", e.what());
    exit(1);
  }
}
