// The worker-thread pool that gathers / scatters tiles of pageable host operands (runtime/host_staging.cpp), run under
// -fsanitize=thread by tests/test_host_sanitizers.py: strided copies of random shapes with 1, 2, 4 and 8 threads, results
// checked; then the stager itself: tiles fetched through the pinned slots, written back by the blocking call and by
// the background thread of the deferred one (more tiles than slots, so the thread recycles them), finished, abandoned
// and torn down with work still queued.  The device layer is replaced by host stand-ins below: only the threads are
// exercised, no GPU.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include "runtime/host_staging.hpp"
#include "paralia_hip.h"
// host stand-ins for the C ABI calls host_staging.cpp links against
extern "C" {
const char* pl_last_error(void) { return ""; }
int pl_malloc_pinned(void** p, long long b) { *p = malloc(b); return 0; }
int pl_free_pinned(void* p) { free(p); return 0; }
int pl_get_device(int* d) { *d = 0; return 0; }
int pl_set_device(int) { return 0; }
int pl_event_create(void** e, int) { *e = malloc(1); return 0; }
int pl_event_destroy(void* e) { free(e); return 0; }
int pl_event_record(void*, void*) { return 0; }
int pl_event_sync(void*) { return 0; }
int pl_stream_wait_event(void*, void*) { return 0; }
int pl_copy_async(void* d, const void* s, long long b, void*) { memcpy(d, s, b); return 0; }
int pl_copy2d_async(void* d, long ldd, const void* s, long lds, long rows, long cols, int elem, void*) {
  for (long c = 0; c < cols; ++c) memcpy((char*)d + c * ldd * elem, (const char*)s + c * lds * elem, rows * elem);
  return 0;
}
}
int main() {
  using namespace paralia;
  for (int nt : {1, 2, 4, 8}) {
    CopyThreads pool(nt);
    for (int rep = 0; rep < 200; ++rep) {
      const long rows = 1 + rand() % 5000, cols = 1 + rand() % 300, ld = rows + rand() % 7;
      std::vector<double> src((size_t)ld * cols), dst((size_t)rows * cols, -1.0);
      for (size_t i = 0; i < src.size(); ++i) src[i] = (double)i;
      pool.copy2d(dst.data(), rows * 8, src.data(), ld * 8, rows * 8, cols);
      for (long c = 0; c < cols; ++c)
        for (long r = 0; r < rows; r += 97)
          if (dst[c * rows + r] != src[c * ld + r]) { printf("mismatch\n"); return 1; }
    }
    std::vector<char> a(9 << 20, 1), b(9 << 20, 0);
    pool.copy2d(b.data(), a.size(), a.data(), a.size(), a.size(), 1);
    if (memcmp(a.data(), b.data(), a.size())) { printf("mismatch long\n"); return 1; }
  }
  // the stager: "device" memory is host memory here, copies complete inside the stand-ins
  for (int round = 0; round < 3; ++round) {
    const long rows = 300 + 50 * round, cols = 40, ld = rows + 5, tiles = 23;
    std::vector<double> host((size_t)ld * cols * tiles), back((size_t)ld * cols * tiles, -1.0), dev((size_t)rows * cols * tiles);
    HostStager st;   // after the buffers: its destructor drops what is still queued before they go
    for (size_t i = 0; i < host.size(); ++i) host[i] = (double)i;
    for (long t = 0; t < tiles; ++t) st.fetch(dev.data() + t * rows * cols, host.data() + t * ld * cols, ld, rows, cols, 8, nullptr);
    void* after[2] = {nullptr, nullptr};
    for (long t = 0; t < tiles; ++t) {
      if (round == 0) st.write_back(back.data() + t * ld * cols, ld, dev.data() + t * rows * cols, rows, cols, 8, nullptr);
      else st.write_back_deferred(back.data() + t * ld * cols, ld, dev.data() + t * rows * cols, rows, cols, 8, nullptr, after, 2);
    }
    if (round == 2) {
      st.abandon();            // whatever was not scattered yet is dropped; nothing may be touched afterwards
      for (long t = 0; t < 3; ++t) st.write_back_deferred(back.data() + t * ld * cols, ld, dev.data() + t * rows * cols, rows, cols, 8, nullptr, after, 0);
      continue;                // destructor with requests possibly still queued
    }
    st.finish();
    for (long t = 0; t < tiles; ++t)
      for (long c = 0; c < cols; ++c)
        for (long r = 0; r < rows; r += 13)
          if (back[t * ld * cols + c * ld + r] != host[t * ld * cols + c * ld + r]) { printf("stager mismatch\n"); return 1; }
  }
  printf("ok\n");
  return 0;
}
