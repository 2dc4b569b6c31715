// The worker-thread pool that gathers / scatters tiles of pageable host operands (runtime/host_staging.cpp), run under
// -fsanitize=thread by tests/test_host_sanitizers.py: strided copies of random shapes with 1, 2, 4 and 8 threads, results
// checked.  The device layer is replaced by host stand-ins below: only the threads are exercised, no GPU.
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
int pl_event_create(void** e, int) { *e = malloc(1); return 0; }
int pl_event_destroy(void* e) { free(e); return 0; }
int pl_event_record(void*, void*) { return 0; }
int pl_event_sync(void*) { return 0; }
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
  printf("ok\n");
  return 0;
}
