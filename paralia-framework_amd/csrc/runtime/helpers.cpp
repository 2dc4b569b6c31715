// Helper surface of the drivers (allocation by location, copies, seeded fill, equality tests, timers) and the
// error()/warning() pair.  These stand where the reference's un-vendored unihelpers stand; call sites:
// Benchmarking/CuCuBLAS/src/PARALia/dgemm_runner.cpp:45-110.
#include <dlfcn.h>
#include <sys/time.h>

#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "backend_wrappers.hpp"
#include "paralia_hip.h"

void error(const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  throw paralia_error(PL_ERR_ARG, buf);
}

void warning(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  fprintf(stderr, "WARNING -> ");
  vfprintf(stderr, fmt, ap);
  va_end(ap);
}

void massert(bool cond, const char* fmt, ...) {
  if (cond) return;
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  throw paralia_error(PL_ERR_ARG, buf);
}

double csecond() {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

static void hip_check(int rc, const char* what) {
  if (rc != 0) throw paralia_error(rc, std::string(what) + ": " + pl_last_error());
}

// The database shipped with the library: <dir of libparalia.so>/../db/mi355x
std::string paralia_default_db_dir() {
  Dl_info info;
  if (dladdr((void*)&paralia_default_db_dir, &info) && info.dli_fname) {
    std::string p(info.dli_fname);
    const size_t slash = p.rfind('/');
    if (slash != std::string::npos) return p.substr(0, slash) + "/../db/mi355x";
  }
  return "db/mi355x";
}

void* CoCoMalloc(long long bytes, short loc, short /*write_flag*/) {
  void* p = nullptr;
  if (bytes <= 0) return nullptr;
  if (loc >= 0) {
    hip_check(pl_set_device(loc), "CoCoMalloc");
    hip_check(pl_malloc_device(&p, bytes), "CoCoMalloc(device)");
  } else if (loc == -1) {
    hip_check(pl_malloc_pinned(&p, bytes), "CoCoMalloc(pinned)");
  } else if (loc == -2) {
    if (posix_memalign(&p, 4096, (size_t)bytes) != 0) p = nullptr;
    if (!p) error("CoCoMalloc: pageable allocation of %lld bytes failed\n", bytes);
  } else {
    error("CoCoMalloc: unknown location %d\n", loc);
  }
  return p;
}

void CoCoFree(void* ptr, short loc) {
  if (!ptr) return;
  if (loc >= 0) hip_check(pl_free_device(ptr), "CoCoFree(device)");
  else if (loc == -1) hip_check(pl_free_pinned(ptr), "CoCoFree(pinned)");
  else free(ptr);
}

void CoCoMemcpy(void* dest, void* src, long long bytes, short loc_dest, short loc_src) {
  if (loc_dest < 0 && loc_src < 0) memcpy(dest, src, (size_t)bytes);
  else hip_check(pl_copy(dest, src, bytes), "CoCoMemcpy");
}

void CoCoSyncCheckErr() { hip_check(pl_sync_check(), "CoCoSyncCheckErr"); }

short CoCoGetPtrLoc(const void* ptr) {
  int loc = PL_LOC_HOST_PAGEABLE;
  hip_check(pl_ptr_location(ptr, &loc), "CoCoGetPtrLoc");
  // the scheduler distinguishes only host from device; pinned-ness matters for copy speed, not for routing
  return (short)loc;
}

void CoCoPeLiaSelectDevice(short dev_id) {
  if (dev_id >= 0) hip_check(pl_set_device(dev_id), "CoCoPeLiaSelectDevice");
}
short CoCoPeLiaGetDevice() {
  int d = 0;
  hip_check(pl_get_device(&d), "CoCoPeLiaGetDevice");
  return (short)d;
}
void CoCoPeLiaDevGetMemInfo(long long* free_dev_mem, long long* max_dev_mem) {
  hip_check(pl_mem_info(free_dev_mem, max_dev_mem), "CoCoPeLiaDevGetMemInfo");
}

namespace {
inline uint64_t splitmix64(uint64_t s) {
  uint64_t z = (s += 0x9E3779B97F4A7C15ULL);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}
inline uint64_t draw(uint64_t seed, uint64_t i) { return splitmix64(seed * 0xD1342543DE82EF95ULL + i * 0x9E3779B97F4A7C15ULL); }
inline void gen(double* p, long long off, long long n, uint64_t seed) {
  for (long long i = 0; i < n; ++i) p[i] = (double)(draw(seed, (uint64_t)(off + i)) >> 11) * (2.0 / 9007199254740992.0) - 1.0;
}
inline void gen(float* p, long long off, long long n, uint64_t seed) {
  for (long long i = 0; i < n; ++i) p[i] = (float)(draw(seed, (uint64_t)(off + i)) >> 40) * (2.0f / 16777216.0f) - 1.0f;
}
}  // namespace

template <typename T> void CoCoVecInit(T* vec, long long length, int seed, short loc) {
  if (length <= 0) return;
  if (loc < 0) {
    gen(vec, 0, length, (uint64_t)seed);
    return;
  }
  const long long chunk = 1LL << 22;
  void* stage = nullptr;
  hip_check(pl_malloc_pinned(&stage, chunk * (long long)sizeof(T)), "CoCoVecInit");
  for (long long off = 0; off < length; off += chunk) {
    const long long n = std::min(chunk, length - off);
    gen((T*)stage, off, n, (uint64_t)seed);
    hip_check(pl_copy(vec + off, stage, n * (long long)sizeof(T)), "CoCoVecInit");
  }
  hip_check(pl_free_pinned(stage), "CoCoVecInit");
}
template void CoCoVecInit<double>(double*, long long, int, short);
template void CoCoVecInit<float>(float*, long long, int, short);

// Matching decimal digits of the worst element.  The difference of element i is taken relative to
// max(|ref_i|, |x_i|, rms(ref)): an element that is small only because its terms cancelled is judged on the scale
// of the vector, not on its own.
template <typename T> static short test_equality(T* ref, T* x, long long n, int cap) {
  long double ss = 0;
  for (long long i = 0; i < n; ++i) ss += (long double)ref[i] * ref[i];
  const double rms = n > 0 ? (double)sqrtl(ss / n) : 0.0;
  int worst = cap;
  for (long long i = 0; i < n; ++i) {
    const double d = fabs((double)ref[i] - (double)x[i]);
    if (d == 0) continue;
    if (std::isnan(d)) return 0;
    const double scale = fmax(fmax(fabs((double)ref[i]), fabs((double)x[i])), rms);
    int digits = (int)floor(-log10(d / scale));
    if (digits < 0) digits = 0;
    if (digits < worst) worst = digits;
  }
  return (short)worst;
}
short Dtest_equality(double* C_comp, double* C, long long size) { return test_equality(C_comp, C, size, 16); }
short Stest_equality(float* C_comp, float* C, long long size) { return test_equality(C_comp, C, size, 7); }
