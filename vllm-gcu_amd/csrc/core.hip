// Library-wide state: thread-local error text, ABI version, device queries.
#include "common.h"

#include <mutex>

namespace mi355q {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int device_cu_count() {
  static int cached[64];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  std::lock_guard<std::mutex> lk(mu);
  if (cached[dev] == 0) {
    hipDeviceProp_t p;
    cached[dev] = (hipGetDeviceProperties(&p, dev) == hipSuccess && p.multiProcessorCount > 0)
                      ? p.multiProcessorCount
                      : 256;
  }
  return cached[dev];
}

}  // namespace mi355q

extern "C" const char* mi355q_last_error(void) { return mi355q::g_err; }
// bumped whenever an entry point changes its arguments: the Python binding refuses a library of another version
// (a stale build would be called with shifted arguments)
extern "C" int mi355q_abi_version(void) { return 5; }
