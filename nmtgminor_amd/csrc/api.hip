// Library-wide plumbing of libnmtg_hip.so: version, per-thread error text, device facts.
#include "common.hip.h"
#include <mutex>

namespace nmtg {

std::string& last_error_slot() {
  static thread_local std::string slot;
  return slot;
}

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  last_error_slot() = buf;
  return code;
}

int num_cus() {
  constexpr int MAX_DEV = 64;
  static int cached[MAX_DEV] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) {
    (void)hipGetLastError();
    return 256;
  }
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    cached[dev] = n;
  }
  return cached[dev];
}

}  // namespace nmtg

extern "C" int nmtg_version(void) { return 100; }

extern "C" const char* nmtg_last_error(void) { return nmtg::last_error_slot().c_str(); }
