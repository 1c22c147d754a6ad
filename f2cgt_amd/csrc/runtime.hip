// Library-level state: per-thread error text and the cached device description.
#include "common.hpp"

namespace f2cgt {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int num_cus() {
  static int cached[64];
  static bool known[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!known[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev] = n;
    known[dev] = true;
  }
  return cached[dev];
}

}  // namespace f2cgt

extern "C" {

int f2cgt_version(void) { return 100; }

const char* f2cgt_last_error(void) { return f2cgt::error_buffer(); }

int f2cgt_num_cus(void) { return f2cgt::num_cus(); }

}  // extern "C"
