// Library-level state: per-thread error text and the cached device description.
#include "common.hpp"

#include <atomic>

namespace f2cgt {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int num_cus() {
  static std::atomic<int> cached[64];   // 0 = not asked yet; callers may come from several threads
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

}  // namespace f2cgt

extern "C" {

int f2cgt_version(void) { return 100; }

const char* f2cgt_last_error(void) { return f2cgt::error_buffer(); }

int f2cgt_num_cus(void) { return f2cgt::num_cus(); }

}  // extern "C"
