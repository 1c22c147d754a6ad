// Library-level state: per-thread error text and the cached device description.
#include "common.hpp"

#include <atomic>

namespace f2cgt {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

namespace {
thread_local bool t_plan_only = false;
thread_local f2cgt_plan t_plan = {};
}  // namespace

bool plan_only() { return t_plan_only; }

void plan_record(const char* kernel, int64_t grid, int block, int64_t lds_bytes, int rows_per_block, int a0,
                 int a1, int a2, int a3) {
  snprintf(t_plan.kernel, sizeof(t_plan.kernel), "%s", kernel);
  t_plan.grid = grid;
  t_plan.block = block;
  t_plan.lds_bytes = lds_bytes;
  t_plan.rows_per_block = rows_per_block;
  t_plan.aux[0] = a0; t_plan.aux[1] = a1; t_plan.aux[2] = a2; t_plan.aux[3] = a3;
}

std::atomic<int> g_store_mode{F2CGT_STORE_AUTO};

bool stream_output(int64_t out_bytes, int64_t row_bytes, double edges_per_row) {
  const int mode = g_store_mode.load(std::memory_order_relaxed);
  if (mode == F2CGT_STORE_STREAM) return true;
  if (mode == F2CGT_STORE_CACHED) return false;
  const bool early = row_bytes % 128 == 0 || edges_per_row >= 6.0;
  return out_bytes > (early ? 140000000ll : 220000000ll);
}

int store_mode() { return g_store_mode.load(std::memory_order_relaxed); }

int num_cus() {
  if (t_plan_only) return 256;   // a dry run must not depend on (or wake) a device
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

int f2cgt_set_store_mode(int mode) {
  if (mode != F2CGT_STORE_AUTO && mode != F2CGT_STORE_STREAM && mode != F2CGT_STORE_CACHED) {
    return f2cgt::fail(F2CGT_E_INVALID, "set_store_mode: mode %d is none of AUTO, STREAM, CACHED", mode);
  }
  return f2cgt::g_store_mode.exchange(mode, std::memory_order_relaxed);
}

int f2cgt_set_plan_only(int on) {
  const int was = f2cgt::t_plan_only ? 1 : 0;
  f2cgt::t_plan_only = on != 0;
  if (on) f2cgt::t_plan = f2cgt_plan{};
  return was;
}

int f2cgt_last_plan(f2cgt_plan* out) {
  if (out == nullptr) return F2CGT_E_INVALID;
  *out = f2cgt::t_plan;
  return f2cgt::t_plan.kernel[0] ? F2CGT_OK : F2CGT_E_INVALID;
}

}  // extern "C"
