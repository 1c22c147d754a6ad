// One Lloyd iteration's centre update (codebook training), after the assignment kernel of
// encode.hip has produced the labels:
//   sums[c]   = sum of the rows assigned to centre c,  count[c] = how many
//   centre[c] = sums[c] / count[c]   (a centre without members keeps its value)
//   shift     = how far the centres moved, in the two forms the reference's two trainers test
// Follows examples/my_kmeans.py:128-147 (compute_new_centers: plain mean whatever the metric,
// empty clusters keep the previous centre) and :100-111 (centre shift and stopping rule);
// raft's kmeans::fit (src/kmeans.cu:61-75) stops on the squared form of the same shift.
//
// The partial sums are scratch memory beyond inputs and outputs (n * k floats and n counters):
// f2cgt_kmeans_update takes them from a workspace the caller passes, f2cgt_kmeans_update_static
// from a device array of this file (for callers that cannot allocate).
#include "common.hpp"

namespace f2cgt {
namespace {

constexpr int kKmThreads = 256;
constexpr int kKmLdsFloats = 12 * 1024;   // per-workgroup partial sums kept in LDS up to this many entries

// Scratch of the allocation-free entry point: 65536 sums and 4096 counters, 272 KB that every device
// the library runs on holds until the process ends.  The name is a host-side stand-in, not a device
// address: host code only ever uses the pointer hipGetSymbolAddress returns for the current device.
constexpr int64_t kStaticSums = 65536;
constexpr int64_t kStaticCenters = 4096;
static __device__ __align__(256) unsigned char scratch[(kStaticSums + kStaticCenters) * 4];

struct KmArgs {
  const float* x;
  const int64_t* labels_i64;
  const uint8_t* labels_u8;
  float* centers;
  float* shift;         // [2]: sum_c |dc|, sum_c |dc|^2
  int32_t* stop;        // may be null; nonzero = the centres are final, the step does nothing (1: rule met, 2: shift is NaN)
  float* sums;          // [n * k]
  uint32_t* counts;     // [n]
  int64_t m;
  int n, k;
  int rule;             // 0: never stop; 1: stop when sum |dc|^2 < tol; 2: stop when (sum |dc|)^2 < tol
  float tol;
  int rows_per_block;
};

__device__ __forceinline__ bool km_stopped(const KmArgs& a) { return a.stop != nullptr && *a.stop != 0; }

__global__ __launch_bounds__(kKmThreads) void km_clear_kernel(KmArgs a) {
  if (km_stopped(a)) return;
  const int64_t words = (int64_t)a.n * a.k + a.n;
  uint32_t* w = reinterpret_cast<uint32_t*>(a.sums);   // sums and counts are one block of the scratch
  for (int64_t i = (int64_t)blockIdx.x * kKmThreads + threadIdx.x; i < words; i += (int64_t)gridDim.x * kKmThreads)
    w[i] = 0u;
  if (blockIdx.x == 0 && threadIdx.x < 2) a.shift[threadIdx.x] = 0.f;
}

// fp32 add in memory: the LDS unit's own add, or the L2's (device memory: never a compare-and-swap loop)
template <bool LDS>
__device__ __forceinline__ void add_f32(float* p, float v) {
  if (LDS) atomicAdd(p, v);
  else unsafeAtomicAdd(p, v);
}

__device__ __forceinline__ int km_label(const KmArgs& a, int64_t row) {
  const int64_t l = a.labels_i64 ? a.labels_i64[row] : (int64_t)a.labels_u8[row];
  return (int)(l < 0 ? 0 : (l >= a.n ? a.n - 1 : l));
}

// A workgroup adds its rows into partial sums (LDS when n * k fits, else straight into the
// scratch) and then adds the partial sums into the scratch.
template <bool LDS>
__global__ __launch_bounds__(kKmThreads) void km_accumulate_kernel(KmArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  if (km_stopped(a)) return;
  float* s_sum = reinterpret_cast<float*>(smem);
  uint32_t* s_cnt = reinterpret_cast<uint32_t*>(s_sum + (LDS ? a.n * a.k : 0));
  const int entries = a.n * a.k;
  if (LDS) {
    for (int i = threadIdx.x; i < entries + a.n; i += kKmThreads) reinterpret_cast<uint32_t*>(smem)[i] = 0u;
    __syncthreads();
  }
  const int64_t row0 = (int64_t)blockIdx.x * a.rows_per_block;
  const int64_t left = a.m - row0;
  const int nrows = (int)(left < a.rows_per_block ? left : a.rows_per_block);
  const int64_t items = (int64_t)nrows * a.k;
  float* sums = LDS ? s_sum : a.sums;
  uint32_t* counts = LDS ? s_cnt : a.counts;
  for (int64_t e = threadIdx.x; e < items; e += kKmThreads) {
    const int r = (int)(e / a.k), col = (int)(e - (int64_t)r * a.k);
    const int c = km_label(a, row0 + r);
    add_f32<LDS>(sums + c * a.k + col, a.x[(row0 + r) * a.k + col]);
    if (col == 0) atomicAdd(counts + c, 1u);
  }
  if (LDS) {
    __syncthreads();
    for (int i = threadIdx.x; i < entries; i += kKmThreads) {
      const float v = s_sum[i];
      if (v != 0.f) add_f32<false>(a.sums + i, v);
    }
    for (int i = threadIdx.x; i < a.n; i += kKmThreads) {
      const uint32_t v = s_cnt[i];
      if (v != 0u) atomicAdd(a.counts + i, v);
    }
  }
}

// One wave per centre: the new centre, and its share of the shift.
__global__ __launch_bounds__(kKmThreads) void km_finalize_kernel(KmArgs a) {
  if (km_stopped(a)) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int c = blockIdx.x * (kKmThreads / kWave) + (threadIdx.x / kWave);
  if (c >= a.n) return;
  const uint32_t cnt = a.counts[c];
  float d2 = 0.f;
  if (cnt > 0u) {
    const float members = (float)cnt;
    for (int j = lane; j < a.k; j += kWave) {
      const float old = a.centers[(int64_t)c * a.k + j];
      const float now = a.sums[(int64_t)c * a.k + j] / members;
      const float d = now - old;
      d2 += d * d;
      a.centers[(int64_t)c * a.k + j] = now;
    }
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) d2 += __shfl_xor(d2, off);
  if (lane == 0 && !(d2 <= 0.f)) {   // a NaN shift is added too: the decide kernel has to see it
    add_f32<false>(a.shift, sqrtf(d2));
    add_f32<false>(a.shift + 1, d2);
  }
}

// Decides, on the device, whether the centres just written are final (so that a training loop
// needs no host read-back per iteration: every later step sees the flag and does nothing).
__global__ void km_decide_kernel(KmArgs a) {
  if (a.stop == nullptr || *a.stop != 0 || a.rule == 0) return;
  const float s = a.rule == 1 ? a.shift[1] : a.shift[0] * a.shift[0];
  // a shift that is not a number never passes `s < tol`: flag it (2) so that the loop ends and the
  // caller can tell (examples/my_kmeans.py:108-109 gives up on such a fit)
  if (s != s) *a.stop = 2;
  else if (s < a.tol) *a.stop = 1;
}

int km_check(const char* what, const float* x, const int64_t* l64, const uint8_t* l8, float* centers, float* shift,
             int64_t m, int64_t n, int64_t k, int rule) {
  F2CGT_REQUIRE(m >= 0 && n > 0 && k > 0, F2CGT_E_INVALID, "%s: sizes must be m >= 0, n > 0, k > 0", what);
  F2CGT_REQUIRE(n <= 65536 && k <= 65536 && n * k < (1ll << 30), F2CGT_E_UNSUPPORTED, "%s: centre set too large", what);
  F2CGT_REQUIRE(rule >= 0 && rule <= 2, F2CGT_E_INVALID, "%s: stop rule must be 0, 1 or 2", what);
  F2CGT_REQUIRE((l64 != nullptr) != (l8 != nullptr), F2CGT_E_INVALID, "%s: give int64 labels or uint8 labels", what);
  F2CGT_REQUIRE(l8 == nullptr || n <= 256, F2CGT_E_INVALID, "%s: uint8 labels need n <= 256", what);
  F2CGT_REQUIRE(centers != nullptr && shift != nullptr && (m == 0 || x != nullptr), F2CGT_E_INVALID,
                "%s: null buffer", what);
  return 0;
}

int km_run(const char* what, KmArgs a, hipStream_t st) {
  const int64_t words = (int64_t)a.n * a.k + a.n;
  const int cus = num_cus();
  int64_t clear_grid = ceil_div(words, kKmThreads * 4);
  clear_grid = clear_grid < 1 ? 1 : (clear_grid > cus * 4 ? cus * 4 : clear_grid);
  km_clear_kernel<<<(unsigned)clear_grid, kKmThreads, 0, st>>>(a);
  if (a.m > 0) {
    // rows per workgroup: enough of them to pay for flushing the partial sums, yet a grid that fills the device
    const bool lds = words <= kKmLdsFloats;
    int64_t rpb = ceil_div(a.m, (int64_t)cus * 8);
    const int64_t floor = lds ? ceil_div(4 * words, a.k) : 64;
    rpb = rpb < floor ? floor : rpb;
    rpb = rpb > (1 << 20) ? (1 << 20) : rpb;
    a.rows_per_block = (int)rpb;
    const int64_t grid = ceil_div(a.m, rpb);
    if (grid > 0x7fffffffll) return fail(F2CGT_E_UNSUPPORTED, "%s: too many rows", what);
    if (lds) km_accumulate_kernel<true><<<(unsigned)grid, kKmThreads, (size_t)words * 4, st>>>(a);
    else km_accumulate_kernel<false><<<(unsigned)grid, kKmThreads, 0, st>>>(a);
  }
  km_finalize_kernel<<<(unsigned)ceil_div(a.n, kKmThreads / kWave), kKmThreads, 0, st>>>(a);
  km_decide_kernel<<<1, 1, 0, st>>>(a);
  return launch_status(what);
}

}  // namespace
}  // namespace f2cgt

using namespace f2cgt;

extern "C" int64_t f2cgt_kmeans_update_workspace_bytes(int64_t n, int64_t k) {
  if (n <= 0 || k <= 0) return 0;
  return ((n * k + n) * 4 + 255) / 256 * 256;
}

extern "C" int f2cgt_kmeans_update(const float* x, const int64_t* labels_i64, const uint8_t* labels_u8,
                                   float* centers, float* shift, int32_t* stop, int stop_rule, float tol,
                                   void* workspace, int64_t workspace_bytes, int64_t m, int64_t n, int64_t k,
                                   void* stream) {
  const char* what = "kmeans_update";
  if (int rc = km_check(what, x, labels_i64, labels_u8, centers, shift, m, n, k, stop_rule)) return rc;
  F2CGT_REQUIRE(workspace != nullptr && workspace_bytes >= f2cgt_kmeans_update_workspace_bytes(n, k) &&
                    aligned(workspace, 16),
                F2CGT_E_INVALID, "%s: workspace of %lld bytes (16-byte aligned) needed", what,
                (long long)f2cgt_kmeans_update_workspace_bytes(n, k));
  KmArgs a{};
  a.x = x; a.labels_i64 = labels_i64; a.labels_u8 = labels_u8; a.centers = centers; a.shift = shift; a.stop = stop;
  a.sums = static_cast<float*>(workspace);
  a.counts = reinterpret_cast<uint32_t*>(a.sums + n * k);
  a.m = m; a.n = (int)n; a.k = (int)k; a.rule = stop_rule; a.tol = tol;
  return km_run(what, a, as_stream(stream));
}

extern "C" int f2cgt_kmeans_update_static(const float* x, const int64_t* labels_i64, const uint8_t* labels_u8,
                                          float* centers, float* shift, int32_t* stop, int stop_rule, float tol,
                                          int64_t m, int64_t n, int64_t k, void* stream) {
  const char* what = "kmeans_update_static";
  if (int rc = km_check(what, x, labels_i64, labels_u8, centers, shift, m, n, k, stop_rule)) return rc;
  F2CGT_REQUIRE(n * k <= kStaticSums && n <= kStaticCenters, F2CGT_E_UNSUPPORTED,
                "%s: at most %lld sums (n * k) and %lld centres fit the built-in scratch (got %lld and %lld); "
                "use f2cgt_kmeans_update with a workspace",
                what, (long long)kStaticSums, (long long)kStaticCenters, (long long)(n * k), (long long)n);
  // the device address of the scratch array, looked up once per device (every device has its own copy)
  static void* scratch_of[64] = {nullptr};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= 64) return fail(F2CGT_E_DEVICE, "%s: no current device", what);
  void* base = __atomic_load_n(&scratch_of[dev], __ATOMIC_ACQUIRE);
  if (base == nullptr) {
    e = hipGetSymbolAddress(&base, HIP_SYMBOL(scratch));
    if (e != hipSuccess || base == nullptr)
      return fail((int)(e != hipSuccess ? e : hipErrorInvalidSymbol), "%s: cannot resolve the scratch array: %s", what,
                  hipGetErrorString(e));
    __atomic_store_n(&scratch_of[dev], base, __ATOMIC_RELEASE);
  }
  KmArgs a{};
  a.x = x; a.labels_i64 = labels_i64; a.labels_u8 = labels_u8; a.centers = centers; a.shift = shift; a.stop = stop;
  a.sums = static_cast<float*>(base);
  a.counts = reinterpret_cast<uint32_t*>(a.sums + n * k);
  a.m = m; a.n = (int)n; a.k = (int)k; a.rule = stop_rule; a.tol = tol;
  return km_run(what, a, as_stream(stream));
}
