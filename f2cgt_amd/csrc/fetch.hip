// Row fetch in front of the fused operators: out[i, :] = row index[i] of a table of opaque
// byte rows (code rows of any width, or plain feature rows), optionally through a per-row slot map
// that redirects hot rows to a second, device-resident table.  The big table may live in pinned
// host memory mapped into the device address space; its rows then travel over the host link,
// which is the reason the hot table exists.
//
// Replaces TensorCache.__getitem__ (examples/tensor_cache.py:49-58): shmtensor.capi.uva_fetch
// (no slot map) and shmtensor.capi.cache_fetch (hot table + id -> slot hash map; here the map is a
// dense int32 array indexed by the id, one dependent load instead of a probe sequence).
//
// A group of 1..64 lanes owns a row and moves it in pieces of V = 16 bytes (8, 4, 2, 1 for rows
// shorter than that) at byte granularity -- the hardware serves unaligned global accesses -- and
// the last piece of a row is moved back so that it ends with the row (the overlap is written
// twice with the same bytes).  Every lane issues the loads of U rows (8 for rows of up to four
// pieces, else 4) before the first store.
#include "common.hpp"

namespace f2cgt {
namespace {

constexpr int kFetchThreads = 256;

struct FetchArgs {
  const uint8_t* table;
  const uint8_t* hot;
  const int32_t* slot;
  uint8_t* out;
  int64_t n, row_bytes, num_rows, num_hot;
  int pieces;       // pieces of V bytes per row
  int group;        // lanes per row (power of two, <= 64)
  int group_shift;
};

template <int V> struct piece_type;
template <> struct piece_type<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct piece_type<8> { typedef uint64_t type; };
template <> struct piece_type<4> { typedef uint32_t type; };
template <> struct piece_type<2> { typedef uint16_t type; };
template <> struct piece_type<1> { typedef uint8_t type; };

template <int V, int kFetchUnroll, typename Idx>
__global__ __launch_bounds__(kFetchThreads) void fetch_rows_kernel(FetchArgs a, const Idx* __restrict__ index) {
  using P = typename piece_type<V>::type;
  const int rows_per_pass = kFetchThreads >> a.group_shift;
  const int sub = threadIdx.x & (a.group - 1);
  const int64_t first = ((int64_t)blockIdx.x * kFetchUnroll) * rows_per_pass + (threadIdx.x >> a.group_shift);

  const uint8_t* src[kFetchUnroll];
#pragma unroll
  for (int u = 0; u < kFetchUnroll; ++u) {
    const int64_t i = first + (int64_t)u * rows_per_pass;
    src[u] = nullptr;
    if (i < a.n) {
      const int64_t id = clamp_idx(index[i], a.num_rows);
      const uint8_t* p = a.table + id * a.row_bytes;
      if (a.slot != nullptr) {
        const int32_t s = a.slot[id];
        if (s >= 0 && (int64_t)s < a.num_hot) p = a.hot + (int64_t)s * a.row_bytes;
      }
      src[u] = p;
    }
  }
  for (int p0 = 0; p0 < a.pieces; p0 += a.group) {
    const int p = p0 + sub;
    int64_t off = (int64_t)p * V;
    off = off + V > a.row_bytes ? a.row_bytes - V : off;
    const bool on = p < a.pieces;
    P v[kFetchUnroll];
#pragma unroll
    for (int u = 0; u < kFetchUnroll; ++u)
      if (on && src[u] != nullptr) v[u] = *reinterpret_cast<const P*>(src[u] + off);
#pragma unroll
    for (int u = 0; u < kFetchUnroll; ++u) {
      const int64_t i = first + (int64_t)u * rows_per_pass;
      if (on && src[u] != nullptr) *reinterpret_cast<P*>(a.out + i * a.row_bytes + off) = v[u];
    }
  }
}

template <int V, int U>
int launch_fetch(FetchArgs a, const void* index, int idx_dtype, hipStream_t st) {
  const int64_t rows_per_block = (int64_t)(kFetchThreads >> a.group_shift) * U;
  const int64_t blocks = ceil_div(a.n, rows_per_block);
  F2CGT_REQUIRE(blocks <= 0x7fffffff, F2CGT_E_UNSUPPORTED, "fetch_rows: %lld rows need more than 2^31 workgroups",
                (long long)a.n);
  if (idx_dtype == F2CGT_DT_I64)
    fetch_rows_kernel<V, U, int64_t><<<dim3((unsigned)blocks), dim3(kFetchThreads), 0, st>>>(
        a, static_cast<const int64_t*>(index));
  else
    fetch_rows_kernel<V, U, int32_t><<<dim3((unsigned)blocks), dim3(kFetchThreads), 0, st>>>(
        a, static_cast<const int32_t*>(index));
  return launch_status("fetch_rows");
}

template <int V>
int launch_fetch(FetchArgs a, const void* index, int idx_dtype, hipStream_t st) {
  a.pieces = (int)ceil_div(a.row_bytes, V);
  a.group = a.pieces >= 64 ? 64 : pow2_ceil(a.pieces);
  a.group_shift = 0;
  while ((1 << a.group_shift) < a.group) ++a.group_shift;
  if (a.pieces <= 4) return launch_fetch<V, 8>(a, index, idx_dtype, st);
  return launch_fetch<V, 4>(a, index, idx_dtype, st);
}

}  // namespace
}  // namespace f2cgt

using namespace f2cgt;

extern "C" int f2cgt_fetch_rows(const void* table, const void* hot, const int32_t* slot_map, const void* index,
                                int idx_dtype, void* out, int64_t num_index, int64_t row_bytes,
                                int64_t num_rows, int64_t num_hot_rows, void* stream) {
  F2CGT_REQUIRE(num_index >= 0 && row_bytes >= 0 && num_rows >= 0 && num_hot_rows >= 0, F2CGT_E_INVALID,
                "fetch_rows: negative size");
  F2CGT_REQUIRE(idx_dtype == F2CGT_DT_I32 || idx_dtype == F2CGT_DT_I64, F2CGT_E_UNSUPPORTED,
                "fetch_rows: index must be int32 or int64");
  if (num_index == 0 || row_bytes == 0) return F2CGT_OK;
  F2CGT_REQUIRE(num_rows > 0, F2CGT_E_INVALID, "fetch_rows: rows requested from an empty table");
  F2CGT_REQUIRE(table && index && out, F2CGT_E_INVALID, "fetch_rows: null buffer");
  F2CGT_REQUIRE((slot_map == nullptr) || (hot != nullptr) || num_hot_rows == 0, F2CGT_E_INVALID,
                "fetch_rows: a slot map needs its hot table");
  FetchArgs a;
  a.table = static_cast<const uint8_t*>(table);
  a.hot = static_cast<const uint8_t*>(hot);
  a.slot = num_hot_rows > 0 ? slot_map : nullptr;
  a.out = static_cast<uint8_t*>(out);
  a.n = num_index;
  a.row_bytes = row_bytes;
  a.num_rows = num_rows;
  a.num_hot = num_hot_rows;
  a.pieces = a.group = a.group_shift = 0;
  hipStream_t st = as_stream(stream);
  if (row_bytes >= 16) return launch_fetch<16>(a, index, idx_dtype, st);
  if (row_bytes >= 8) return launch_fetch<8>(a, index, idx_dtype, st);
  if (row_bytes >= 4) return launch_fetch<4>(a, index, idx_dtype, st);
  if (row_bytes >= 2) return launch_fetch<2>(a, index, idx_dtype, st);
  return launch_fetch<1>(a, index, idx_dtype, st);
}
