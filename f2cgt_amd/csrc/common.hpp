// Shared host/device helpers of libf2cgt_hip.so (gfx950 only, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/f2cgt.h"

namespace f2cgt {

constexpr int kWave = 64;

// ---- error reporting ---------------------------------------------------------
char* error_buffer();  // thread-local, 512 bytes (defined in runtime.hip)

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

// Checks the launch that was just enqueued; returns 0 or the hipError_t (> 0).
inline int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  snprintf(error_buffer(), 512, "%s: %s", what, hipGetErrorString(e));
  return (int)e;
}

#define F2CGT_REQUIRE(cond, code, ...) \
  do {                                 \
    if (!(cond)) return ::f2cgt::fail((code), __VA_ARGS__); \
  } while (0)

int num_cus();  // compute units of the current device (cached per device; 256 without a device)

// ---- dry runs ------------------------------------------------------------------
// While plan_only() is true for the calling thread, the fused aggregation launchers record the
// kernel they chose and its launch geometry with plan_record() and return without touching the
// device (no attribute call, no launch, no pointer dereferenced).
bool plan_only();
void plan_record(const char* kernel, int64_t grid, int block, int64_t lds_bytes, int rows_per_block,
                 int a0 = 0, int a1 = 0, int a2 = 0, int a3 = 0);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

__host__ __device__ constexpr int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline int pow2_ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

// ---- device helpers ----------------------------------------------------------
template <typename Idx>
__device__ __forceinline__ int64_t clamp_idx(Idx v, int64_t hi_exclusive) {
  int64_t x = (int64_t)v;
  x = x < 0 ? 0 : x;
  return x >= hi_exclusive ? hi_exclusive - 1 : x;
}

// Edge range of CSC row r, clamped to [0, num_edges] and made monotone.
template <typename Idx>
__device__ __forceinline__ void row_range(const Idx* __restrict__ indptr, int64_t r,
                                          int64_t num_edges, int64_t& b, int64_t& e) {
  int64_t b0 = (int64_t)indptr[r];
  int64_t e0 = (int64_t)indptr[r + 1];
  b0 = b0 < 0 ? 0 : (b0 > num_edges ? num_edges : b0);
  e0 = e0 < b0 ? b0 : (e0 > num_edges ? num_edges : e0);
  b = b0;
  e = e0;
}

// An output that fits the 256 MB last-level cache is best written with plain stores (it stays
// there for the consumer, and a 100 MB block is absorbed at 7+ TB/s); a larger one is best
// streamed past the caches with non-temporal stores: 4-bit affine aggregation, 400-byte rows,
// 1e6 rows: 124 us plain, 94 us non-temporal; 5e5 rows: 48 us plain, 51 us non-temporal.
// The crossover measured with dense 16-byte-per-lane stores lies between 200 and 240 MB.
// That holds for a buffer that is written again while its lines are still cached.  With six
// 100 MB outputs in rotation (nothing of a buffer left in the cache when its turn comes) the plain
// form takes 32.7 us per launch and the non-temporal one 27.7 us, which is also what it takes on
// one buffer: the streamed form does not depend on the cache state.  The size rule is therefore
// only the default (F2CGT_STORE_AUTO); f2cgt_set_store_mode overrides it either way.
// The crossover comes earlier when a launch reads more per output row or writes whole 128-byte lines:
// at 10 edges per row plain against streamed stores take 62.9 / 56.1 us at 160 MB and 95.3 / 69.2 us at
// 200 MB (8-bit codes, 128 columns; 76.1 / 66.2 and 110.5 / 81.0 us at 4 bit and 100 columns), at 3 edges
// per row 37.6 / 38.4 and 48.7 / 44.2 us (128 columns) but 36.4 / 40.9 and 49.9 / 50.9 us at 100 columns,
// whose 400-byte rows leave partial lines to merge.  Hence 140 MB for rows of whole lines or at least six
// edges per row, and 220 MB otherwise.
bool stream_output(int64_t out_bytes, int64_t row_bytes, double edges_per_row);
int store_mode();   // F2CGT_STORE_AUTO / _STREAM / _CACHED as last set by f2cgt_set_store_mode

// Non-temporal stores: the aggregation output is written once and never re-read by
// the kernel, so it should not displace gathered code rows from L2 / MALL.
__device__ __forceinline__ void store_nt(float* p, float v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void store_nt2(float* p, float a, float b) {
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 v = {a, b};
  __builtin_nontemporal_store(v, reinterpret_cast<f2*>(p));
}
__device__ __forceinline__ void store_nt4(float* p, float a, float b, float c, float d) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  f4 v = {a, b, c, d};
  __builtin_nontemporal_store(v, reinterpret_cast<f4*>(p));
}

// The same 16 bytes at an address that is only a multiple of 8 (rows of 4 k + 2 columns): global memory takes a
// four-dword store at any dword, so this is still one instruction.
__device__ __forceinline__ void store_nt4_align8(float* p, float a, float b, float c, float d) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  typedef f4 f4a8 __attribute__((aligned(8)));
  f4 v = {a, b, c, d};
  __builtin_nontemporal_store(v, reinterpret_cast<f4a8*>(p));
}

__device__ __forceinline__ void store4_align8(float* p, float a, float b, float c, float d) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  typedef f4 f4a8 __attribute__((aligned(8)));
  f4 v = {a, b, c, d};
  *reinterpret_cast<f4a8*>(p) = v;
}

// Stages the 128-column tile `tile` of VQ codebooks [n_cb][K][w] (w a multiple of 4) into LDS as
// [code][128 columns], columns from tile_cols on zero.  A thread issues UNROLL loads back to back
// before it waits for the first, so the 128 KB of a 256-code tile cost a few load latencies
// instead of one per element.  PAIR places column 8 j + 4 h + t at h * 64 + 4 j + t (the layout
// of the kernels that give one lane a whole 8-column code); with lg > 0 the lanes own their columns
// in groups of g = 2^lg (pair_pos).  With 16-byte aligned codebooks and tile_cols a multiple of 4 the
// loads are float4.
//
// pair_pos: where the PAIR layout keeps tile column c (a multiple of 4).  Lane j = g c' + k of a row owns the
// columns 8 g c' + 4 g h + 4 k + t (h = 0, 1; t < 4) and reads them at h * 64 + 4 j + t: g = 1 is a lane's own
// eight columns; with g = 4 (codebooks of 32 columns and more: the four lanes share their code) the h-th store
// instruction of a wave writes the 64 contiguous bytes 4 k + t of every group instead of 16 of every 32.
__device__ __forceinline__ int pair_pos(int c, int lg) {
  const int g1 = (1 << lg) - 1;
  const int j = ((c >> (3 + lg)) << lg) + ((c >> 2) & g1);
  return ((c >> (2 + lg)) & 1) * 64 + 4 * j;
}
template <int THREADS, bool PAIR>
__device__ __forceinline__ void stage_codebook_tile(float* __restrict__ s_cb, const float* __restrict__ codebooks,
                                                    int K, int w, int tile, int tile_cols, int lg = 0) {
  constexpr int UNROLL = 8;
  const bool vec = (reinterpret_cast<uintptr_t>(codebooks) & 15) == 0 && (tile_cols & 3) == 0 && (w & 3) == 0;
  if (vec) {
    const int n4 = K * 32;
    for (int i0 = threadIdx.x; i0 < n4; i0 += THREADS * UNROLL) {
      float4 v[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int i = i0 + u * THREADS;
        const int code = i >> 5, c = (i & 31) * 4;
        const bool on = i < n4 && c < tile_cols;
        const int col = tile * 128 + c;
        const int sub = col / w;
        const int64_t at = on ? ((int64_t)sub * K + code) * w + (col - sub * w) : 0;
        v[u] = *reinterpret_cast<const float4*>(codebooks + at);
        if (!on) v[u] = float4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int i = i0 + u * THREADS;
        const int code = i >> 5, c = (i & 31) * 4;
        const int pos = PAIR ? pair_pos(c, lg) : c;
        if (i < n4) *reinterpret_cast<float4*>(s_cb + (code << 7) + pos) = v[u];
      }
    }
    return;
  }
  const int n = K * 128;
  for (int i0 = threadIdx.x; i0 < n; i0 += THREADS * UNROLL) {
    float v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int i = i0 + u * THREADS;
      const int code = i >> 7, c = i & 127;
      const bool on = i < n && c < tile_cols;
      const int col = tile * 128 + c;
      const int sub = col / w;
      const int64_t at = on ? ((int64_t)sub * K + code) * w + (col - sub * w) : 0;
      v[u] = on ? codebooks[at] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int i = i0 + u * THREADS;
      const int code = i >> 7, c = i & 127;
      const int pos = PAIR ? pair_pos(c & ~3, lg) + (c & 3) : c;
      if (i < n) s_cb[(code << 7) + pos] = v[u];
    }
  }
}

// The same staging in two halves for a kernel that has other loads to issue while the tile is on
// its way: stage_codebook_load fills v[8] (K <= 256: one pass of eight float4 per thread of a
// 1024-thread workgroup), stage_codebook_store writes them to LDS.  Needs the float4 conditions of
// stage_codebook_tile (stage_codebook_vec_ok).
__device__ __forceinline__ bool stage_codebook_vec_ok(const float* codebooks, int w, int tile_cols) {
  return (reinterpret_cast<uintptr_t>(codebooks) & 15) == 0 && (tile_cols & 3) == 0 && (w & 3) == 0;
}
template <int THREADS>
__device__ __forceinline__ void stage_codebook_load(float4 (&v)[8], const float* __restrict__ codebooks, int K, int w,
                                                    int tile, int tile_cols) {
  const int n4 = K * 32;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int i = threadIdx.x + u * THREADS;
    const int code = i >> 5, c = (i & 31) * 4;
    const bool on = i < n4 && c < tile_cols;
    const int col = tile * 128 + c;
    const int sub = col / w;
    const int64_t at = on ? ((int64_t)sub * K + code) * w + (col - sub * w) : 0;
    v[u] = *reinterpret_cast<const float4*>(codebooks + at);
    if (!on) v[u] = float4{0.f, 0.f, 0.f, 0.f};
  }
}
template <int THREADS, bool PAIR>
__device__ __forceinline__ void stage_codebook_store(float* __restrict__ s_cb, const float4 (&v)[8], int K, int lg = 0) {
  const int n4 = K * 32;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int i = threadIdx.x + u * THREADS;
    const int code = i >> 5, c = (i & 31) * 4;
    const int pos = PAIR ? pair_pos(c, lg) : c;
    if (i < n4) *reinterpret_cast<float4*>(s_cb + (code << 7) + pos) = v[u];
  }
}

// Correctly rounded fp32 exp2 / log2: the fp64 library result rounded once.
__device__ __forceinline__ float exp2_cr(float x) { return (float)exp2((double)x); }
__device__ __forceinline__ float log2_cr(float x) { return (float)log2((double)x); }

// Decoded value of one log-domain SQ code (bits > 1).  `signed_code` is the code after
// removing the storage bias; fp32, product and sum rounded separately.
__device__ __forceinline__ float sq_log_decode(float signed_code, float k, float emin) {
  float v = signed_code + 0.5f;
  float s = v >= 0.f ? 1.f : -1.f;
  float t = __fadd_rn(__fmul_rn(fabsf(v), k), emin);
  return exp2_cr(t) * s;
}

}  // namespace f2cgt
