// Vector-quantisation decode: out[i][j] = codebooks[j / w][codes[i][j / w]][j % w].
//
// A pure gather bounded by the fp32 output stream.  The codebook is staged once per
// workgroup in LDS (as fp32, whatever its storage type) when it fits; otherwise it is
// read through L1/L2.
#include "common.hpp"

namespace f2cgt {
namespace {

constexpr int kBlock = 512;
constexpr int64_t kMaxLdsBytes = 128 * 1024;

template <typename T> __device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }

template <typename CT, typename CBT, int VEC, bool USE_LDS>
__global__ __launch_bounds__(kBlock) void vq_decompress_kernel(
    const CT* __restrict__ codes, const CBT* __restrict__ codebooks, float* __restrict__ out,
    int64_t rows, int64_t feat_dim, int num_codebooks, int K, int w) {
  extern __shared__ float lds_cb[];
  if (USE_LDS) {
    const int total = num_codebooks * K * w;
    for (int t = threadIdx.x; t < total; t += kBlock) lds_cb[t] = to_f32(codebooks[t]);
    __syncthreads();
  }
  const int64_t vpr = feat_dim / VEC;
  const int64_t n = rows * vpr;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / vpr;
    const int col = (int)(i - r * vpr) * VEC;
    const int c = col / w;
    const int off = col - c * w;
    int code = (int)codes[r * num_codebooks + c];
    code = code < 0 ? 0 : (code >= K ? K - 1 : code);
    const int64_t e = ((int64_t)c * K + code) * w + off;
    float v[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) v[k] = USE_LDS ? lds_cb[e + k] : to_f32(codebooks[e + k]);
    float* o = out + r * feat_dim + col;
    if (VEC == 4) {
      *reinterpret_cast<float4*>(o) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) o[k] = v[k];
    }
  }
}

// ---- uint8 codes, fp32 codebooks, K <= 256, width dividing 128 ---------------------------
// One persistent 1024-thread workgroup per CU keeps a 128-column tile of the codebooks in LDS as
// [code][128 columns]: lane (t % 32) reads the 16 bytes at code * 512 + 16 * (t % 32), so the
// eight lanes that the LDS serves per clock always cover all 32 banks.  A lane owns one float4
// column group and takes eight rows (32 apart) per step: eight code-byte loads in flight, eight
// LDS reads, eight non-temporal float4 stores; the code bytes of the next step are loaded
// before the stores of the current one are issued.  Full steps run without predicates so the
// prefetch never has to wait for the stores behind it.
constexpr int kTileThreads = 1024;
constexpr int kTileRows = 256;   // rows per step: 32 lane groups x 8

struct VqTileArgs {
  const uint8_t* codes;
  const float* codebooks;
  float* out;
  int64_t rows;
  int feat_dim, n_cb, K, w;
  int n_tiles, n_stripes;
};

// HALF: rows of 4 k + 2 columns.  Output rows start at multiples of 8 bytes only, which a 16-byte store takes at any
// dword; the row's last column group holds two columns and stores them alone (the tile is staged up to the next
// multiple of four: the codebooks hold those columns, n_cb * w being a multiple of four that is at least feat_dim).
template <bool HALF>
__global__ __launch_bounds__(kTileThreads) void vq_decompress_tile_kernel(VqTileArgs a) {
  extern __shared__ __align__(16) float s_cb[];
  const int tile = blockIdx.x % a.n_tiles;
  const int stripe = blockIdx.x / a.n_tiles;
  const int tile_cols_out = (a.feat_dim - tile * 128) >= 128 ? 128 : (a.feat_dim - tile * 128);
  const int tile_cols = HALF ? (tile_cols_out + 3) & ~3 : tile_cols_out;
  stage_codebook_tile<kTileThreads, false>(s_cb, a.codebooks, a.K, a.w, tile, tile_cols);
  __syncthreads();
  const int c4 = threadIdx.x & 31;
  const int rs = threadIdx.x >> 5;
  if (c4 * 4 >= tile_cols) return;
  const int col0 = tile * 128 + c4 * 4;
  const uint8_t* cp = a.codes + col0 / a.w;
  const float* cbp = s_cb + c4 * 4;
  float* op = a.out + col0;
  const bool pair = HALF && c4 * 4 + 2 == tile_cols_out;   // the row's last two columns
  auto store = [&](float* dst, const float4& x) {
    if constexpr (HALF) {
      if (pair) store_nt2(dst, x.x, x.y);
      else store_nt4_align8(dst, x.x, x.y, x.z, x.w);
    } else {
      store_nt4(dst, x.x, x.y, x.z, x.w);
    }
  };
  const int64_t steps = a.rows / kTileRows;   // full steps
  const uint32_t kmax = (uint32_t)a.K - 1u;

  uint32_t code[8];
  int64_t s = stripe;
  if (s < steps) {
#pragma unroll
    for (int u = 0; u < 8; ++u) code[u] = cp[(s * kTileRows + rs + 32 * u) * a.n_cb];
  }
  for (; s < steps; s += a.n_stripes) {
    const int64_t sn = s + a.n_stripes < steps ? s + a.n_stripes : s;  // last step reloads itself
    uint32_t next[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) next[u] = cp[(sn * kTileRows + rs + 32 * u) * a.n_cb];
    float4 x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint32_t c = code[u] < kmax ? code[u] : kmax;
      x[u] = *reinterpret_cast<const float4*>(cbp + c * 128);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      store(op + (s * kTileRows + rs + 32 * u) * (int64_t)a.feat_dim, x[u]);
#pragma unroll
    for (int u = 0; u < 8; ++u) code[u] = next[u];
  }
  // the rows after the last full step, one stripe
  if (stripe == (int)(steps % a.n_stripes)) {
    for (int64_t r = steps * kTileRows + rs; r < a.rows; r += 32) {
      uint32_t c = cp[r * a.n_cb];
      c = c < kmax ? c : kmax;
      const float4 x = *reinterpret_cast<const float4*>(cbp + c * 128);
      store(op + r * (int64_t)a.feat_dim, x);
    }
  }
}

// Returns -1 when the shape is not covered.
int launch_tile(const uint8_t* codes, const float* codebooks, float* out, int64_t rows, int64_t feat_dim,
                int n_cb, int K, int w, hipStream_t st) {
  if (K > 256 || w < 4 || 128 % w != 0 || feat_dim % 2 != 0 || feat_dim < 64) return -1;
  if (!aligned(out, 16) || rows < 4 * kTileRows) return -1;
  VqTileArgs a{codes, codebooks, out, rows, (int)feat_dim, n_cb, K, w, 0, 0};
  a.n_tiles = (int)ceil_div(feat_dim, 128);
  const int cus = num_cus();
  if (a.n_tiles > cus) return -1;
  a.n_stripes = cus / a.n_tiles;
  const size_t lds = (size_t)K * 128 * 4;
  const bool half = feat_dim % 4 != 0;
  hipError_t e = hipFuncSetAttribute(half ? reinterpret_cast<const void*>(vq_decompress_tile_kernel<true>)
                                          : reinterpret_cast<const void*>(vq_decompress_tile_kernel<false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail((int)e, "vq_decompress: cannot reserve %zu B of LDS", lds);
  if (half) vq_decompress_tile_kernel<true><<<(unsigned)(a.n_stripes * a.n_tiles), kTileThreads, lds, st>>>(a);
  else vq_decompress_tile_kernel<false><<<(unsigned)(a.n_stripes * a.n_tiles), kTileThreads, lds, st>>>(a);
  return launch_status("vq_decompress");
}

template <typename CT, typename CBT>
int launch(const void* codes, const void* codebooks, float* out, int64_t rows, int64_t feat_dim,
           int n_cb, int K, int w, hipStream_t st) {
  const int64_t cb_bytes = (int64_t)n_cb * K * w * (int64_t)sizeof(float);
  const bool use_lds = cb_bytes <= kMaxLdsBytes;
  const bool vec4 = (w % 4 == 0) && (feat_dim % 4 == 0) && aligned(out, 16);
  const int64_t items = rows * (vec4 ? feat_dim / 4 : feat_dim);
  int64_t blocks = ceil_div(items, kBlock);
  int per_cu = use_lds ? (int)(kMaxLdsBytes / (cb_bytes > 32 * 1024 ? cb_bytes : 32 * 1024)) : 4;
  int64_t cap = (int64_t)num_cus() * (per_cu < 1 ? 1 : per_cu);
  const int grid = (int)(blocks < cap ? blocks : cap);
  const CT* c = static_cast<const CT*>(codes);
  const CBT* cb = static_cast<const CBT*>(codebooks);
#define F2CGT_GO(V, L)                                                                          \
  do {                                                                                          \
    auto kern = vq_decompress_kernel<CT, CBT, V, L>;                                            \
    if (L && cb_bytes > 48 * 1024) {                                                            \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                   \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)cb_bytes); \
      if (e != hipSuccess) return fail((int)e, "vq_decompress: cannot reserve %lld B of LDS",   \
                                       (long long)cb_bytes);                                    \
    }                                                                                           \
    kern<<<grid, kBlock, L ? (size_t)cb_bytes : 0, st>>>(c, cb, out, rows, feat_dim, n_cb, K, w); \
  } while (0)
  if (use_lds) {
    if (vec4) F2CGT_GO(4, true); else F2CGT_GO(1, true);
  } else {
    if (vec4) F2CGT_GO(4, false); else F2CGT_GO(1, false);
  }
#undef F2CGT_GO
  return launch_status("vq_decompress");
}

}  // namespace
}  // namespace f2cgt

using namespace f2cgt;

extern "C" int f2cgt_vq_decompress(const void* codes, int code_dtype, const void* codebooks,
                                   int cb_dtype, float* out, int64_t rows, int64_t feat_dim,
                                   int64_t num_codebooks, int64_t K, int64_t width, void* stream) {
  F2CGT_REQUIRE(rows >= 0 && feat_dim >= 0, F2CGT_E_INVALID, "vq_decompress: negative size");
  F2CGT_REQUIRE(num_codebooks > 0 && K > 0 && width > 0, F2CGT_E_INVALID,
                "vq_decompress: codebooks must be [n>0, K>0, w>0]");
  F2CGT_REQUIRE(num_codebooks * K * width < (1ll << 31) && feat_dim < (1ll << 31), F2CGT_E_UNSUPPORTED,
                "vq_decompress: codebook or feat_dim too large");
  F2CGT_REQUIRE(feat_dim <= num_codebooks * width, F2CGT_E_INVALID,
                "vq_decompress: feat_dim %lld exceeds %lld codebooks x width %lld", (long long)feat_dim,
                (long long)num_codebooks, (long long)width);
  F2CGT_REQUIRE(cb_dtype == F2CGT_DT_F32 || cb_dtype == F2CGT_DT_F16, F2CGT_E_UNSUPPORTED,
                "vq_decompress: codebooks must be float32 or float16");
  if (rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(codes && out && codebooks, F2CGT_E_INVALID, "vq_decompress: null buffer");
  hipStream_t st = as_stream(stream);
  const int n_cb = (int)num_codebooks, k = (int)K, w = (int)width;
  const bool f32 = cb_dtype == F2CGT_DT_F32;
  if (code_dtype == F2CGT_DT_U8 && f32) {
    const int rc = launch_tile(static_cast<const uint8_t*>(codes), static_cast<const float*>(codebooks), out, rows,
                               feat_dim, n_cb, k, w, st);
    if (rc >= 0) return rc;
  }
  switch (code_dtype) {
    case F2CGT_DT_U8:
      return f32 ? launch<uint8_t, float>(codes, codebooks, out, rows, feat_dim, n_cb, k, w, st)
                 : launch<uint8_t, __half>(codes, codebooks, out, rows, feat_dim, n_cb, k, w, st);
    case F2CGT_DT_I8:
      return f32 ? launch<int8_t, float>(codes, codebooks, out, rows, feat_dim, n_cb, k, w, st)
                 : launch<int8_t, __half>(codes, codebooks, out, rows, feat_dim, n_cb, k, w, st);
    case F2CGT_DT_I16:
      return f32 ? launch<int16_t, float>(codes, codebooks, out, rows, feat_dim, n_cb, k, w, st)
                 : launch<int16_t, __half>(codes, codebooks, out, rows, feat_dim, n_cb, k, w, st);
    default:
      return fail(F2CGT_E_UNSUPPORTED, "vq_decompress: codes must be uint8, int8 or int16");
  }
}
