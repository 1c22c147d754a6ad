// Scalar quantisation: encode (log domain), decode (log domain via per-codebook LUT in
// LDS, or direct for 16 bits), and the per-column affine decode.
//
// All three are streaming kernels bounded by the fp32 side of the transfer
// (4 B per element against bits/8 B on the packed side).
#include "common.hpp"

namespace f2cgt {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxLutBytes = 64 * 1024;

int grid_for(int64_t items, int per_cu) {
  int64_t blocks = ceil_div(items, kBlock);
  int64_t cap = (int64_t)num_cus() * per_cu;
  return (int)(blocks < cap ? (blocks < 1 ? 1 : blocks) : cap);
}

// ---- encode -------------------------------------------------------------------
template <int BITS>
__global__ __launch_bounds__(kBlock) void sq_compress_kernel(const float* __restrict__ src,
                                                             float* __restrict__ dst,
                                                             const float* __restrict__ codebooks,
                                                             int64_t n, int64_t D,
                                                             int64_t column_slice,
                                                             int64_t num_codebooks) {
  const float drange = (float)(1 << (BITS - 1));
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const float x = src[i];
    if (BITS == 1) {
      dst[i] = x <= 0.f ? 0.f : 1.f;
      continue;
    }
    const int64_t col = i % D;
    int64_t cb = col / column_slice;
    cb = cb < num_codebooks ? cb : num_codebooks - 1;
    const float fmin = codebooks[cb * 5 + 0];
    const float fmax = codebooks[cb * 5 + 1];
    const float emin = codebooks[cb * 5 + 2];
    const float emax = codebooks[cb * 5 + 3];
    const bool neg = x <= 0.f;
    float v = fabsf(x);
    v = fminf(fmaxf(v, fmin), fmax);
    v = log2_cr(v);
    v = __fmul_rn(__fdiv_rn(__fsub_rn(v, emin), __fsub_rn(emax, emin)), drange);
    v = floorf(v);
    v = neg ? -1.f - v : v;
    if (BITS < 8) v += drange;
    dst[i] = v;
  }
}

// ---- log-domain decode ----------------------------------------------------------
// Raw stored bit pattern -> value, for one codebook (fmin,fmax,emin,emax,mean).
template <int BITS>
__device__ __forceinline__ float sq_log_value(uint32_t raw, const float* __restrict__ cb) {
  if (BITS == 1) return ((float)raw - 0.5f) * (2.f * cb[4]);
  const float drange = (float)(1 << (BITS - 1));
  const float emin = cb[2];
  const float k = __fdiv_rn(__fsub_rn(cb[3], emin), drange);
  float code;
  if (BITS < 8)
    code = (float)raw - drange;
  else if (BITS == 8)
    code = (float)(int8_t)raw;
  else
    code = (float)(int16_t)raw;
  return sq_log_decode(code, k, emin);
}

// One lane per packed byte (bits <= 8); LUT[num_codebooks][2^BITS] in LDS.
template <int BITS>
__global__ __launch_bounds__(kBlock) void sq_decompress_lut_kernel(
    const uint8_t* __restrict__ codes, float* __restrict__ out, const float* __restrict__ codebooks,
    int64_t rows, int64_t src_dim, int64_t feat_dim, int64_t column_slice, int num_codebooks) {
  constexpr int PER = 8 / BITS;
  constexpr int NCODE = 1 << BITS;
  constexpr uint32_t MASK = NCODE - 1;
  extern __shared__ float lut[];
  for (int t = threadIdx.x; t < num_codebooks * NCODE; t += kBlock)
    lut[t] = sq_log_value<BITS>((uint32_t)(t & MASK), codebooks + (int64_t)(t >> BITS) * 5);
  __syncthreads();

  const int64_t used = ceil_div(feat_dim, PER);  // packed bytes per row that hold output columns
  const int64_t n = rows * used;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / used;
    const int64_t j = i - r * used;
    const uint32_t byte = codes[r * src_dim + j];
    float* o = out + r * feat_dim;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int64_t col = j * PER + k;
      if (col < feat_dim) {
        int cb = (int)(col / column_slice);
        cb = cb < num_codebooks ? cb : num_codebooks - 1;
        o[col] = lut[cb * NCODE + ((byte >> (BITS * k)) & MASK)];
      }
    }
  }
}

// Direct evaluation (16-bit codes, or LUTs too large for LDS): one lane per output.
template <int BITS, typename CT>
__global__ __launch_bounds__(kBlock) void sq_decompress_direct_kernel(
    const CT* __restrict__ codes, float* __restrict__ out, const float* __restrict__ codebooks,
    int64_t rows, int64_t src_dim, int64_t feat_dim, int64_t column_slice, int num_codebooks) {
  constexpr int PER = BITS < 8 ? 8 / BITS : 1;
  constexpr uint32_t MASK = (BITS >= 16) ? 0xffffu : ((1u << BITS) - 1u);
  const int64_t n = rows * feat_dim;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / feat_dim;
    const int64_t col = i - r * feat_dim;
    const uint32_t word = (uint32_t)codes[r * src_dim + col / PER];
    const uint32_t raw = (word >> (BITS < 8 ? BITS * (int)(col % PER) : 0)) & MASK;
    int cb = (int)(col / column_slice);
    cb = cb < num_codebooks ? cb : num_codebooks - 1;
    out[i] = sq_log_value<BITS>(raw, codebooks + (int64_t)cb * 5);
  }
}

// ---- affine decode ------------------------------------------------------------
template <int BITS>
__global__ __launch_bounds__(kBlock) void sq_affine_decompress_kernel(
    const uint8_t* __restrict__ codes, float* __restrict__ out, const float* __restrict__ params,
    int64_t param_stride, int64_t rows, int64_t src_dim, int64_t feat_dim) {
  constexpr int PER = 8 / BITS;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  const int64_t used = ceil_div(feat_dim, PER);
  const int64_t n = rows * used;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / used;
    const int64_t j = i - r * used;
    const uint32_t byte = codes[r * src_dim + j];
    float* o = out + r * feat_dim;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int64_t col = j * PER + k;
      if (col < feat_dim) {
        const float code = (float)((byte >> (BITS * k)) & MASK);
        o[col] = __fadd_rn(params[col], __fmul_rn(code, params[param_stride + col]));
      }
    }
  }
}

template <int BITS>
int decompress_lut_launch(const uint8_t* codes, float* out, const float* codebooks, int64_t rows,
                          int64_t src_dim, int64_t feat_dim, int64_t column_slice, int n_cb,
                          hipStream_t st) {
  const int64_t items = rows * ceil_div(feat_dim, 8 / BITS);
  const size_t lds = (size_t)n_cb * (1 << BITS) * sizeof(float);
  sq_decompress_lut_kernel<BITS><<<grid_for(items, 8), kBlock, lds, st>>>(
      codes, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb);
  return launch_status("sq_decompress");
}

template <int BITS, typename CT>
int decompress_direct_launch(const void* codes, float* out, const float* codebooks, int64_t rows,
                             int64_t src_dim, int64_t feat_dim, int64_t column_slice, int n_cb,
                             hipStream_t st) {
  sq_decompress_direct_kernel<BITS, CT><<<grid_for(rows * feat_dim, 16), kBlock, 0, st>>>(
      static_cast<const CT*>(codes), out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb);
  return launch_status("sq_decompress");
}

}  // namespace
}  // namespace f2cgt

using namespace f2cgt;

extern "C" int f2cgt_sq_compress(const float* src, float* dst, const float* codebooks,
                                 int64_t rows, int64_t feat_dim, int64_t num_codebooks,
                                 int target_bits, int64_t column_slice, void* stream) {
  F2CGT_REQUIRE(rows >= 0 && feat_dim >= 0, F2CGT_E_INVALID, "sq_compress: negative size");
  F2CGT_REQUIRE(column_slice > 0 && num_codebooks > 0, F2CGT_E_INVALID,
                "sq_compress: column_slice and num_codebooks must be positive");
  F2CGT_REQUIRE(num_codebooks * column_slice >= feat_dim, F2CGT_E_INVALID,
                "sq_compress: %lld codebooks of %lld columns do not cover feat_dim %lld",
                (long long)num_codebooks, (long long)column_slice, (long long)feat_dim);
  const int64_t n = rows * feat_dim;
  if (n == 0) return 0;
  F2CGT_REQUIRE(src && dst && codebooks, F2CGT_E_INVALID, "sq_compress: null buffer");
  hipStream_t st = as_stream(stream);
  const int grid = grid_for(n, 16);
#define F2CGT_CASE(B)                                                                       \
  case B:                                                                                   \
    sq_compress_kernel<B><<<grid, kBlock, 0, st>>>(src, dst, codebooks, n, feat_dim,        \
                                                   column_slice, num_codebooks);            \
    break;
  switch (target_bits) {
    F2CGT_CASE(1) F2CGT_CASE(2) F2CGT_CASE(4) F2CGT_CASE(8) F2CGT_CASE(16)
    default:
      return fail(F2CGT_E_UNSUPPORTED, "sq_compress: target_bits must be 1,2,4,8 or 16 (got %d)",
                  target_bits);
  }
#undef F2CGT_CASE
  return launch_status("sq_compress");
}

extern "C" int f2cgt_sq_decompress(const void* codes, int code_dtype, float* out,
                                   const float* codebooks, int64_t rows, int64_t src_dim,
                                   int64_t feat_dim, int64_t num_codebooks, int target_bits,
                                   int64_t column_slice, void* stream) {
  F2CGT_REQUIRE(rows >= 0 && src_dim >= 0 && feat_dim >= 0, F2CGT_E_INVALID,
                "sq_decompress: negative size");
  F2CGT_REQUIRE(column_slice > 0 && num_codebooks > 0 && num_codebooks < (1 << 20), F2CGT_E_INVALID,
                "sq_decompress: column_slice and num_codebooks must be positive");
  F2CGT_REQUIRE(num_codebooks * column_slice >= feat_dim, F2CGT_E_INVALID,
                "sq_decompress: %lld codebooks of %lld columns do not cover feat_dim %lld",
                (long long)num_codebooks, (long long)column_slice, (long long)feat_dim);
  const bool byte_codes = code_dtype == F2CGT_DT_U8 || code_dtype == F2CGT_DT_I8;
  switch (target_bits) {
    case 1: case 2: case 4: case 8:
      F2CGT_REQUIRE(byte_codes, F2CGT_E_UNSUPPORTED,
                    "sq_decompress: %d-bit codes must be uint8 or int8", target_bits);
      F2CGT_REQUIRE(src_dim * (8 / target_bits) >= feat_dim, F2CGT_E_INVALID,
                    "sq_decompress: %lld packed bytes per row cannot hold %lld columns",
                    (long long)src_dim, (long long)feat_dim);
      break;
    case 16:
      F2CGT_REQUIRE(code_dtype == F2CGT_DT_I16, F2CGT_E_UNSUPPORTED,
                    "sq_decompress: 16-bit codes must be int16");
      F2CGT_REQUIRE(src_dim >= feat_dim, F2CGT_E_INVALID, "sq_decompress: src_dim < feat_dim");
      break;
    default:
      return fail(F2CGT_E_UNSUPPORTED, "sq_decompress: target_bits must be 1,2,4,8 or 16 (got %d)",
                  target_bits);
  }
  if (rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(codes && out && codebooks, F2CGT_E_INVALID, "sq_decompress: null buffer");
  hipStream_t st = as_stream(stream);
  const int n_cb = (int)num_codebooks;
  const uint8_t* c8 = static_cast<const uint8_t*>(codes);
  if (target_bits == 16)
    return decompress_direct_launch<16, uint16_t>(codes, out, codebooks, rows, src_dim, feat_dim,
                                                  column_slice, n_cb, st);
  const bool lut_fits = (int64_t)n_cb * (1 << target_bits) * 4 <= kMaxLutBytes;
  switch (target_bits) {
    case 1:
      return lut_fits ? decompress_lut_launch<1>(c8, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st)
                      : decompress_direct_launch<1, uint8_t>(codes, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st);
    case 2:
      return lut_fits ? decompress_lut_launch<2>(c8, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st)
                      : decompress_direct_launch<2, uint8_t>(codes, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st);
    case 4:
      return lut_fits ? decompress_lut_launch<4>(c8, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st)
                      : decompress_direct_launch<4, uint8_t>(codes, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st);
    default:
      return lut_fits ? decompress_lut_launch<8>(c8, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st)
                      : decompress_direct_launch<8, uint8_t>(codes, out, codebooks, rows, src_dim, feat_dim, column_slice, n_cb, st);
  }
}

extern "C" int f2cgt_sq_affine_decompress(const uint8_t* codes, float* out, const float* params,
                                          int64_t param_stride, int64_t rows, int64_t src_dim,
                                          int64_t feat_dim, int target_bits, void* stream) {
  F2CGT_REQUIRE(rows >= 0 && src_dim >= 0 && feat_dim >= 0, F2CGT_E_INVALID,
                "sq_affine_decompress: negative size");
  F2CGT_REQUIRE(target_bits == 1 || target_bits == 2 || target_bits == 4 || target_bits == 8,
                F2CGT_E_UNSUPPORTED, "sq_affine_decompress: target_bits must be 1,2,4 or 8 (got %d)",
                target_bits);
  F2CGT_REQUIRE(param_stride >= feat_dim, F2CGT_E_INVALID,
                "sq_affine_decompress: param_stride %lld < feat_dim %lld", (long long)param_stride,
                (long long)feat_dim);
  F2CGT_REQUIRE(src_dim * (8 / target_bits) >= feat_dim, F2CGT_E_INVALID,
                "sq_affine_decompress: %lld packed bytes per row cannot hold %lld columns",
                (long long)src_dim, (long long)feat_dim);
  if (rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(codes && out && params, F2CGT_E_INVALID, "sq_affine_decompress: null buffer");
  hipStream_t st = as_stream(stream);
  const int grid = grid_for(rows * ceil_div(feat_dim, 8 / target_bits), 16);
#define F2CGT_CASE(B)                                                                          \
  case B:                                                                                      \
    sq_affine_decompress_kernel<B><<<grid, kBlock, 0, st>>>(codes, out, params, param_stride, \
                                                            rows, src_dim, feat_dim);          \
    break;
  switch (target_bits) { F2CGT_CASE(1) F2CGT_CASE(2) F2CGT_CASE(4) F2CGT_CASE(8) }
#undef F2CGT_CASE
  return launch_status("sq_affine_decompress");
}
