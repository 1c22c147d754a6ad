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
// Bucket floor(g(L)) of a clamped magnitude v, L = correctly rounded fp32 log2(v).
template <int BITS>
__device__ __forceinline__ float sq_bucket_exact(float v, float emin, float span) {
  const float drange = (float)(1 << (BITS - 1));
  return floorf(__fmul_rn(__fdiv_rn(__fsub_rn(log2_cr(v), emin), span), drange));
}

// The same bucket without the fp64 logarithm, for most values: g is non-decreasing and the
// hardware log2 is within a few ulp of L, so when an error bound below and above the approximate g
// lands in one bucket (b_lo == b_hi) that bucket is exact; the caller sends only the values next
// to a bucket edge to sq_bucket_exact.  v must be a normal number; k = fl(2^(BITS-1) / span).
//
// With L the fp32 logarithm the exact chain starts from, that chain gives
// u = (L - emin) / span * 2^(BITS-1) with two roundings (the power of two is exact); the product t
// below is the same expression at the hardware logarithm with three.  So
// |u - t| <= |L - approx| * k + 6 * 2^-24 * |t|, and `mt` bounds that with room to spare for its
// own roundings; floor is monotone, so floor(u) lies between the two floors returned.
__device__ __forceinline__ void sq_bucket_bounds(float v, float emin, float k, float& b_lo, float& b_hi) {
  const float approx = __builtin_amdgcn_logf(v);
  const float m_log = fmaf(fabsf(approx), 1.0e-6f, 2.0e-7f);   // > 8 ulp, and 2^-22 absolute next to log = 0
  const float t = __fmul_rn(__fsub_rn(approx, emin), k);
  const float mt = fmaf(fabsf(t), 1.0e-6f, m_log * k * 1.001f);
  b_lo = floorf(t - mt);
  b_hi = floorf(t + mt);
}

// Code of one element as the float the encoder returns (src/sq_quantization.cu:33-60).
template <int BITS>
__device__ __forceinline__ float sq_code_of(float x, const float* __restrict__ cb) {
  if (BITS == 1) return x <= 0.f ? 0.f : 1.f;
  const float drange = (float)(1 << (BITS - 1));
  const float fmin = cb[0], fmax = cb[1], emin = cb[2], emax = cb[3];
  const bool neg = x <= 0.f;
  float v = fabsf(x);
  v = fminf(fmaxf(v, fmin), fmax);
  v = sq_bucket_exact<BITS>(v, emin, __fsub_rn(emax, emin));
  v = neg ? -1.f - v : v;
  if (BITS < 8) v += drange;
  return v;
}

// Encode straight to the storage form: what `packbits(uint8(sq_compress(x)))` (bits < 8),
// `int8(sq_compress(x))` or `int16(sq_compress(x))` give, in one pass over the fp32 input.  One
// lane per stored element (a packed byte covers 8 / bits columns).
template <int BITS, typename OT>
__global__ __launch_bounds__(kBlock) void sq_encode_kernel(const float* __restrict__ src, OT* __restrict__ dst,
                                                           const float* __restrict__ codebooks, int64_t rows,
                                                           int64_t D, int64_t dst_dim, int64_t column_slice,
                                                           int64_t num_codebooks) {
  constexpr int PER = BITS < 8 ? 8 / BITS : 1;
  const int64_t n = rows * dst_dim;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / dst_dim;
    const int64_t j = i - r * dst_dim;
    uint32_t packed = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int64_t col = j * PER + k;
      if (col < D) {
        int64_t cb = col / column_slice;
        cb = cb < num_codebooks ? cb : num_codebooks - 1;
        const float c = sq_code_of<BITS>(src[r * D + col], codebooks + cb * 5);
        if (BITS < 8)
          packed |= ((uint32_t)(int)c & ((1u << BITS) - 1u)) << (BITS * k);
        else
          packed = (uint32_t)(int)c;
      }
    }
    dst[i] = (OT)packed;
  }
}

template <int BITS>
__global__ __launch_bounds__(kBlock) void sq_compress_kernel(const float* __restrict__ src,
                                                             float* __restrict__ dst,
                                                             const float* __restrict__ codebooks,
                                                             int64_t n, int64_t D,
                                                             int64_t column_slice,
                                                             int64_t num_codebooks) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t col = i % D;
    int64_t cb = col / column_slice;
    cb = cb < num_codebooks ? cb : num_codebooks - 1;
    dst[i] = sq_code_of<BITS>(src[i], codebooks + cb * 5);
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

// ---- float4-per-lane streaming decoders ------------------------------------------------
// Both decoders above walk the packed side (one lane per byte, scalar stores).  When rows are
// whole float4 groups the output side can drive instead: one lane per output float4, eight
// float4 per lane, a workgroup writes one dense 32 KB span with non-temporal stores, and the
// (row, column group) of an item comes from a 32-bit multiply-high instead of a 64-bit divide.
// The lane loads exactly the code bits of its four columns (1-4 bytes, byte granular).
constexpr int kF4Items = 8;

struct F4Args {
  const uint8_t* codes;
  float* out;
  const float* table;     // affine: params [2, param_stride]; log domain: codebooks [n_cb, 5]
  int64_t param_stride;
  int64_t column_slice;
  int n_cb;
  int64_t src_dim;
  int64_t total_f4;
  uint32_t f4_per_row;
  uint32_t magic;         // ceil(2^32 / f4_per_row)
  int feat_dim;           // sq_decode_pairs_kernel: columns of a row
};

template <int BITS, bool AFFINE>
__global__ __launch_bounds__(kBlock) void sq_decode_f4_kernel(F4Args a) {
  constexpr int NCODE = 1 << BITS;
  constexpr uint32_t MASK = NCODE - 1;
  extern __shared__ __align__(16) float s_tab[];
  // affine: [f4][mn x4, scale x4]; log domain: LUT [n_cb][NCODE], then the codebook of each column
  const int feat_dim = (int)a.f4_per_row * 4;
  int* s_cbi = reinterpret_cast<int*>(s_tab + ((a.n_cb * NCODE + 3) & ~3));
  if (AFFINE) {
    for (int i = threadIdx.x; i < feat_dim; i += kBlock) {
      s_tab[(i >> 2) * 8 + (i & 3)] = a.table[i];
      s_tab[(i >> 2) * 8 + 4 + (i & 3)] = a.table[a.param_stride + i];
    }
  } else {
    for (int i = threadIdx.x; i < a.n_cb * NCODE; i += kBlock)
      s_tab[i] = sq_log_value<BITS>((uint32_t)(i & MASK), a.table + (int64_t)(i >> BITS) * 5);
    for (int i = threadIdx.x; i < feat_dim; i += kBlock) {
      int64_t cb = i / a.column_slice;
      cb = cb < a.n_cb ? cb : a.n_cb - 1;
      s_cbi[i] = (int)cb * NCODE;
    }
  }
  __syncthreads();

  const int64_t base = (int64_t)blockIdx.x * (kF4Items * kBlock);
  // first row of the span: floor(base / f4_per_row), from the fp64 quotient and a fix-up
  int64_t rb = (int64_t)((double)base / (double)a.f4_per_row);
  if (rb * a.f4_per_row > base) --rb;
  if ((rb + 1) * (int64_t)a.f4_per_row <= base) ++rb;
  const uint32_t cb0 = (uint32_t)(base - rb * a.f4_per_row);

  uint32_t word[kF4Items], c4s[kF4Items];
#pragma unroll
  for (int k = 0; k < kF4Items; ++k) {
    const uint32_t li = cb0 + threadIdx.x + k * kBlock;
    const uint32_t rl = __umulhi(li, a.magic);
    const uint32_t c4 = li - rl * a.f4_per_row;
    const bool on = base + threadIdx.x + k * kBlock < a.total_f4;
    const uint8_t* src = a.codes + (on ? (rb + rl) * a.src_dim : 0);
    c4s[k] = c4;
    if (BITS == 8) {
      uint32_t w; __builtin_memcpy(&w, src + (on ? 4 * c4 : 0), 4); word[k] = w;
    } else if (BITS == 4) {
      uint16_t w; __builtin_memcpy(&w, src + (on ? 2 * c4 : 0), 2); word[k] = w;
    } else if (BITS == 2) {
      word[k] = src[on ? c4 : 0];
    } else {
      word[k] = (src[on ? (c4 >> 1) : 0] >> ((c4 & 1) * 4)) & 0xfu;
    }
  }
#pragma unroll
  for (int k = 0; k < kF4Items; ++k) {
    const int64_t i = base + threadIdx.x + k * kBlock;
    if (i >= a.total_f4) break;
    const uint32_t c4 = c4s[k];
    float v[4];
    if (AFFINE) {
      const float4 mn = *reinterpret_cast<const float4*>(s_tab + c4 * 8);
      const float4 sc = *reinterpret_cast<const float4*>(s_tab + c4 * 8 + 4);
      v[0] = __fadd_rn(mn.x, __fmul_rn((float)(word[k] & MASK), sc.x));
      v[1] = __fadd_rn(mn.y, __fmul_rn((float)((word[k] >> BITS) & MASK), sc.y));
      v[2] = __fadd_rn(mn.z, __fmul_rn((float)((word[k] >> (2 * BITS)) & MASK), sc.z));
      v[3] = __fadd_rn(mn.w, __fmul_rn((float)((word[k] >> (3 * BITS)) & MASK), sc.w));
    } else {
      const int4 cbi = *reinterpret_cast<const int4*>(s_cbi + c4 * 4);
      v[0] = s_tab[cbi.x + (word[k] & MASK)];
      v[1] = s_tab[cbi.y + ((word[k] >> BITS) & MASK)];
      v[2] = s_tab[cbi.z + ((word[k] >> (2 * BITS)) & MASK)];
      v[3] = s_tab[cbi.w + ((word[k] >> (3 * BITS)) & MASK)];
    }
    store_nt4(a.out + i * 4, v[0], v[1], v[2], v[3]);
  }
}

// Rows of 4 k + 2 columns, decoded through a flat view of the output: the matrix as a whole is still a run of
// 16-byte pieces (rows * feat_dim is a multiple of 4 when the row count is even; an odd count leaves one pair),
// and a piece is two column pairs, of one row or of the end of a row and the start of the next.  A lane owns
// a piece: two (row, pair) positions from one multiply-high each, the code bits of the two pairs (2 / 1 bytes,
// a nibble, two bits), the per-column tables from LDS, and one aligned 16-byte store, so that the stores of a
// workgroup are as dense as for rows of whole float4 groups (4e5 rows of 602 columns, 4 bit: 253 us with a group of
// four columns per lane and stores that start 8 bytes off, 176 us at 600 columns).
template <int BITS, bool AFFINE>
__global__ __launch_bounds__(kBlock) void sq_decode_pairs_kernel(F4Args a) {
  constexpr int NCODE = 1 << BITS;
  constexpr uint32_t MASK = NCODE - 1;
  extern __shared__ __align__(16) float s_tab[];
  // affine: [column][min, scale]; log domain: LUT [n_cb][NCODE], then the LUT base of each column
  int* s_cbi = reinterpret_cast<int*>(s_tab + ((a.n_cb * NCODE + 3) & ~3));
  if (AFFINE) {
    for (int i = threadIdx.x; i < a.feat_dim; i += kBlock) {
      s_tab[2 * i] = a.table[i];
      s_tab[2 * i + 1] = a.table[a.param_stride + i];
    }
  } else {
    for (int i = threadIdx.x; i < a.n_cb * NCODE; i += kBlock)
      s_tab[i] = sq_log_value<BITS>((uint32_t)(i & MASK), a.table + (int64_t)(i >> BITS) * 5);
    for (int i = threadIdx.x; i < a.feat_dim; i += kBlock) {
      int64_t cb = i / a.column_slice;
      cb = cb < a.n_cb ? cb : a.n_cb - 1;
      s_cbi[i] = (int)cb * NCODE;
    }
  }
  __syncthreads();
  const uint32_t ppr = a.f4_per_row;             // pairs per row (feat_dim / 2)
  const int64_t total_pairs = a.total_f4;        // rows * pairs per row
  const int64_t base = (int64_t)blockIdx.x * (kF4Items * kBlock);
  // first row of the workgroup's span of pairs: floor(2 base / ppr), from the fp64 quotient and a fix-up; the pairs
  // of the span are then counted from that row's first, small enough for the 32-bit multiply-high to be exact
  int64_t rb = (int64_t)((double)(2 * base) / (double)ppr);
  if (rb * ppr > 2 * base) --rb;
  if ((rb + 1) * (int64_t)ppr <= 2 * base) ++rb;
  const uint32_t l0 = (uint32_t)(2 * base - rb * ppr);
  auto pair = [&](int64_t p, float& v0, float& v1) {
    const uint32_t li = l0 + (uint32_t)(p - 2 * base);
    const uint32_t rl = __umulhi(li, a.magic);
    const uint32_t cp = li - rl * ppr;
    const uint8_t* src = a.codes + (rb + rl) * a.src_dim;
    uint32_t c0, c1;
    if (BITS == 8) {
      uint16_t w; __builtin_memcpy(&w, src + 2 * cp, 2);
      c0 = w & 0xffu; c1 = w >> 8;
    } else if (BITS == 4) {
      const uint32_t w = src[cp];
      c0 = w & 0xfu; c1 = w >> 4;
    } else if (BITS == 2) {
      const uint32_t w = src[cp >> 1] >> ((cp & 1) * 4);
      c0 = w & 3u; c1 = (w >> 2) & 3u;
    } else {
      const uint32_t w = src[cp >> 2] >> ((cp & 3) * 2);
      c0 = w & 1u; c1 = (w >> 1) & 1u;
    }
    const uint32_t col = 2 * cp;
    if (AFFINE) {
      const float4 t = *reinterpret_cast<const float4*>(s_tab + 2 * col);   // min, scale of the two columns
      v0 = __fadd_rn(t.x, __fmul_rn((float)c0, t.y));
      v1 = __fadd_rn(t.z, __fmul_rn((float)c1, t.w));
    } else {
      const int2 cbi = *reinterpret_cast<const int2*>(s_cbi + col);
      v0 = s_tab[cbi.x + c0];
      v1 = s_tab[cbi.y + c1];
    }
  };
  const int64_t n4 = total_pairs >> 1;
#pragma unroll
  for (int k = 0; k < kF4Items; ++k) {
    const int64_t i = base + threadIdx.x + k * kBlock;
    if (i < n4) {
      float v[4];
      pair(2 * i, v[0], v[1]);
      pair(2 * i + 1, v[2], v[3]);
      store_nt4(a.out + 4 * i, v[0], v[1], v[2], v[3]);
    } else if (i == n4 && (total_pairs & 1)) {   // an odd number of rows: the matrix ends with one pair
      float v0, v1;
      pair(2 * i, v0, v1);
      store_nt2(a.out + 4 * i, v0, v1);
    }
  }
}

// Launches the float4 decoder when the shape allows it; returns -1 when it does not.
template <int BITS, bool AFFINE>
int decode_f4_launch(const uint8_t* codes, float* out, const float* table, int64_t param_stride,
                     int64_t column_slice, int n_cb, int64_t rows, int64_t src_dim, int64_t feat_dim,
                     hipStream_t st, const char* what) {
  // (one float4 per row would need the reciprocal 2^32, which does not fit the 32-bit multiplier)
  if (feat_dim % 2 != 0 || feat_dim < 8 || feat_dim > 8192 || !aligned(out, 16)) return -1;
  const size_t lds = AFFINE ? (size_t)feat_dim * 8
                            : ((((size_t)n_cb << BITS) + 3) / 4 * 4 + (size_t)feat_dim) * 4;
  if (lds > (size_t)kMaxLutBytes) return -1;
  F4Args a{};
  a.codes = codes; a.out = out; a.table = table;
  a.param_stride = param_stride; a.column_slice = column_slice; a.n_cb = AFFINE ? 0 : n_cb;
  a.src_dim = src_dim;
  a.feat_dim = (int)feat_dim;
  // items per row: float4 groups, or column pairs for rows of 4 k + 2 columns (the flat view: two pairs per lane,
  // plus one lane for the last pair of an odd number of rows)
  const bool pairs = feat_dim % 4 != 0;
  a.f4_per_row = (uint32_t)(pairs ? feat_dim / 2 : feat_dim / 4);
  a.total_f4 = rows * a.f4_per_row;
  a.magic = (uint32_t)((0x100000000ull + a.f4_per_row - 1) / a.f4_per_row);
  const int64_t lanes = pairs ? a.total_f4 / 2 + 1 : a.total_f4;
  const int64_t grid = ceil_div(lanes, kF4Items * kBlock);
  if (grid > 0x7fffffffll) return -1;
  if (pairs) sq_decode_pairs_kernel<BITS, AFFINE><<<(unsigned)grid, kBlock, lds, st>>>(a);
  else sq_decode_f4_kernel<BITS, AFFINE><<<(unsigned)grid, kBlock, lds, st>>>(a);
  return launch_status(what);
}

// ---- float4-per-lane encoders ----------------------------------------------------------------
// Same indexing as the float4 decoders: a lane takes four consecutive columns of a row (eight
// for 1-bit storage, so that it owns a whole byte), the codebook of each column comes from a
// small table in LDS, and the result goes out as one float4 (codes as fp32, the reference form)
// or as the 1-4 bytes of the storage form.
template <int BITS, bool STORAGE, bool SINGLE>
__global__ __launch_bounds__(kBlock) void sq_encode_f4_kernel(F4Args a, const float* __restrict__ src,
                                                              void* __restrict__ dst) {
  constexpr int COLS = (STORAGE && BITS == 1) ? 8 : 4;   // columns per lane
  extern __shared__ __align__(16) float s_tab[];
  // per codebook: fmin, fmax, emin, 2^(BITS-1)/span, bucket(fmin), bucket(fmax), span (+1 pad); then the table
  // offset of every column.  Values clamped to fmin / fmax (about 1 % of a table by construction
  // of the codebooks) sit exactly on a bucket edge, so their buckets are evaluated once, exactly.
  float* s_cb = s_tab;
  int* s_cbi = reinterpret_cast<int*>(s_tab + a.n_cb * 8);
  const int feat_dim = (int)a.f4_per_row * COLS;
  for (int i = threadIdx.x; i < a.n_cb; i += kBlock) {
    const float* cb = a.table + (int64_t)i * 5;
    const float span = __fsub_rn(cb[3], cb[2]);
    s_cb[i * 8 + 0] = cb[0];
    s_cb[i * 8 + 1] = cb[1];
    s_cb[i * 8 + 2] = cb[2];
    s_cb[i * 8 + 3] = __fdiv_rn((float)(1 << (BITS - 1)), span);
    s_cb[i * 8 + 4] = BITS == 1 ? 0.f : sq_bucket_exact<BITS>(fminf(fmaxf(cb[0], cb[0]), cb[1]), cb[2], span);
    s_cb[i * 8 + 5] = BITS == 1 ? 0.f : sq_bucket_exact<BITS>(fminf(fmaxf(cb[1], cb[0]), cb[1]), cb[2], span);
    s_cb[i * 8 + 6] = span;
  }
  for (int i = threadIdx.x; i < feat_dim; i += kBlock) {
    int64_t cb = i / a.column_slice;
    cb = cb < a.n_cb ? cb : a.n_cb - 1;
    s_cbi[i] = (int)cb * 8;
  }
  __syncthreads();
  // Codes of four columns.  The common part runs without a branch for all four; the columns whose
  // error bound straddles a bucket edge are collected in a mask and take the exact path in one
  // rolled loop, so the fp64 logarithm exists once in the code, not once per column.
  auto code4 = [&](const float4 xv, const int4 tabs, float* c) {
    const float xs[4] = {xv.x, xv.y, xv.z, xv.w};
    if (BITS == 1) {
#pragma unroll
      for (int e = 0; e < 4; ++e) c[e] = xs[e] <= 0.f ? 0.f : 1.f;
      return;
    }
    const float drange = (float)(1 << (BITS - 1));
    const int tb[4] = {SINGLE ? 0 : tabs.x, SINGLE ? 0 : tabs.y, SINGLE ? 0 : tabs.z, SINGLE ? 0 : tabs.w};
    float m[4], bkt[4];
    uint32_t need = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float4 q = *reinterpret_cast<const float4*>(s_cb + tb[e]);      // fmin, fmax, emin, 2^(BITS-1)/span
      const float2 cl = *reinterpret_cast<const float2*>(s_cb + tb[e] + 4);  // bucket(fmin), bucket(fmax)
      m[e] = fabsf(xs[e]);
      float b_lo, b_hi;
      sq_bucket_bounds(m[e], q.z, q.w, b_lo, b_hi);
      const bool at_min = !(m[e] > q.x);        // clamps to fmin (NaN too: the reference's fmaxf picks fmin)
      const bool at_max = m[e] >= q.y;
      bkt[e] = at_min ? cl.x : at_max ? cl.y : b_lo;
      need |= (!at_min && !at_max && !(b_lo == b_hi)) ? 1u << e : 0u;
    }
    if (need) {
#pragma nounroll
      for (int e = 0; e < 4; ++e) {
        if (!((need >> e) & 1u)) continue;
        const float me = e == 0 ? m[0] : e == 1 ? m[1] : e == 2 ? m[2] : m[3];
        const int te = e == 0 ? tb[0] : e == 1 ? tb[1] : e == 2 ? tb[2] : tb[3];
        const float r = sq_bucket_exact<BITS>(me, s_cb[te + 2], s_cb[te + 6]);
#pragma unroll
        for (int j = 0; j < 4; ++j) bkt[j] = e == j ? r : bkt[j];
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float v = xs[e] <= 0.f ? -1.f - bkt[e] : bkt[e];
      if (BITS < 8) v += drange;
      c[e] = v;
    }
  };
  const int64_t base = (int64_t)blockIdx.x * (kF4Items * kBlock);
  int64_t rb = (int64_t)((double)base / (double)a.f4_per_row);
  if (rb * a.f4_per_row > base) --rb;
  if ((rb + 1) * (int64_t)a.f4_per_row <= base) ++rb;
  const uint32_t cb0 = (uint32_t)(base - rb * a.f4_per_row);
  float4 x[kF4Items][COLS / 4];
#pragma unroll
  for (int k = 0; k < kF4Items; ++k) {
    const int64_t i = base + threadIdx.x + k * kBlock;
    const float4* p = reinterpret_cast<const float4*>(src) + (i < a.total_f4 ? i : 0) * (COLS / 4);
#pragma unroll
    for (int h = 0; h < COLS / 4; ++h) x[k][h] = p[h];
  }
#pragma unroll
  for (int k = 0; k < kF4Items; ++k) {
    const int64_t i = base + threadIdx.x + k * kBlock;
    if (i >= a.total_f4) break;
    const uint32_t li = cb0 + threadIdx.x + k * kBlock;
    const uint32_t rl = __umulhi(li, a.magic);
    const uint32_t g = li - rl * a.f4_per_row;            // column group of the row
    float c[COLS];
#pragma unroll
    for (int h = 0; h < COLS / 4; ++h) {
      int4 cbi = {0, 0, 0, 0};
      if (!SINGLE) cbi = *reinterpret_cast<const int4*>(s_cbi + g * COLS + 4 * h);
      code4(x[k][h], cbi, c + 4 * h);
    }
    if (!STORAGE) {
      store_nt4(static_cast<float*>(dst) + i * 4, c[0], c[1], c[2], c[3]);
    } else if (BITS == 16) {
      typedef short s4 __attribute__((ext_vector_type(4)));
      s4 v = {(short)(int)c[0], (short)(int)c[1], (short)(int)c[2], (short)(int)c[3]};
      __builtin_nontemporal_store(v, static_cast<s4*>(dst) + i);
    } else {
      uint32_t packed = 0;
      constexpr int FIELD = BITS;                          // 8-bit codes: one byte each
#pragma unroll
      for (int q = 0; q < COLS; ++q) packed |= ((uint32_t)(int)c[q] & ((1u << FIELD) - 1u)) << (FIELD * q);
      // storage bytes of the lane: COLS * BITS / 8, at the same offset in every row pitch
      uint8_t* o = static_cast<uint8_t*>(dst) + (rb + rl) * a.src_dim + (int64_t)g * (COLS * BITS / 8);
      if (COLS * BITS == 32) { __builtin_memcpy(o, &packed, 4); }
      else if (COLS * BITS == 16) { const uint16_t h2 = (uint16_t)packed; __builtin_memcpy(o, &h2, 2); }
      else *o = (uint8_t)packed;
    }
  }
}

// Launches the float4 encoder when the shape allows it; returns -1 when it does not.
template <int BITS, bool STORAGE>
int encode_f4_launch(const float* src, void* dst, const float* codebooks, int64_t column_slice, int n_cb,
                     int64_t rows, int64_t feat_dim, int64_t dst_dim, hipStream_t st, const char* what) {
  constexpr int COLS = (STORAGE && BITS == 1) ? 8 : 4;
  // (one lane per row would need the reciprocal 2^32, which does not fit the 32-bit multiplier)
  if (feat_dim % COLS != 0 || feat_dim < 2 * COLS || feat_dim > 8192 || !aligned(src, 16) ||
      (!STORAGE && !aligned(dst, 16)) ||
      (STORAGE && BITS == 16 && !aligned(dst, 8)))
    return -1;
  F4Args a{};
  a.table = codebooks;
  a.column_slice = column_slice;
  a.n_cb = n_cb;
  a.src_dim = dst_dim;                       // bytes per storage row
  a.f4_per_row = (uint32_t)(feat_dim / COLS);
  a.total_f4 = rows * (feat_dim / COLS);
  a.magic = (uint32_t)((0x100000000ull + a.f4_per_row - 1) / a.f4_per_row);
  const int64_t grid = ceil_div(a.total_f4, kF4Items * kBlock);
  if (grid > 0x7fffffffll) return -1;
  const size_t lds = ((size_t)n_cb * 8 + (size_t)feat_dim) * 4;
  if (lds > (size_t)kMaxLutBytes) return -1;
  if (n_cb == 1) sq_encode_f4_kernel<BITS, STORAGE, true><<<(unsigned)grid, kBlock, lds, st>>>(a, src, dst);
  else sq_encode_f4_kernel<BITS, STORAGE, false><<<(unsigned)grid, kBlock, lds, st>>>(a, src, dst);
  return launch_status(what);
}

template <int BITS>
int decompress_lut_launch(const uint8_t* codes, float* out, const float* codebooks, int64_t rows,
                          int64_t src_dim, int64_t feat_dim, int64_t column_slice, int n_cb,
                          hipStream_t st) {
  const int rc = decode_f4_launch<BITS, false>(codes, out, codebooks, 0, column_slice, n_cb, rows, src_dim,
                                               feat_dim, st, "sq_decompress");
  if (rc >= 0) return rc;
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
  {
    int rc = -1;
    const int ncb = (int)num_codebooks;
    switch (target_bits) {
      case 1: rc = encode_f4_launch<1, false>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, 0, st, "sq_compress"); break;
      case 2: rc = encode_f4_launch<2, false>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, 0, st, "sq_compress"); break;
      case 4: rc = encode_f4_launch<4, false>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, 0, st, "sq_compress"); break;
      case 8: rc = encode_f4_launch<8, false>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, 0, st, "sq_compress"); break;
      case 16: rc = encode_f4_launch<16, false>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, 0, st, "sq_compress"); break;
      default: break;
    }
    if (rc >= 0) return rc;
  }
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

extern "C" int f2cgt_sq_encode(const float* src, void* dst, const float* codebooks, int64_t rows,
                               int64_t feat_dim, int64_t num_codebooks, int target_bits,
                               int64_t column_slice, void* stream) {
  F2CGT_REQUIRE(rows >= 0 && feat_dim >= 0, F2CGT_E_INVALID, "sq_encode: negative size");
  F2CGT_REQUIRE(column_slice > 0 && num_codebooks > 0, F2CGT_E_INVALID,
                "sq_encode: column_slice and num_codebooks must be positive");
  F2CGT_REQUIRE(num_codebooks * column_slice >= feat_dim, F2CGT_E_INVALID,
                "sq_encode: %lld codebooks of %lld columns do not cover feat_dim %lld",
                (long long)num_codebooks, (long long)column_slice, (long long)feat_dim);
  F2CGT_REQUIRE(target_bits == 1 || target_bits == 2 || target_bits == 4 || target_bits == 8 || target_bits == 16,
                F2CGT_E_UNSUPPORTED, "sq_encode: target_bits must be 1,2,4,8 or 16 (got %d)", target_bits);
  const int64_t dst_dim = target_bits < 8 ? ceil_div(feat_dim * target_bits, 8) : feat_dim;
  const int64_t n = rows * dst_dim;
  if (n == 0) return 0;
  F2CGT_REQUIRE(src && dst && codebooks, F2CGT_E_INVALID, "sq_encode: null buffer");
  hipStream_t st = as_stream(stream);
  if (num_codebooks < (1 << 20)) {
    int rc = -1;
    const int ncb = (int)num_codebooks;
    switch (target_bits) {
      case 1: rc = encode_f4_launch<1, true>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, dst_dim, st, "sq_encode"); break;
      case 2: rc = encode_f4_launch<2, true>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, dst_dim, st, "sq_encode"); break;
      case 4: rc = encode_f4_launch<4, true>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, dst_dim, st, "sq_encode"); break;
      case 8: rc = encode_f4_launch<8, true>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, dst_dim * 1, st, "sq_encode"); break;
      default: rc = encode_f4_launch<16, true>(src, dst, codebooks, column_slice, ncb, rows, feat_dim, dst_dim * 2, st, "sq_encode"); break;
    }
    if (rc >= 0) return rc;
  }
  const int grid = grid_for(n, 16);
#define F2CGT_CASE(B, T)                                                                              \
  case B:                                                                                             \
    sq_encode_kernel<B, T><<<grid, kBlock, 0, st>>>(src, static_cast<T*>(dst), codebooks, rows,      \
                                                    feat_dim, dst_dim, column_slice, num_codebooks);  \
    break;
  switch (target_bits) {
    F2CGT_CASE(1, uint8_t) F2CGT_CASE(2, uint8_t) F2CGT_CASE(4, uint8_t) F2CGT_CASE(8, int8_t)
    default: F2CGT_CASE(16, int16_t)
  }
#undef F2CGT_CASE
  return launch_status("sq_encode");
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
      // 8-bit codes are signed (sq_compress yields -128..127); the reference reads a uint8 tensor as
      // 0..255, values its encoder never produces, so that combination is refused instead of guessed
      F2CGT_REQUIRE(target_bits != 8 || code_dtype == F2CGT_DT_I8, F2CGT_E_UNSUPPORTED,
                    "sq_decompress: 8-bit codes are signed, pass them as int8 (got uint8)");
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
  {
    int rc = -1;
    switch (target_bits) {
      case 1: rc = decode_f4_launch<1, true>(codes, out, params, param_stride, 1, 0, rows, src_dim, feat_dim, st, "sq_affine_decompress"); break;
      case 2: rc = decode_f4_launch<2, true>(codes, out, params, param_stride, 1, 0, rows, src_dim, feat_dim, st, "sq_affine_decompress"); break;
      case 4: rc = decode_f4_launch<4, true>(codes, out, params, param_stride, 1, 0, rows, src_dim, feat_dim, st, "sq_affine_decompress"); break;
      default: rc = decode_f4_launch<8, true>(codes, out, params, param_stride, 1, 0, rows, src_dim, feat_dim, st, "sq_affine_decompress"); break;
    }
    if (rc >= 0) return rc;
  }
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
