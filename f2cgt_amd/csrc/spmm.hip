// CSC mean aggregation with the decode of the source rows inlined ("decompress-SpMM").
//
// One skeleton, many decoders.  A destination row is owned by a group of G lanes
// (G = 4..64, a power of two, so 1..16 rows share a wave64).  Lane l of the group owns
// NOUT consecutive output columns; for every edge it loads just the packed bytes that
// feed those columns, decodes them in registers and adds them to fp32 accumulators in
// edge order, so no decompressed tensor exists and the per-column summation order is
// the sequential one of the reference kernels (src/fusion_spmm.cu:28-36).  The mean is
// one IEEE division per output; the store is non-temporal.
//
// Decoders (struct *Dec): plain features, log-domain SQ through an LDS look-up table,
// log-domain SQ evaluated directly (16-bit codes), per-column affine SQ, VQ with the
// codebook window staged in LDS, and the two-table hybrid.
#include "common.hpp"
#include "spmm_fast.hpp"

#include <cstdlib>

#include <type_traits>

namespace f2cgt {
namespace {

constexpr int kUnroll = 4;
constexpr int kMaxBlock = 1024;
constexpr int64_t kLdsBudget = 128 * 1024;  // of the 160 KB per CU

template <int BYTES> struct packed_word;
template <> struct packed_word<1> { using type = uint8_t; };
template <> struct packed_word<2> { using type = uint16_t; };
template <> struct packed_word<4> { using type = uint32_t; };

// ---- output store ----------------------------------------------------------------
// A decoder that declares kAlign8 writes rows that start at multiples of 8 bytes only (4 k + 2 columns).
template <class Dec, class = void> struct dec_align8 : std::false_type {};
template <class Dec> struct dec_align8<Dec, std::void_t<decltype(Dec::kAlign8)>> : std::bool_constant<Dec::kAlign8> {};

template <int NOUT, typename Acc, typename Out, bool A8 = false>
__device__ __forceinline__ void store_mean(Out* __restrict__ o, const Acc (&acc)[NOUT], Acc deg,
                                           int nvalid, bool vec_ok) {
  if constexpr (A8) {
    static_assert(NOUT == 4 && std::is_same<Out, float>::value, "four fp32 columns per lane");
    if (nvalid >= 4) store_nt4_align8(o, acc[0] / deg, acc[1] / deg, acc[2] / deg, acc[3] / deg);
    else store_nt2(o, acc[0] / deg, acc[1] / deg);   // the row's last two columns
    return;
  }
  if constexpr (std::is_same<Out, float>::value) {
    if (vec_ok && nvalid >= NOUT) {
      if constexpr (NOUT == 2) {
        store_nt2(o, acc[0] / deg, acc[1] / deg);
        return;
      } else if constexpr (NOUT % 4 == 0) {
#pragma unroll
        for (int i = 0; i < NOUT; i += 4)
          store_nt4(o + i, acc[i] / deg, acc[i + 1] / deg, acc[i + 2] / deg, acc[i + 3] / deg);
        return;
      }
    }
#pragma unroll
    for (int i = 0; i < NOUT; ++i)
      if (i < nvalid) store_nt(o + i, acc[i] / deg);
  } else {
#pragma unroll
    for (int i = 0; i < NOUT; ++i)
      if (i < nvalid) o[i] = (Out)(acc[i] / deg);
  }
}

// ---- the skeleton ------------------------------------------------------------------
template <class Dec, typename Idx>
__global__ __launch_bounds__(kMaxBlock) void agg_kernel(Dec dec, const Idx* __restrict__ indptr,
                                                        const Idx* __restrict__ indices,
                                                        typename Dec::Out* __restrict__ out,
                                                        int64_t R, int64_t E, int64_t N,
                                                        int feat_dim, int tile_cols, int G,
                                                        bool vec_ok) {
  constexpr int NOUT = Dec::NOUT;
  using Acc = typename Dec::Acc;
  extern __shared__ __align__(16) unsigned char smem[];

  const int col_begin = blockIdx.y * tile_cols;
  const int col_end = (col_begin + tile_cols < feat_dim) ? col_begin + tile_cols : feat_dim;
  dec.block_setup(smem, col_begin, col_end);

  const int lane = threadIdx.x & (G - 1);
  const int group = threadIdx.x / G;
  const int gpb = blockDim.x / G;
  const int64_t row_stride = (int64_t)gridDim.x * gpb;

  for (int col0 = col_begin + lane * NOUT; col0 < col_end; col0 += G * NOUT) {
    const typename Dec::Ctx ctx = dec.column_setup(col0);
    const int nvalid = (feat_dim - col0) < NOUT ? (feat_dim - col0) : NOUT;
    for (int64_t r = (int64_t)blockIdx.x * gpb + group; r < R; r += row_stride) {
      int64_t b, e;
      row_range(indptr, r, E, b, e);
      const Acc deg = (Acc)(float)((e - b) == 0 ? 1 : (e - b));
      Acc acc[NOUT];
#pragma unroll
      for (int i = 0; i < NOUT; ++i) acc[i] = (Acc)0;
      for (int64_t k = b; k < e; k += kUnroll) {
        int64_t s[kUnroll];
        typename Dec::Raw raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) s[u] = (k + u < e) ? clamp_idx(indices[k + u], N) : -1;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
          if (s[u] >= 0) raw[u] = dec.load(ctx, s[u]);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
          if (s[u] >= 0) dec.accum(ctx, raw[u], acc);
      }
      store_mean<NOUT, Acc, typename Dec::Out, dec_align8<Dec>::value>(out + r * (int64_t)feat_dim + col0, acc, deg,
                                                                       nvalid, vec_ok);
    }
  }
}

// ---- decoders ---------------------------------------------------------------------

// Uncompressed fp32 features of 4 k + 2 columns (602): rows start at multiples of 8 bytes only.  A lane still owns
// four columns and moves them with one 16-byte access, which global memory takes at any dword; the lane of the row's
// last two columns moves those alone (2e6 edges at 10 per row, 602 columns: 1703 us with one column per lane, 961 us
// with two, 679 us so; 620 us at 600 columns).
struct PlainPairsDec {
  static constexpr int NOUT = 4;
  static constexpr bool kAlign8 = true;
  using Acc = float;
  using Out = float;
  struct Ctx { int col0; bool whole; };
  struct Raw { float v[4]; };
  const float* __restrict__ feat;
  int64_t D;
  __device__ void block_setup(unsigned char*, int, int) {}
  __device__ Ctx column_setup(int col0) const { return Ctx{col0, col0 + 4 <= D}; }
  __device__ Raw load(const Ctx& c, int64_t s) const {
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef f4 f4a8 __attribute__((aligned(8)));
    Raw r;
    const float* p = feat + s * D + c.col0;
    if (c.whole) {
      const f4 q = *reinterpret_cast<const f4a8*>(p);
      r.v[0] = q.x; r.v[1] = q.y; r.v[2] = q.z; r.v[3] = q.w;
    } else {
      const float2 q = *reinterpret_cast<const float2*>(p);
      r.v[0] = q.x; r.v[1] = q.y; r.v[2] = 0.f; r.v[3] = 0.f;
    }
    return r;
  }
  __device__ void accum(const Ctx&, const Raw& r, float (&acc)[4]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] += r.v[i];
  }
};

// Uncompressed features (spmm_csr).
template <typename T, int NOUT_>
struct PlainDec {
  static constexpr int NOUT = NOUT_;
  using Acc = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
  using Out = T;
  struct Ctx { int col0; };
  struct Raw { T v[NOUT_]; };
  const T* __restrict__ feat;
  int64_t D;
  __device__ void block_setup(unsigned char*, int, int) {}
  __device__ Ctx column_setup(int col0) const { return Ctx{col0}; }
  __device__ Raw load(const Ctx& c, int64_t s) const {
    Raw r;
    const T* p = feat + s * D + c.col0;
    if constexpr (NOUT_ == 4 && std::is_same<T, float>::value) {
      const float4 q = *reinterpret_cast<const float4*>(p);
      r.v[0] = q.x; r.v[1] = q.y; r.v[2] = q.z; r.v[3] = q.w;
    } else if constexpr (NOUT_ == 2 && std::is_same<T, float>::value) {
      const float2 q = *reinterpret_cast<const float2*>(p);
      r.v[0] = q.x; r.v[1] = q.y;
    } else {
#pragma unroll
      for (int i = 0; i < NOUT_; ++i) r.v[i] = p[i];
    }
    return r;
  }
  __device__ void accum(const Ctx&, const Raw& r, Acc (&acc)[NOUT_]) const {
    if constexpr (std::is_same<T, __half>::value) {
      // the reference sums in the feature type (src/fusion_spmm.cu:30-34): a half-precision sum is
      // rounded to half after every edge, which the fp32 accumulator reproduces by rounding here
#pragma unroll
      for (int i = 0; i < NOUT_; ++i) acc[i] = __half2float(__float2half_rn(acc[i] + __half2float(r.v[i])));
    } else {
#pragma unroll
      for (int i = 0; i < NOUT_; ++i) acc[i] += (Acc)r.v[i];
    }
  }
};

// Log-domain SQ, bits <= 8, through LUT[num_codebooks][2^BITS] in LDS.  The codebook is
// chosen per packed byte (src/fusion_spmm.cu:180).
template <int BITS, int BYTES>
struct SqLutDec {
  static constexpr int PER = 8 / BITS;
  static constexpr int NCODE = 1 << BITS;
  static constexpr int NOUT = BYTES * PER;
  using Acc = float;
  using Out = float;
  struct Ctx { int j0; int lut_base[BYTES]; };
  using Raw = uint32_t;
  const uint8_t* __restrict__ codes;
  const float* __restrict__ codebooks;
  int64_t src_dim;
  int64_t column_slice;
  int num_codebooks;
  const float* lut;
  __device__ void block_setup(unsigned char* smem, int, int) {
    float* l = reinterpret_cast<float*>(smem);
    for (int t = threadIdx.x; t < num_codebooks * NCODE; t += blockDim.x) {
      const float* cb = codebooks + (int64_t)(t >> BITS) * 5;
      const uint32_t raw = (uint32_t)(t & (NCODE - 1));
      float v;
      if (BITS == 1) {
        v = ((float)raw - 0.5f) * (2.f * cb[4]);
      } else {
        const float drange = (float)(1 << (BITS - 1));
        const float k = __fdiv_rn(__fsub_rn(cb[3], cb[2]), drange);
        const float code = BITS < 8 ? (float)raw - drange : (float)(int8_t)raw;
        v = sq_log_decode(code, k, cb[2]);
      }
      l[t] = v;
    }
    __syncthreads();
    lut = l;
  }
  __device__ Ctx column_setup(int col0) const {
    Ctx c;
    c.j0 = col0 / PER;
#pragma unroll
    for (int b = 0; b < BYTES; ++b) {
      int64_t cb = ((int64_t)(c.j0 + b) * PER) / column_slice;
      cb = cb < num_codebooks ? cb : num_codebooks - 1;
      c.lut_base[b] = (int)cb * NCODE;
    }
    return c;
  }
  __device__ Raw load(const Ctx& c, int64_t s) const {
    using W = typename packed_word<BYTES>::type;
    return (uint32_t)*reinterpret_cast<const W*>(codes + s * src_dim + c.j0);
  }
  __device__ void accum(const Ctx& c, Raw raw, float (&acc)[NOUT]) const {
#pragma unroll
    for (int b = 0; b < BYTES; ++b) {
      const uint32_t byte = (raw >> (8 * b)) & 0xffu;
#pragma unroll
      for (int k = 0; k < PER; ++k)
        acc[b * PER + k] += lut[c.lut_base[b] + ((byte >> (BITS * k)) & (NCODE - 1))];
    }
  }
};

// Log-domain SQ evaluated per edge (16-bit codes, or a LUT too large for LDS).
template <int BITS, typename CT>
struct SqDirectDec {
  static constexpr int PER = BITS < 8 ? 8 / BITS : 1;
  static constexpr int NOUT = 1;
  using Acc = float;
  using Out = float;
  struct Ctx { int64_t j; int shift; float k; float emin; float mean; };
  using Raw = uint32_t;
  const CT* __restrict__ codes;
  const float* __restrict__ codebooks;
  int64_t src_dim;
  int64_t column_slice;
  int num_codebooks;
  __device__ void block_setup(unsigned char*, int, int) {}
  __device__ Ctx column_setup(int col0) const {
    Ctx c;
    c.j = col0 / PER;
    c.shift = BITS < 8 ? BITS * (col0 % PER) : 0;
    int64_t cb = (c.j * PER) / column_slice;
    cb = cb < num_codebooks ? cb : num_codebooks - 1;
    const float* p = codebooks + cb * 5;
    c.emin = p[2];
    c.k = __fdiv_rn(__fsub_rn(p[3], p[2]), (float)(1 << (BITS > 1 ? BITS - 1 : 1)));
    c.mean = p[4];
    return c;
  }
  __device__ Raw load(const Ctx& c, int64_t s) const { return (uint32_t)codes[s * src_dim + c.j]; }
  __device__ void accum(const Ctx& c, Raw raw, float (&acc)[1]) const {
    constexpr uint32_t MASK = BITS >= 16 ? 0xffffu : ((1u << BITS) - 1u);
    const uint32_t bitsv = (raw >> c.shift) & MASK;
    float v;
    if (BITS == 1) {
      v = ((float)bitsv - 0.5f) * (2.f * c.mean);
    } else {
      float code;
      if (BITS < 8) code = (float)bitsv - (float)(1 << (BITS - 1));
      else if (BITS == 8) code = (float)(int8_t)bitsv;
      else code = (float)(int16_t)bitsv;
      v = sq_log_decode(code, c.k, c.emin);
    }
    acc[0] += v;
  }
};

// Per-column affine SQ: value = min_c + code * scale_c, product rounded before the sum.
template <int BITS, int BYTES>
struct SqAffineDec {
  static constexpr int PER = 8 / BITS;
  static constexpr int NOUT = BYTES * PER;
  using Acc = float;
  using Out = float;
  struct Ctx { int j0; float mn[NOUT]; float sc[NOUT]; };
  using Raw = uint32_t;
  const uint8_t* __restrict__ codes;
  const float* __restrict__ params;
  int64_t param_stride;
  int64_t src_dim;
  int feat_dim;
  __device__ void block_setup(unsigned char*, int, int) {}
  __device__ Ctx column_setup(int col0) const {
    Ctx c;
    c.j0 = col0 / PER;
#pragma unroll
    for (int i = 0; i < NOUT; ++i) {
      const bool ok = col0 + i < feat_dim;
      c.mn[i] = ok ? params[col0 + i] : 0.f;
      c.sc[i] = ok ? params[param_stride + col0 + i] : 0.f;
    }
    return c;
  }
  __device__ Raw load(const Ctx& c, int64_t s) const {
    using W = typename packed_word<BYTES>::type;
    return (uint32_t)*reinterpret_cast<const W*>(codes + s * src_dim + c.j0);
  }
  __device__ void accum(const Ctx& c, Raw raw, float (&acc)[NOUT]) const {
#pragma unroll
    for (int i = 0; i < NOUT; ++i) {
      const float code = (float)((raw >> (BITS * i)) & ((1u << BITS) - 1u));
      acc[i] += __fadd_rn(c.mn[i], __fmul_rn(code, c.sc[i]));
    }
  }
};

// VQ: the codebook slices of the column window [col_begin, col_end) live in LDS as
// [subspace][code][w] (or stay in global memory when one slice exceeds the budget).
template <typename CT, int NOUT_, bool USE_LDS>
struct VqDec {
  static constexpr int NOUT = NOUT_;
  using Acc = float;
  using Out = float;
  struct Ctx { int c; int base; };
  using Raw = int;
  const CT* __restrict__ codes;
  const float* __restrict__ codebooks;
  int num_codebooks, K, w;
  const float* table;
  int c_first;
  __device__ void block_setup(unsigned char* smem, int col_begin, int col_end) {
    if (USE_LDS) {
      float* l = reinterpret_cast<float*>(smem);
      c_first = col_begin / w;
      const int c_last = (col_end + w - 1) / w;
      const int total = (c_last - c_first) * K * w;
      const float* src = codebooks + (int64_t)c_first * K * w;
      if ((total & 3) == 0) {
        for (int t = threadIdx.x * 4; t < total; t += blockDim.x * 4)
          *reinterpret_cast<float4*>(l + t) = *reinterpret_cast<const float4*>(src + t);
      } else {
        for (int t = threadIdx.x; t < total; t += blockDim.x) l[t] = src[t];
      }
      __syncthreads();
      table = l;
    } else {
      c_first = 0;
      table = codebooks;
    }
  }
  __device__ Ctx column_setup(int col0) const {
    Ctx c;
    c.c = col0 / w;
    c.base = (c.c - c_first) * K * w + (col0 - c.c * w);
    return c;
  }
  __device__ Raw load(const Ctx& c, int64_t s) const { return (int)codes[s * num_codebooks + c.c]; }
  __device__ void accum(const Ctx& c, Raw code, float (&acc)[NOUT_]) const {
    code = code < 0 ? 0 : (code >= K ? K - 1 : code);
    const float* p = table + c.base + code * w;
    if constexpr (NOUT_ == 4) {
      const float4 q = *reinterpret_cast<const float4*>(p);
      acc[0] += q.x; acc[1] += q.y; acc[2] += q.z; acc[3] += q.w;
    } else if constexpr (NOUT_ == 2) {
      const float2 q = *reinterpret_cast<const float2*>(p);
      acc[0] += q.x; acc[1] += q.y;
    } else {
#pragma unroll
      for (int i = 0; i < NOUT_; ++i) acc[i] += p[i];
    }
  }
};

// Two tables selected per source row by row_map (>= 0: 8-bit affine SQ row, < 0: VQ row).
template <int NOUT_>
struct HybridDec {
  static constexpr int NOUT = NOUT_;
  using Acc = float;
  using Out = float;
  struct Ctx { int col0; int c; int base; float mn[NOUT_]; float sc[NOUT_]; };
  struct Raw { uint32_t payload; int is_sq; };
  const int32_t* __restrict__ row_map;
  const uint8_t* __restrict__ sq_codes;
  const float* __restrict__ sq_params;
  int64_t param_stride;
  const uint8_t* __restrict__ vq_codes;
  const float* __restrict__ vq_codebooks;
  int64_t n_sq, n_vq;
  int feat_dim, num_codebooks, K, w;
  const float* table;
  bool in_lds;   // codebooks staged in LDS; larger ones are read through the caches
  __device__ void block_setup(unsigned char* smem, int, int) {
    if (!in_lds) {
      table = vq_codebooks;
      return;
    }
    float* l = reinterpret_cast<float*>(smem);
    const int total = num_codebooks * K * w;
    if ((total & 3) == 0) {
      for (int t = threadIdx.x * 4; t < total; t += blockDim.x * 4)
        *reinterpret_cast<float4*>(l + t) = *reinterpret_cast<const float4*>(vq_codebooks + t);
    } else {
      for (int t = threadIdx.x; t < total; t += blockDim.x) l[t] = vq_codebooks[t];
    }
    __syncthreads();
    table = l;
  }
  __device__ Ctx column_setup(int col0) const {
    Ctx c;
    c.col0 = col0;
    c.c = col0 / w;
    c.base = c.c * K * w + (col0 - c.c * w);
#pragma unroll
    for (int i = 0; i < NOUT_; ++i) {
      c.mn[i] = sq_params[col0 + i];
      c.sc[i] = sq_params[param_stride + col0 + i];
    }
    return c;
  }
  __device__ Raw load(const Ctx& c, int64_t s) const {
    using W = typename packed_word<NOUT_>::type;
    Raw r;
    const int64_t m = (int64_t)row_map[s];
    if (m >= 0) {
      const int64_t row = m < n_sq ? m : n_sq - 1;
      r.is_sq = 1;
      r.payload = (uint32_t)*reinterpret_cast<const W*>(sq_codes + row * feat_dim + c.col0);
    } else {
      int64_t row = -m - 1;
      row = row < n_vq ? row : n_vq - 1;
      r.is_sq = 0;
      r.payload = (uint32_t)vq_codes[row * num_codebooks + c.c];
    }
    return r;
  }
  __device__ void accum(const Ctx& c, const Raw& r, float (&acc)[NOUT_]) const {
    if (r.is_sq) {
#pragma unroll
      for (int i = 0; i < NOUT_; ++i) {
        const float code = (float)((r.payload >> (8 * i)) & 0xffu);
        acc[i] += __fadd_rn(c.mn[i], __fmul_rn(code, c.sc[i]));
      }
    } else {
      int code = (int)r.payload;
      code = code >= K ? K - 1 : code;
      const float* p = table + c.base + code * w;
#pragma unroll
      for (int i = 0; i < NOUT_; ++i) acc[i] += p[i];
    }
  }
};

// ---- launch ---------------------------------------------------------------------------
struct Geometry {
  int G;       // lanes per destination row
  int block;   // threads per workgroup
  dim3 grid;   // x: row groups, y: column tiles
  int tile_cols;
};

// `cols` output columns per tile, NOUT per lane; lds_bytes decides how many workgroups
// can share a CU and therefore how persistent the grid is.
Geometry plan(int64_t R, int cols, int n_tiles, int nout, size_t lds_bytes) {
  Geometry g;
  int lanes = (int)ceil_div(cols, nout);
  g.G = pow2_ceil(lanes);
  if (g.G < 4) g.G = 4;
  if (g.G > kWave) g.G = kWave;
  g.block = lds_bytes > 32 * 1024 ? kMaxBlock : 256;
  const int gpb = g.block / g.G;
  int64_t need = ceil_div(R, gpb);
  int wg_per_cu = lds_bytes > 32 * 1024 ? (int)((160 * 1024) / (int64_t)lds_bytes)
                                        : (2048 / g.block);
  if (wg_per_cu < 1) wg_per_cu = 1;
  int64_t cap = (int64_t)num_cus() * wg_per_cu / n_tiles;
  if (cap < 1) cap = 1;
  if (need < 1) need = 1;
  g.grid = dim3((unsigned)(need < cap ? need : cap), (unsigned)n_tiles, 1);
  g.tile_cols = cols;
  return g;
}

template <class Dec>
int run(Dec dec, const void* indptr, const void* indices, int idx_dtype, typename Dec::Out* out,
        int64_t R, int64_t E, int64_t N, int feat_dim, const Geometry& g, size_t lds_bytes,
        bool vec_ok, hipStream_t st, const char* what) {
  if (plan_only()) {
    plan_record("agg_kernel", (int64_t)g.grid.x * g.grid.y, g.block, (int64_t)lds_bytes, 0, g.block / g.G);
    return 0;
  }
  if (lds_bytes > 48 * 1024) {
    hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(agg_kernel<Dec, int32_t>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(agg_kernel<Dec, int64_t>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e1 != hipSuccess || e2 != hipSuccess)
      return fail((int)(e1 != hipSuccess ? e1 : e2), "%s: cannot reserve %zu B of LDS", what, lds_bytes);
  }
  if (idx_dtype == F2CGT_DT_I32) {
    agg_kernel<Dec, int32_t><<<g.grid, g.block, lds_bytes, st>>>(
        dec, static_cast<const int32_t*>(indptr), static_cast<const int32_t*>(indices), out, R, E, N,
        feat_dim, g.tile_cols, g.G, vec_ok);
  } else {
    agg_kernel<Dec, int64_t><<<g.grid, g.block, lds_bytes, st>>>(
        dec, static_cast<const int64_t*>(indptr), static_cast<const int64_t*>(indices), out, R, E, N,
        feat_dim, g.tile_cols, g.G, vec_ok);
  }
  return launch_status(what);
}

int check_graph(const char* what, const void* indptr, const void* indices, int idx_dtype,
                const void* out, int64_t R, int64_t E, int64_t N, int64_t feat_dim) {
  F2CGT_REQUIRE(R >= 0 && E >= 0 && N >= 0 && feat_dim >= 0, F2CGT_E_INVALID, "%s: negative size", what);
  F2CGT_REQUIRE(feat_dim < (1ll << 30), F2CGT_E_UNSUPPORTED, "%s: feat_dim too large", what);
  F2CGT_REQUIRE(idx_dtype == F2CGT_DT_I32 || idx_dtype == F2CGT_DT_I64, F2CGT_E_UNSUPPORTED,
                "%s: indptr/indices must be int32 or int64", what);
  F2CGT_REQUIRE(indptr != nullptr, F2CGT_E_INVALID, "%s: null indptr", what);
  F2CGT_REQUIRE(E == 0 || indices != nullptr, F2CGT_E_INVALID, "%s: null indices", what);
  F2CGT_REQUIRE(E == 0 || N > 0, F2CGT_E_INVALID, "%s: edges but no source rows", what);
  F2CGT_REQUIRE(R * feat_dim == 0 || out != nullptr, F2CGT_E_INVALID, "%s: null out", what);
  return 0;
}

template <int BITS>
int run_sq_lut(const uint8_t* codes, const float* codebooks, const void* indptr, const void* indices,
               int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int64_t src_dim,
               int feat_dim, int n_cb, int64_t column_slice, hipStream_t st) {
  constexpr int PER = 8 / BITS;
  const size_t lds = (size_t)n_cb * (1 << BITS) * sizeof(float);
  const char* what = "sq_decompress_spmm_csr";
  const int bytes = (src_dim % 4 == 0 && aligned(codes, 4) && feat_dim > 16 * PER)   ? 4
                    : (src_dim % 2 == 0 && aligned(codes, 2) && feat_dim > 8 * PER) ? 2
                                                                                    : 1;
  const int nout = bytes * PER;
  const bool vec_ok = (feat_dim % (nout < 4 ? nout : 4) == 0) && aligned(out, 16);
  const Geometry g = plan(R, feat_dim, 1, nout, lds);
  if (bytes == 4) {
    SqLutDec<BITS, 4> d{codes, codebooks, src_dim, column_slice, n_cb, nullptr};
    return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, lds, vec_ok, st, what);
  } else if (bytes == 2) {
    SqLutDec<BITS, 2> d{codes, codebooks, src_dim, column_slice, n_cb, nullptr};
    return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, lds, vec_ok, st, what);
  }
  SqLutDec<BITS, 1> d{codes, codebooks, src_dim, column_slice, n_cb, nullptr};
  return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, lds, vec_ok, st, what);
}

template <int BITS, typename CT>
int run_sq_direct(const void* codes, const float* codebooks, const void* indptr, const void* indices,
                  int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int64_t src_dim,
                  int feat_dim, int n_cb, int64_t column_slice, hipStream_t st) {
  SqDirectDec<BITS, CT> d{static_cast<const CT*>(codes), codebooks, src_dim, column_slice, n_cb};
  const Geometry g = plan(R, feat_dim, 1, 1, 0);
  return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, 0, false, st,
             "sq_decompress_spmm_csr");
}

template <int BITS>
int run_sq_affine(const uint8_t* codes, const float* params, int64_t param_stride, const void* indptr,
                  const void* indices, int idx_dtype, float* out, int64_t R, int64_t E, int64_t N,
                  int64_t src_dim, int feat_dim, hipStream_t st) {
  constexpr int PER = 8 / BITS;
  const char* what = "sq_affine_decompress_spmm_csr";
  const int bytes = (src_dim % 4 == 0 && aligned(codes, 4) && feat_dim > 16 * PER && PER * 4 <= 8)   ? 4
                    : (src_dim % 2 == 0 && aligned(codes, 2) && feat_dim > 8 * PER && PER * 2 <= 8) ? 2
                                                                                                    : 1;
  const int nout = bytes * PER;
  const bool vec_ok = (feat_dim % (nout < 4 ? nout : 4) == 0) && aligned(out, 16);
  const Geometry g = plan(R, feat_dim, 1, nout, 0);
  if (bytes == 4) {
    if constexpr (PER * 4 <= 8) {
      SqAffineDec<BITS, 4> d{codes, params, param_stride, src_dim, feat_dim};
      return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, 0, vec_ok, st, what);
    }
  } else if (bytes == 2) {
    if constexpr (PER * 2 <= 8) {
      SqAffineDec<BITS, 2> d{codes, params, param_stride, src_dim, feat_dim};
      return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, 0, vec_ok, st, what);
    }
  }
  SqAffineDec<BITS, 1> d{codes, params, param_stride, src_dim, feat_dim};
  return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, 0, vec_ok, st, what);
}

template <typename CT>
int run_vq(const void* codes_v, const float* codebooks, const void* indptr, const void* indices,
           int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int feat_dim, int n_cb, int K,
           int w, hipStream_t st) {
  const char* what = "vq_decompress_spmm_csr";
  const CT* codes = static_cast<const CT*>(codes_v);
  const int64_t slice_bytes = (int64_t)K * w * 4;
  const int nout = (w % 4 == 0 && feat_dim % 4 == 0 && feat_dim >= 256) ? 4
                   : (w % 2 == 0 && feat_dim % 2 == 0)                   ? 2
                                                                         : 1;
  const bool vec_ok = aligned(out, 16) && aligned(codebooks, 16);
  if (slice_bytes > kLdsBudget) {  // not even one subspace fits: read the codebook through L2
    const Geometry g = plan(R, feat_dim, 1, 1, 0);
    VqDec<CT, 1, false> d{codes, codebooks, n_cb, K, w, nullptr, 0};
    return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, 0, false, st, what);
  }
  const int used_cb = (int)ceil_div(feat_dim, w);
  int cb_per_tile = (int)(kLdsBudget / slice_bytes);
  if (cb_per_tile > used_cb) cb_per_tile = used_cb;
  const int n_tiles = (int)ceil_div(used_cb, cb_per_tile);
  cb_per_tile = (int)ceil_div(used_cb, n_tiles);  // balance the tiles
  const size_t lds = (size_t)cb_per_tile * slice_bytes;
  const int tile_cols = cb_per_tile * w;
  Geometry g = plan(R, tile_cols < feat_dim ? tile_cols : feat_dim, n_tiles, nout, lds);
  g.tile_cols = tile_cols;
  if (nout == 4 && vec_ok) {
    VqDec<CT, 4, true> d{codes, codebooks, n_cb, K, w, nullptr, 0};
    return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g, lds, true, st, what);
  } else if (nout >= 2 && vec_ok) {
    VqDec<CT, 2, true> d{codes, codebooks, n_cb, K, w, nullptr, 0};
    Geometry g2 = plan(R, tile_cols < feat_dim ? tile_cols : feat_dim, n_tiles, 2, lds);
    g2.tile_cols = tile_cols;
    return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g2, lds, true, st, what);
  }
  VqDec<CT, 1, true> d{codes, codebooks, n_cb, K, w, nullptr, 0};
  Geometry g1 = plan(R, tile_cols < feat_dim ? tile_cols : feat_dim, n_tiles, 1, lds);
  g1.tile_cols = tile_cols;
  return run(d, indptr, indices, idx_dtype, out, R, E, N, feat_dim, g1, lds, false, st, what);
}

}  // namespace
}  // namespace f2cgt

using namespace f2cgt;

extern "C" int f2cgt_spmm_csr(const void* feat, int feat_dtype, void* out, const void* indptr,
                              const void* indices, int idx_dtype, int64_t num_rows,
                              int64_t num_edges, int64_t num_src_rows, int64_t feat_dim,
                              void* stream) {
  const char* what = "spmm_csr";
  if (int rc = check_graph(what, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, feat_dim)) return rc;
  if (num_rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(num_edges == 0 || feat != nullptr, F2CGT_E_INVALID, "%s: null feat", what);
  hipStream_t st = as_stream(stream);
  const int D = (int)feat_dim;
  switch (feat_dtype) {
    case F2CGT_DT_F32: {
      const bool v4 = D % 4 == 0 && aligned(feat, 16) && aligned(out, 16);
      if (v4) {
        PlainDec<float, 4> d{static_cast<const float*>(feat), feat_dim};
        return run(d, indptr, indices, idx_dtype, static_cast<float*>(out), num_rows, num_edges,
                   num_src_rows, D, plan(num_rows, D, 1, 4, 0), 0, true, st, what);
      }
      if (D % 2 == 0 && D >= 6 && aligned(feat, 8) && aligned(out, 8)) {   // rows of 4 k + 2 columns
        PlainPairsDec d{static_cast<const float*>(feat), feat_dim};
        return run(d, indptr, indices, idx_dtype, static_cast<float*>(out), num_rows, num_edges,
                   num_src_rows, D, plan(num_rows, D, 1, 4, 0), 0, true, st, what);
      }
      if (D % 2 == 0 && aligned(feat, 8) && aligned(out, 8)) {   // two columns
        PlainDec<float, 2> d{static_cast<const float*>(feat), feat_dim};
        return run(d, indptr, indices, idx_dtype, static_cast<float*>(out), num_rows, num_edges,
                   num_src_rows, D, plan(num_rows, D, 1, 2, 0), 0, true, st, what);
      }
      PlainDec<float, 1> d{static_cast<const float*>(feat), feat_dim};
      return run(d, indptr, indices, idx_dtype, static_cast<float*>(out), num_rows, num_edges,
                 num_src_rows, D, plan(num_rows, D, 1, 1, 0), 0, false, st, what);
    }
    case F2CGT_DT_F16: {
      PlainDec<__half, 1> d{static_cast<const __half*>(feat), feat_dim};
      return run(d, indptr, indices, idx_dtype, static_cast<__half*>(out), num_rows, num_edges,
                 num_src_rows, D, plan(num_rows, D, 1, 1, 0), 0, false, st, what);
    }
    case F2CGT_DT_F64: {
      PlainDec<double, 1> d{static_cast<const double*>(feat), feat_dim};
      return run(d, indptr, indices, idx_dtype, static_cast<double*>(out), num_rows, num_edges,
                 num_src_rows, D, plan(num_rows, D, 1, 1, 0), 0, false, st, what);
    }
    default:
      return fail(F2CGT_E_UNSUPPORTED, "%s: feat must be float32, float16 or float64", what);
  }
}

extern "C" int f2cgt_vq_decompress_spmm_csr(const void* codes, int code_dtype, const float* codebooks,
                                            const void* indptr, const void* indices, int idx_dtype,
                                            float* out, int64_t num_rows, int64_t num_edges,
                                            int64_t num_src_rows, int64_t feat_dim,
                                            int64_t num_codebooks, int64_t K, int64_t width,
                                            void* stream) {
  const char* what = "vq_decompress_spmm_csr";
  if (int rc = check_graph(what, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, feat_dim)) return rc;
  F2CGT_REQUIRE(num_codebooks > 0 && K > 0 && width > 0, F2CGT_E_INVALID,
                "%s: codebooks must be [n>0, K>0, w>0]", what);
  F2CGT_REQUIRE(num_codebooks * K * width < (1ll << 31), F2CGT_E_UNSUPPORTED, "%s: codebook too large", what);
  F2CGT_REQUIRE(feat_dim <= num_codebooks * width, F2CGT_E_INVALID,
                "%s: feat_dim %lld exceeds %lld codebooks x width %lld", what, (long long)feat_dim,
                (long long)num_codebooks, (long long)width);
  if (num_rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(codebooks && (num_edges == 0 || codes), F2CGT_E_INVALID, "%s: null buffer", what);
  hipStream_t st = as_stream(stream);
  const int D = (int)feat_dim, n_cb = (int)num_codebooks, k = (int)K, w = (int)width;
  bool fast_ok = code_dtype == F2CGT_DT_U8;
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_VQ_GENERIC")) fast_ok = fast_ok && v[0] != '1';   // per-row skeleton for every shape
#endif
  if (fast_ok &&
      vq_pipe_eligible(codes, codebooks, out, num_rows, num_edges, num_src_rows, D, n_cb, k, w))
    return vq_pipe_run(static_cast<const uint8_t*>(codes), codebooks, indptr, indices, idx_dtype, out, num_rows,
                       num_edges, num_src_rows, D, n_cb, k, w, st, what);
  switch (code_dtype) {
    case F2CGT_DT_U8:
      return run_vq<uint8_t>(codes, codebooks, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, D, n_cb, k, w, st);
    case F2CGT_DT_I8:
      return run_vq<int8_t>(codes, codebooks, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, D, n_cb, k, w, st);
    case F2CGT_DT_I16:
      return run_vq<int16_t>(codes, codebooks, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, D, n_cb, k, w, st);
    default:
      return fail(F2CGT_E_UNSUPPORTED, "%s: codes must be uint8, int8 or int16", what);
  }
}

extern "C" int f2cgt_sq_decompress_spmm_csr(const void* codes, int code_dtype, const float* codebooks,
                                            const void* indptr, const void* indices, int idx_dtype,
                                            float* out, int64_t num_rows, int64_t num_edges,
                                            int64_t num_src_rows, int64_t src_dim, int64_t feat_dim,
                                            int64_t num_codebooks, int target_bits,
                                            int64_t column_slice, void* stream) {
  const char* what = "sq_decompress_spmm_csr";
  if (int rc = check_graph(what, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, feat_dim)) return rc;
  F2CGT_REQUIRE(column_slice > 0 && num_codebooks > 0 && num_codebooks < (1 << 20), F2CGT_E_INVALID,
                "%s: column_slice and num_codebooks must be positive", what);
  F2CGT_REQUIRE(target_bits == 1 || target_bits == 2 || target_bits == 4 || target_bits == 8 ||
                    target_bits == 16,
                F2CGT_E_UNSUPPORTED, "%s: target_bit must be 1,2,4,8 or 16 (got %d)", what, target_bits);
  const int per = target_bits < 8 ? 8 / target_bits : 1;
  F2CGT_REQUIRE(num_codebooks * column_slice >= feat_dim, F2CGT_E_INVALID,
                "%s: %lld codebooks of %lld columns do not cover feat_dim %lld", what,
                (long long)num_codebooks, (long long)column_slice, (long long)feat_dim);
  F2CGT_REQUIRE(src_dim * per >= feat_dim, F2CGT_E_INVALID,
                "%s: %lld code words per row cannot hold %lld columns", what, (long long)src_dim,
                (long long)feat_dim);
  const bool byte_codes = code_dtype == F2CGT_DT_U8 || code_dtype == F2CGT_DT_I8;
  F2CGT_REQUIRE(target_bits == 16 ? code_dtype == F2CGT_DT_I16 : byte_codes, F2CGT_E_UNSUPPORTED,
                "%s: code dtype does not match target_bit %d", what, target_bits);
  // 8-bit codes are signed; a uint8 tensor would mean 0..255 to the reference's dtype dispatch
  // (src/common.h:68-82), values its encoder never produces: refused instead of guessed
  F2CGT_REQUIRE(target_bits != 8 || code_dtype == F2CGT_DT_I8, F2CGT_E_UNSUPPORTED,
                "%s: 8-bit codes are signed, pass them as int8 (got uint8)", what);
  if (num_rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(codebooks && (num_edges == 0 || codes), F2CGT_E_INVALID, "%s: null buffer", what);
  hipStream_t st = as_stream(stream);
  const int D = (int)feat_dim, n_cb = (int)num_codebooks;
  const uint8_t* c8 = static_cast<const uint8_t*>(codes);
  if (target_bits == 16)
    return run_sq_direct<16, uint16_t>(codes, codebooks, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, src_dim, D, n_cb, column_slice, st);
  if (sq_block_eligible(codes, out, num_src_rows, src_dim, D, target_bits, (int64_t)n_cb << target_bits))
    return sq_block_run(false, c8, codebooks, 0, column_slice, n_cb, indptr, indices, idx_dtype, out,
                        num_rows, num_edges, num_src_rows, src_dim, D, target_bits, st, what);
  const bool lut_fits = (int64_t)n_cb * (1 << target_bits) * 4 <= 32 * 1024;
#define F2CGT_CASE(B)                                                                                   \
  case B:                                                                                               \
    return lut_fits ? run_sq_lut<B>(c8, codebooks, indptr, indices, idx_dtype, out, num_rows, num_edges, \
                                    num_src_rows, src_dim, D, n_cb, column_slice, st)                   \
                    : run_sq_direct<B, uint8_t>(codes, codebooks, indptr, indices, idx_dtype, out,      \
                                                num_rows, num_edges, num_src_rows, src_dim, D, n_cb,    \
                                                column_slice, st);
  switch (target_bits) { F2CGT_CASE(1) F2CGT_CASE(2) F2CGT_CASE(4) default: F2CGT_CASE(8) }
#undef F2CGT_CASE
}

extern "C" int f2cgt_sq_affine_decompress_spmm_csr(const uint8_t* codes, const float* params,
                                                   int64_t param_stride, const void* indptr,
                                                   const void* indices, int idx_dtype, float* out,
                                                   int64_t num_rows, int64_t num_edges,
                                                   int64_t num_src_rows, int64_t src_dim,
                                                   int64_t feat_dim, int target_bits, void* stream) {
  const char* what = "sq_affine_decompress_spmm_csr";
  if (int rc = check_graph(what, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, feat_dim)) return rc;
  F2CGT_REQUIRE(target_bits == 1 || target_bits == 2 || target_bits == 4 || target_bits == 8,
                F2CGT_E_UNSUPPORTED, "%s: target_bit must be 1,2,4 or 8 (got %d)", what, target_bits);
  F2CGT_REQUIRE(param_stride >= feat_dim, F2CGT_E_INVALID, "%s: param_stride %lld < feat_dim %lld",
                what, (long long)param_stride, (long long)feat_dim);
  F2CGT_REQUIRE(src_dim * (8 / target_bits) >= feat_dim, F2CGT_E_INVALID,
                "%s: %lld packed bytes per row cannot hold %lld columns", what, (long long)src_dim,
                (long long)feat_dim);
  if (num_rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(params && (num_edges == 0 || codes), F2CGT_E_INVALID, "%s: null buffer", what);
  hipStream_t st = as_stream(stream);
  const int D = (int)feat_dim;
  // rows of more than ~250 edges overflow the row-block kernels' edge staging; the
  // per-row skeleton, whose cost per row is amortised over a long row, takes those graphs
  const bool long_rows = num_edges > 200 * num_rows;
  if (!long_rows && sq_affine_acc_eligible(codes, out, num_src_rows, src_dim, D, target_bits))
    return sq_affine_acc_run(codes, params, param_stride, indptr, indices, idx_dtype, out, num_rows,
                              num_edges, num_src_rows, src_dim, D, target_bits, st, what);
  if (!long_rows && sq_block_eligible(codes, out, num_src_rows, src_dim, D, target_bits, 0))
    return sq_block_run(true, codes, params, param_stride, 1, 1, indptr, indices, idx_dtype, out, num_rows,
                        num_edges, num_src_rows, src_dim, D, target_bits, st, what);
  switch (target_bits) {
    case 1: return run_sq_affine<1>(codes, params, param_stride, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, src_dim, D, st);
    case 2: return run_sq_affine<2>(codes, params, param_stride, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, src_dim, D, st);
    case 4: return run_sq_affine<4>(codes, params, param_stride, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, src_dim, D, st);
    default: return run_sq_affine<8>(codes, params, param_stride, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, src_dim, D, st);
  }
}

extern "C" int f2cgt_hybrid_decompress_spmm_csr(
    const int32_t* row_map, const uint8_t* sq_codes, const float* sq_params, int64_t param_stride,
    const uint8_t* vq_codes, const float* vq_codebooks, const void* indptr, const void* indices,
    int idx_dtype, float* out, int64_t num_rows, int64_t num_edges, int64_t num_src_rows,
    int64_t num_sq_rows, int64_t num_vq_rows, int64_t feat_dim, int64_t num_codebooks, int64_t K,
    int64_t width, void* stream) {
  const char* what = "hybrid_decompress_spmm_csr";
  if (int rc = check_graph(what, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, feat_dim)) return rc;
  F2CGT_REQUIRE(num_codebooks > 0 && K > 0 && K <= 256 && width > 0, F2CGT_E_INVALID,
                "%s: VQ codebooks must be [n>0, 0<K<=256, w>0]", what);
  F2CGT_REQUIRE(feat_dim == num_codebooks * width, F2CGT_E_UNSUPPORTED,
                "%s: feat_dim %lld must equal %lld codebooks x width %lld", what, (long long)feat_dim,
                (long long)num_codebooks, (long long)width);
  F2CGT_REQUIRE(param_stride >= feat_dim, F2CGT_E_INVALID, "%s: param_stride < feat_dim", what);
  F2CGT_REQUIRE(num_sq_rows >= 0 && num_vq_rows >= 0 && num_sq_rows + num_vq_rows > 0, F2CGT_E_INVALID,
                "%s: both code tables are empty", what);
  F2CGT_REQUIRE(num_codebooks * K * width < (1ll << 28), F2CGT_E_UNSUPPORTED, "%s: VQ codebooks too large", what);
  const int64_t cb_bytes = num_codebooks * K * width * 4;
  const bool in_lds = cb_bytes <= kLdsBudget;
  const int64_t lds = in_lds ? cb_bytes : 0;
  if (num_rows * feat_dim == 0) return 0;
  F2CGT_REQUIRE(row_map && sq_params && vq_codebooks, F2CGT_E_INVALID, "%s: null buffer", what);
  F2CGT_REQUIRE((num_sq_rows == 0 || sq_codes) && (num_vq_rows == 0 || vq_codes), F2CGT_E_INVALID,
                "%s: null code table", what);
  // An empty table is never dereferenced: clamp targets need at least one row each.
  F2CGT_REQUIRE(num_sq_rows > 0 && num_vq_rows > 0, F2CGT_E_UNSUPPORTED,
                "%s: both tables must hold at least one row", what);
  hipStream_t st = as_stream(stream);
  const int D = (int)feat_dim, n_cb = (int)num_codebooks, k = (int)K, w = (int)width;
  if (hybrid_acc_eligible(sq_codes, vq_codebooks, out, num_src_rows, num_sq_rows, num_vq_rows, D, w))
    return hybrid_acc_run(row_map, sq_codes, sq_params, param_stride, vq_codes, vq_codebooks, indptr, indices,
                          idx_dtype, out, num_rows, num_edges, num_src_rows, num_sq_rows, num_vq_rows, D, n_cb, k, w,
                          st, what);
  const bool a16 = aligned(out, 16) && aligned(vq_codebooks, 16);
  if (w % 4 == 0 && D >= 256 && aligned(sq_codes, 4) && a16) {
    HybridDec<4> d{row_map, sq_codes, sq_params, param_stride, vq_codes, vq_codebooks, num_sq_rows, num_vq_rows, D, n_cb, k, w, nullptr, in_lds};
    return run(d, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, D, plan(num_rows, D, 1, 4, (size_t)lds), (size_t)lds, true, st, what);
  }
  if (w % 2 == 0 && aligned(sq_codes, 2) && a16) {
    HybridDec<2> d{row_map, sq_codes, sq_params, param_stride, vq_codes, vq_codebooks, num_sq_rows, num_vq_rows, D, n_cb, k, w, nullptr, in_lds};
    return run(d, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, D, plan(num_rows, D, 1, 2, (size_t)lds), (size_t)lds, true, st, what);
  }
  HybridDec<1> d{row_map, sq_codes, sq_params, param_stride, vq_codes, vq_codebooks, num_sq_rows, num_vq_rows, D, n_cb, k, w, nullptr, in_lds};
  return run(d, indptr, indices, idx_dtype, out, num_rows, num_edges, num_src_rows, D, plan(num_rows, D, 1, 1, (size_t)lds), (size_t)lds, false, st, what);
}
