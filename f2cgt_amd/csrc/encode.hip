// VQ encode: pairwise distance and nearest-centre assignment.
//
// pairwise_distance materialises the [m,n] matrix.  With 9 to 64 dimensions the scores come from
// the matrix cores, as in predict_split_kernel below (its PW mode): |x|^2 + |y|^2 - 2 x.y with x.y
// from three bf16 pieces per value, after the mean of y has been subtracted from both (L2).  That
// form loses what x and y have in common, so an entry below an eighth of |x|^2 + |y|^2 is
// evaluated again as sum((x-y)^2) by its lane (cosine: rows and columns whose |x||y| can reach the
// reference's 1e-8 clamp); the 128-byte row
// segments of a tile are turned around through LDS so that a store instruction writes whole
// lines, and the matrix write bounds the kernel.  Other dimensions take pairwise_kernel: the
// unexpanded form with fused multiply-adds on the vector ALUs.
//
// kmeans_predict never writes the matrix.  For L2 it works, like pairwise_distance, on x - mu and
// c - mu (mu = mean of the centres): a common offset of the data then costs nothing, and the rows
// whose best two centres are closer than the rounding of that subtraction are decided from the
// original arrays.  For cosine the normalised centres lose their mean direction m when |m| > 1/2
// (argmin -x . c^ = argmin -x . (c^ - m)): the scores then resolve the differences between the
// centres' directions, which is all that data far from the origin leaves.  A wave owns rows of x and walks the centres a tile
// at a time on the matrix core: A = centre tile, B = x tile, so every lane holds 16 centre
// scores of ONE x row per tile and the running arg-min stays in registers.  Scores use the
// expanded form (|c|^2 - 2 x.c, the row constant |x|^2 dropped); rows whose two best scores are
// closer than the rounding bound of that evaluation are re-evaluated exactly in fp64 by the
// whole wave, so the label is the true first minimum.  Two evaluations of x.c:
//   * predict_split_kernel (up to 64 dimensions, operands within 96 KB of LDS): every fp32
//     value as three bf16 pieces, six v_mfma_f32_32x32x16_bf16 per 16 dimensions;
//   * predict_mfma_kernel: fp32 MFMA (v_mfma_f32_32x32x2_f32).  Vector instructions do not run in
//     the shadow of fp32 matrix instructions of the same SIMD (measured: a 128-instruction update
//     per 34 MFMAs costs its full issue time with one to three waves per SIMD), so there the
//     update is kept to four instructions per score and everything else is folded into the
//     MFMA operands.
#include "common.hpp"

#include <cfloat>
#include <climits>

namespace f2cgt {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Absolute part of the near-tie bound: the matrix core flushes products (and, for the split form,
// piece products 2^-8 and 2^-16 of the full one) that fall below the smallest normal fp32 number,
// which the relative bound does not see.  A few hundred such terms stay below this.
constexpr float kTinyGap = 1e-33f;

// ---- exact assignment of one row by a whole wave (fp64) ------------------------------
__device__ int exact_argmin_row(const float* __restrict__ xrow, const float* __restrict__ centers,
                                int n, int k, int metric, int lane) {
  double bestv = DBL_MAX;
  int besti = INT_MAX;
  double xn = 0.0;
  if (metric == F2CGT_METRIC_COSINE)
    for (int t = 0; t < k; ++t) xn += (double)xrow[t] * (double)xrow[t];
  for (int c = lane; c < n; c += kWave) {
    const float* cr = centers + (int64_t)c * k;
    double d;
    if (metric == F2CGT_METRIC_COSINE) {
      double dot = 0.0, cn = 0.0;
      for (int t = 0; t < k; ++t) {
        dot += (double)xrow[t] * (double)cr[t];
        cn += (double)cr[t] * (double)cr[t];
      }
      double den = sqrt(xn) * sqrt(cn);
      den = den > 1e-8 ? den : 1e-8;
      d = 1.0 - dot / den;
    } else {
      d = 0.0;
      for (int t = 0; t < k; ++t) {
        const double df = (double)xrow[t] - (double)cr[t];
        d += df * df;
      }
    }
    if (d < bestv) { bestv = d; besti = c; }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const double ov = __shfl_xor(bestv, off);
    const int oi = __shfl_xor(besti, off);
    if (ov < bestv || (ov == bestv && oi < besti)) { bestv = ov; besti = oi; }
  }
  // a row without a single comparable distance (NaN or infinite entries) goes to centre 0, where the
  // callers' trainer sends it (examples/my_kmeans.py:92-94 turns such distances into 1 before the
  // arg-min); the label must be a valid index whatever the data
  return besti == INT_MAX ? 0 : besti;
}

// LDS layout of the MFMA A operands: [pair of 32-centre tiles][step][half][centre % 32][tile of pair].
// Step 0 is the bias step, step 1 + t holds dimension half * khalf + t.  A lane reads both tiles
// of a step with one 8-byte access whose address is the pair base plus an immediate offset.
__device__ __forceinline__ int a_index(int centre, int step, int half, int KH) {
  return ((((centre >> 6) * (KH + 1) + step) * 2 + half) * 32 + (centre & 31)) * 2 + ((centre >> 5) & 1);
}

// Same for the L2 metric with the centres already staged in LDS, transposed as
// (layout: a_index).
__device__ int exact_argmin_row_l2_lds(const float* __restrict__ xrow, const float* cT, int n, int n_pad, int KH,
                                       int khalf, int k, int lane) {
  double bestv = DBL_MAX;
  int besti = INT_MAX;
  for (int c = lane; c < n; c += kWave) {
    // dimension h * khalf + t of centre c sits 128 * t + 64 * h floats after its step-1 slot
    const float* cp = cT + a_index(c, 1, 0, KH);
    double d = 0.0;
    for (int t = 0; t < khalf; ++t) {
      const double df = (double)xrow[t] - (double)cp[128 * t];
      d += df * df;
    }
    for (int t = 0; khalf + t < k; ++t) {
      const double df = (double)xrow[khalf + t] - (double)cp[128 * t + 64];
      d += df * df;
    }
    if (d < bestv) { bestv = d; besti = c; }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const double ov = __shfl_xor(bestv, off);
    const int oi = __shfl_xor(besti, off);
    if (ov < bestv || (ov == bestv && oi < besti)) { bestv = ov; besti = oi; }
  }
  // a row without a single comparable distance (NaN or infinite entries) goes to centre 0, where the
  // callers' trainer sends it (examples/my_kmeans.py:92-94 turns such distances into 1 before the
  // arg-min); the label must be a valid index whatever the data
  return besti == INT_MAX ? 0 : besti;
}

// ---- general fallback: one wave per row, exact -------------------------------------------
__global__ __launch_bounds__(256) void predict_exact_kernel(const float* __restrict__ x,
                                                            const float* __restrict__ centers,
                                                            int64_t* __restrict__ lab64,
                                                            uint8_t* __restrict__ lab8, int64_t m,
                                                            int n, int k, int metric) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t stride = (int64_t)gridDim.x * 4;
  for (int64_t row = wave; row < m; row += stride) {
    const int best = exact_argmin_row(x + row * k, centers, n, k, metric, lane);
    if (lane == 0) {
      if (lab64) lab64[row] = best;
      if (lab8) lab8[row] = (uint8_t)best;
    }
  }
}

// ---- MFMA path ----------------------------------------------------------------------------
// KH = per-half register depth: the k dimensions are split in two halves of
// khalf = ceil(k/2); lanes 0-31 feed half 0, lanes 32-63 half 1 (zero padded to KH).
// The whole score comes out of the matrix core: x is pre-scaled (-2 x for L2, -x for cosine;
// cosine centres are staged divided by their norm) and one extra k step multiplies the centre's
// bias (|c|^2, or +inf for the padding centres) by 1, so the epilogue is only the running
// (best, second, arg) update: compare, select, v_med3, v_min per score.  Two centre tiles are
// accumulated at a time, so one tile's MFMA chain runs under the other's epilogue.
__device__ __forceinline__ void argmin_update(const floatx16& acc, int ct, float& best, float& second, int& bv,
                                              int& bct) {
  const float before = best;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const float s = acc[v];
    const bool lt = s < best;
    second = __builtin_amdgcn_fmed3f(best, second, s);
    bv = lt ? v : bv;
    best = lt ? s : best;
  }
  bct = best < before ? ct : bct;
}

template <int KH>
__global__ __launch_bounds__(256) void predict_mfma_kernel(const float* __restrict__ x,
                                                           const float* __restrict__ centers,
                                                           int64_t* __restrict__ lab64,
                                                           uint8_t* __restrict__ lab8, int64_t m,
                                                           int n, int k, int metric, int n_pad) {
  extern __shared__ float smem[];
  float* cT = smem;                   // [n_pad / 64][KH + 1][2][32][2], see a_index
  const int a_floats = (n_pad >> 6) * (KH + 1) * 128;
  int* cmax_bits = reinterpret_cast<int*>(cT + a_floats);  // max |c|^2 as ordered int bits

  const int khalf = (k + 1) / 2;
  const bool cosine = metric == F2CGT_METRIC_COSINE;
  if (threadIdx.x == 0) *cmax_bits = 0;
  // stage the centres: coalesced reads of the [n, k] array, scattered LDS writes
  for (int i = threadIdx.x; i < a_floats; i += blockDim.x) cT[i] = 0.f;
  __syncthreads();
#pragma unroll 8
  for (int i = threadIdx.x; i < n * k; i += blockDim.x) {
    const int jj = i / k, dim = i - jj * k;
    const int hh = dim >= khalf ? 1 : 0;
    cT[a_index(jj, 1 + dim - hh * khalf, hh, KH)] = centers[i];
  }
  __syncthreads();
  for (int jj = threadIdx.x; jj < n_pad; jj += blockDim.x) {
    float cn = 0.f;
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll 4
      for (int t = 0; t < KH; ++t) {
        const float v = cT[a_index(jj, 1 + t, hh, KH)];
        cn += v * v;
      }
    if (cosine) {
      const float nr = sqrtf(cn);
      const float scale = 1.f / (nr > 1e-30f ? nr : 1e-30f);
      for (int hh = 0; hh < 2; ++hh)
        for (int t = 0; t < KH; ++t) cT[a_index(jj, 1 + t, hh, KH)] *= scale;
    }
    cT[a_index(jj, 0, 0, KH)] = jj >= n ? INFINITY : (cosine ? 0.f : cn);  // bias, times 1 in half 0
    if (jj < n && !cosine) atomicMax(cmax_bits, __float_as_int(cn));
  }
  __syncthreads();
  const float cmax = __int_as_float(*cmax_bits);

  const int lane = threadIdx.x & 63;
  const int j = lane & 31;
  const int h = lane >> 5;
  const int64_t n_tiles = (m + 31) / 32;
  const float unit = 5.9604645e-8f * (float)(4 * k + 16);
  const bool vec4 = (k % 8 == 0) && (KH % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
  const float xscale = cosine ? -1.f : -2.f;
  const float xb = h == 0 ? 1.f : 0.f;
  const float2* ap = reinterpret_cast<const float2*>(cT) + h * 32 + j;  // + (pair * (KH + 1) + step) * 64

  // raw coordinates of this lane's x row (its half of the k dimensions) for one tile
  auto load_x = [&](int64_t tile, float (&q)[KH]) {
    const int64_t row = tile * 32 + j;
    const bool valid = row < m;
    const float* xp = x + row * k + h * khalf;
    if (vec4) {
#pragma unroll
      for (int t = 0; t < KH; t += 4) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (valid && t < khalf) v = *reinterpret_cast<const float4*>(xp + t);
        q[t] = v.x; q[t + 1] = v.y; q[t + 2] = v.z; q[t + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int t = 0; t < KH; ++t) {
        const int dim = h * khalf + t;
        q[t] = (valid && t < khalf && dim < k) ? xp[t] : 0.f;
      }
    }
  };
  const int64_t tile0 = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t tstride = (int64_t)gridDim.x * 4;
  float xq[KH];
  if (tile0 < n_tiles) load_x(tile0, xq);
  for (int64_t tile = tile0; tile < n_tiles; tile += tstride) {
    const int64_t row = tile * 32 + j;
    const bool valid = row < m;
    float xr[KH];
    float xn = 0.f;
#pragma unroll
    for (int t = 0; t < KH; ++t) {
      xn += xq[t] * xq[t];
      xr[t] = xq[t] * xscale;
    }
    xn += __shfl_xor(xn, 32);
    // the next tile's rows travel from HBM while this tile is scored
    load_x(tile + tstride < n_tiles ? tile + tstride : tile, xq);
    asm volatile("" ::: "memory");

    float best = INFINITY, second = INFINITY;
    int bv = 0, bct = 0;
    for (int ct = 0; ct < n_pad; ct += 64) {
      floatx16 zero;
#pragma unroll
      for (int v = 0; v < 16; ++v) zero[v] = 0.f;
      const float2* pp = ap + (ct >> 6) * (KH + 1) * 64;
      const float2 b01 = pp[0];
      floatx16 acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(b01.x, xb, zero, 0, 0, 0);
      floatx16 acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(b01.y, xb, zero, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < KH; ++t) {
        const float2 a01 = pp[(t + 1) * 64];
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a01.x, xr[t], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a01.y, xr[t], acc1, 0, 0, 0);
      }
      argmin_update(acc0, ct, best, second, bv, bct);
      argmin_update(acc1, ct + 32, best, second, bv, bct);
    }
    int besti = bct + 8 * (bv >> 2) + 4 * h + (bv & 3);
    {  // merge the two halves of the wave (same x row, disjoint centres)
      const float ob = __shfl_xor(best, 32);
      const float os = __shfl_xor(second, 32);
      const int oi = __shfl_xor(besti, 32);
      if (ob < best || (ob == best && oi < besti)) {
        second = fminf(best, os);
        best = ob;
        besti = oi;
      } else {
        second = fminf(second, ob);
      }
    }
    const float scale = cosine ? sqrtf(xn) : xn + cmax;
    // + kTinyGap: products below the smallest normal number are flushed inside the matrix core
    const bool near_tie = valid && h == 0 && !((second - best) > unit * scale + kTinyGap);
    uint64_t todo = __ballot(near_tie);
    while (todo) {
      const int src = __ffsll((unsigned long long)todo) - 1;
      todo &= todo - 1;
      const int64_t rrow = tile * 32 + (src & 31);
      const int exact = cosine ? exact_argmin_row(x + rrow * k, centers, n, k, metric, lane)
                               : exact_argmin_row_l2_lds(x + rrow * k, cT, n, n_pad, KH, khalf, k, lane);
      if (lane == src) besti = exact;
    }
    if (valid && h == 0) {
      if (lab64) lab64[row] = besti;
      if (lab8) lab8[row] = (uint8_t)besti;
    }
  }
}

// ---- split-bf16 MFMA path ------------------------------------------------------------------
// The same scores at the bf16 matrix rate.  An fp32 value is the exact sum of three bf16 pieces
// (round to nearest, then the residual, then its residual: 3 x 8 significand bits plus the signs
// cover 24), a product of two pieces is exact in fp32, and of the nine piece products of x * c the
// three of relative size <= 2^-24 are dropped, so six v_mfma_f32_32x32x16_bf16 per 16 dimensions
// give x . c to fp32 accuracy at a sixth of the bf16 rate, 2.7 times the fp32 MFMA rate, and, unlike
// fp32 MFMA, with the vector ALUs free for the arg-min update while the matrix core runs.  The
// centre pieces sit in LDS in operand order ([piece][tile][step][lane] x 16 B, one ds_read_b128 per
// operand), a wave keeps the pieces of NB x 32 rows of x in registers so that every operand read
// feeds NB instructions, and the bias |c|^2 enters as the C operand of a tile's first instruction.
// Labels are decided as in the fp32 kernel: rows whose two best scores are closer than the
// rounding bound of this evaluation are re-evaluated exactly in fp64.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ void split3(float v, __bf16& p0, __bf16& p1, __bf16& p2) {
  p0 = (__bf16)v;
  float r = v - (float)p0;      // exact: the rounding error of a narrower format
  p1 = (__bf16)r;
  r = r - (float)p1;
  p2 = (__bf16)r;
}

// Exact L2 assignment of one row by a whole wave from the centre pieces in LDS (their sum is the
// fp32 centre, exactly); same result as exact_argmin_row on the array in HBM.  The unexpanded fp32
// distance has relative error <= (k + 3) 2^-24 (all terms positive), so it decides which centres
// can be the minimum at all; only those, usually two, are evaluated in fp64.
// The pieces hold the centres minus mu and the row is compared as fl(x - mu): the decision is exact
// for those rounded vectors, whose distances differ from the original ones by at most
// 2^-22 (|x - mu|^2 + |c - mu|^2) each.  When the best two are closer than twice that, the original
// row decides between them (fp64, from the arrays in HBM); with three or more that close the
// function returns -1 - (its choice) and the caller evaluates every centre.
template <int S>
__device__ int exact_argmin_row_l2_pieces(const float* __restrict__ xrow, float* xs, const bf16x8* ap, int n, int n_ct,
                                          int k, int lane, const float* mu, float cmax,
                                          const float* __restrict__ centers) {
  // the row goes through a wave-private LDS slot (16 S floats, zero padded) and the loops over the
  // 8-dimension chunks stay rolled: this rare path must not raise the kernel's register count
  const int piece_stride = n_ct * S * 64;                // operands per piece
  if (lane < 16 * S) xs[lane] = lane < k ? xrow[lane] - mu[lane] : 0.f;
  __builtin_amdgcn_wave_barrier();                       // LDS operations of one wave execute in order
  // fp32 centre values of chunk ch (dimensions [8 ch, 8 ch + 8)) of centre c: one operand per piece
  auto centre8 = [&](int c, int ch, float (&cv)[8]) {
    const bf16x8* q = ap + (c >> 5) * S * 64 + (ch >> 1) * 64 + (ch & 1) * 32 + (c & 31);
    const bf16x8 p0 = q[0], p1 = q[piece_stride], p2 = q[2 * piece_stride];
#pragma unroll
    for (int e = 0; e < 8; ++e) cv[e] = ((float)p0[e] + (float)p1[e]) + (float)p2[e];
  };
  // first pass: distance from the leading pieces only (relative error of a centre value 2^-8),
  // one operand per chunk
  auto dist_lead = [&](int c) -> float {
    float d = 0.f;
#pragma nounroll
    for (int ch = 0; ch < 2 * S; ++ch) {
      const bf16x8 p0 = ap[(c >> 5) * S * 64 + (ch >> 1) * 64 + (ch & 1) * 32 + (c & 31)];
      const float4 xa = *reinterpret_cast<const float4*>(xs + 8 * ch);
      const float4 xb = *reinterpret_cast<const float4*>(xs + 8 * ch + 4);
      const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float df = xv[e] - (float)p0[e];
        d = __fmaf_rn(df, df, d);
      }
    }
    return d;
  };
  auto dist32 = [&](int c) -> float {
    float d = 0.f;
#pragma nounroll
    for (int ch = 0; ch < 2 * S; ++ch) {
      float cv[8];
      centre8(c, ch, cv);
      const float4 xa = *reinterpret_cast<const float4*>(xs + 8 * ch);
      const float4 xb = *reinterpret_cast<const float4*>(xs + 8 * ch + 4);
      const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float df = xv[e] - cv[e];                  // dimensions >= k hold zeros on both sides
        d = __fmaf_rn(df, df, d);
      }
    }
    return d;
  };
  // With c' the leading pieces (8 significant bits, round to nearest), |c - c'| <= 2^-8 |c| per
  // component, so | sqrt(d) - sqrt(d') | <= 2^-8 |c| <= 2^-8 (|x| + sqrt(d)): the centre c0 with the
  // smallest d' has sqrt(d0) <= (sqrt(dmin') + 2^-8 |x|) / (1 - 2^-8), the true minimum is no
  // farther, and so its own sqrt(d') <= (sqrt(dmin') + 2^-7 |x|) * (1 + 2^-6) (slack for the fp32
  // sums included).
  constexpr int kKeep = 4;            // first-pass distances kept in registers (all of them up to 256 centres)
  float dkeep[kKeep] = {0.f, 0.f, 0.f, 0.f};
  float dmin = INFINITY;
  // the lane's first four centres two at a time: two independent chains per chunk
#pragma unroll
  for (int i0 = 0; i0 < kKeep; i0 += 2) {
    int slot[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int c = lane + (i0 + i) * kWave;
      c = c < n ? c : 0;
      slot[i] = (c >> 5) * S * 64 + (c & 31);
    }
#pragma nounroll
    for (int ch = 0; ch < 2 * S; ++ch) {
      const int at = (ch >> 1) * 64 + (ch & 1) * 32;
      const bf16x8 pa = ap[slot[0] + at], pb = ap[slot[1] + at];
      const float4 xa = *reinterpret_cast<const float4*>(xs + 8 * ch);
      const float4 xb = *reinterpret_cast<const float4*>(xs + 8 * ch + 4);
      const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float da = xv[e] - (float)pa[e], db = xv[e] - (float)pb[e];
        dkeep[i0] = __fmaf_rn(da, da, dkeep[i0]);
        dkeep[i0 + 1] = __fmaf_rn(db, db, dkeep[i0 + 1]);
      }
    }
    asm volatile("" ::: "memory");
  }
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    if (lane + i * kWave >= n) dkeep[i] = INFINITY;
    dmin = fminf(dmin, dkeep[i]);
  }
  for (int c = lane + kKeep * kWave; c < n; c += kWave) dmin = fminf(dmin, dist_lead(c));
  float xnorm2 = lane < 16 * S ? xs[lane] * xs[lane] : 0.f;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    dmin = fminf(dmin, __shfl_xor(dmin, off));
    xnorm2 += __shfl_xor(xnorm2, off);
  }
  // centres whose exact distance is within `margin` of the smallest must reach the fp64 stage, so
  // that everything left out is known to be farther than that (2^-21 = 4.77e-7; the constants
  // leave room for the fp32 evaluation of the norms)
  const float marginf = 5.2e-7f * (xnorm2 + cmax);
  const float reach = (sqrtf(dmin) + 0.0078125f * sqrtf(xnorm2) + sqrtf(marginf)) * 1.015625f;
  const float lead_limit = reach * reach * 1.0001f + 1e-37f;
  // second pass: full fp32 distance of the survivors, then the exact fp64 one of those that can
  // still be the minimum (relative error of the fp32 sum <= (k + 3) 2^-24, all terms positive)
  float d32min = INFINITY;
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {      // the kept distances become the fp32 ones
    const int c = lane + i * kWave;
    dkeep[i] = (c < n && dkeep[i] <= lead_limit) ? dist32(c) : INFINITY;
    d32min = fminf(d32min, dkeep[i]);
    asm volatile("" ::: "memory");
  }
  for (int c = lane + kKeep * kWave; c < n; c += kWave)
    if (dist_lead(c) <= lead_limit) d32min = fminf(d32min, dist32(c));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) d32min = fminf(d32min, __shfl_xor(d32min, off));
  const float limit = d32min * (1.f + 1.1920929e-7f * (float)(k + 4)) + 1e-37f + marginf;
  double bestv = DBL_MAX, nextv = DBL_MAX, thirdv = DBL_MAX;   // the three smallest exact distances
  int besti = INT_MAX, nexti = INT_MAX;
  for (int c = lane, i = 0; c < n; c += kWave, ++i) {
    float d32 = dkeep[0];
#pragma unroll
    for (int q = 1; q < kKeep; ++q) d32 = i == q ? dkeep[q] : d32;
    if (i >= kKeep) d32 = dist_lead(c) <= lead_limit ? dist32(c) : INFINITY;
    if (!(d32 <= limit)) continue;
    double dd = 0.0;
#pragma nounroll
    for (int ch = 0; ch < 2 * S; ++ch) {
      float cv[8];
      centre8(c, ch, cv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const double df = (double)xs[8 * ch + e] - (double)cv[e];
        dd += df * df;
      }
    }
    if (dd < bestv) { thirdv = nextv; nextv = bestv; nexti = besti; bestv = dd; besti = c; }
    else if (dd < nextv) { thirdv = nextv; nextv = dd; nexti = c; }
    else if (dd < thirdv) thirdv = dd;
  }
  // merge of two sorted triples (a lane's centres ascend, and ties go to the smaller index)
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const double ob = __shfl_xor(bestv, off), on = __shfl_xor(nextv, off), ot = __shfl_xor(thirdv, off);
    const int oi = __shfl_xor(besti, off), oj = __shfl_xor(nexti, off);
    double m1, m2, m3;
    int i1, i2;
    if (ob < bestv || (ob == bestv && oi < besti)) {       // the other triple leads
      m1 = ob; i1 = oi;
      if (on < bestv || (on == bestv && oj < besti)) { m2 = on; i2 = oj; m3 = ot < bestv ? ot : bestv; }
      else { m2 = bestv; i2 = besti; m3 = on < nextv ? on : nextv; }
    } else {
      m1 = bestv; i1 = besti;
      if (ob < nextv || (ob == nextv && oi < nexti)) { m2 = ob; i2 = oi; m3 = on < nextv ? on : nextv; }
      else { m2 = nextv; i2 = nexti; m3 = ob < thirdv ? ob : thirdv; }
    }
    bestv = m1; besti = i1; nextv = m2; nexti = i2; thirdv = m3;
  }
  const double margin = 4.9e-7 * ((double)xnorm2 + (double)cmax);
  // no candidate at all (a row with NaN or infinite entries: nothing compares below the limit), or one:
  // the stages below index the centres with besti and nexti and must not see INT_MAX
  if (besti == INT_MAX) return 0;
  if (nexti == INT_MAX) return besti;
  if (nextv - bestv > margin) return besti;
  if (thirdv - bestv <= margin) return -1 - besti;       // three or more: the caller takes every centre
  // exactly two centres can be the nearest one of the original row: decide between them there
  double da = 0.0, db = 0.0;
  for (int t = lane; t < k; t += kWave) {
    const double xv = (double)xrow[t];
    const double ea = xv - (double)centers[(int64_t)besti * k + t], eb = xv - (double)centers[(int64_t)nexti * k + t];
    da += ea * ea;
    db += eb * eb;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    da += __shfl_xor(da, off);
    db += __shfl_xor(db, off);
  }
  const int lo = besti < nexti ? besti : nexti, hi = besti < nexti ? nexti : besti;
  const double dlo = besti < nexti ? da : db, dhi = besti < nexti ? db : da;
  return dhi < dlo ? hi : lo;
}

// Exact cosine assignment of one row by a whole wave.  The LDS pieces hold d = c / |c| - m (m: the
// mean direction or zero, the same for every centre, so x . m does not matter), |d| <= cdev; with
// d' their leading pieces, |x . d - x . d'| <= 2^-8 |x| cdev (1 + 2^-20), so only
// centres whose leading-piece dot product is within 2^-6 |x| cdev of the largest can have the smallest
// distance; those go through the fp32 dot product with all three pieces, and what that leaves is
// evaluated exactly, in fp64 from the centres in HBM, by the formula of exact_argmin_row.  Needs every centre to have a direction (|c|^2 > 1e-12).
template <int S>
__device__ int exact_argmin_row_cosine_pieces(const float* __restrict__ xrow, float* xs, const bf16x8* ap,
                                              const float* __restrict__ centers, int n, int n_ct, int k,
                                              int lane, float cdev) {
  if (lane < 16 * S) xs[lane] = lane < k ? xrow[lane] : 0.f;
  __builtin_amdgcn_wave_barrier();
  float xnorm2 = lane < 16 * S ? xs[lane] * xs[lane] : 0.f;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) xnorm2 += __shfl_xor(xnorm2, off);
  auto dot_lead = [&](int c) -> float {
    float d = 0.f;
#pragma nounroll
    for (int ch = 0; ch < 2 * S; ++ch) {
      const bf16x8 p0 = ap[(c >> 5) * S * 64 + (ch >> 1) * 64 + (ch & 1) * 32 + (c & 31)];
      const float4 xa = *reinterpret_cast<const float4*>(xs + 8 * ch);
      const float4 xb = *reinterpret_cast<const float4*>(xs + 8 * ch + 4);
      const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) d = __fmaf_rn(xv[e], (float)p0[e], d);
    }
    return d;
  };
  float smax = -INFINITY;
  for (int c = lane; c < n; c += kWave) smax = fmaxf(smax, dot_lead(c));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) smax = fmaxf(smax, __shfl_xor(smax, off));
  const float floor_s = smax - 0.015625f * cdev * sqrtf(xnorm2) - 1e-30f;
  // second filter: the fp32 dot product with the whole operand (the sum of its pieces) is within
  // ((k + 2) cdev + 3) 2^-24 |x| of x . (c / |c| - m) (the sum; the roundings of 1 / |c|, of the
  // product and of the subtraction), so the nearest centre is within twice that of the largest one.  Data far from the origin passes
  // the first filter with every centre; this one leaves the few that the fp64 stage has to read.
  auto dot32 = [&](int c) -> float {
    float d = 0.f;
    const int piece_stride = n_ct * S * 64;
#pragma nounroll
    for (int ch = 0; ch < 2 * S; ++ch) {
      const bf16x8* q = ap + (c >> 5) * S * 64 + (ch >> 1) * 64 + (ch & 1) * 32 + (c & 31);
      const bf16x8 p0 = q[0], p1 = q[piece_stride], p2 = q[2 * piece_stride];
      const float4 xa = *reinterpret_cast<const float4*>(xs + 8 * ch);
      const float4 xb = *reinterpret_cast<const float4*>(xs + 8 * ch + 4);
      const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) d = __fmaf_rn(xv[e], ((float)p0[e] + (float)p1[e]) + (float)p2[e], d);
    }
    return d;
  };
  float s32max = -INFINITY;
  for (int c = lane; c < n; c += kWave)
    if (dot_lead(c) >= floor_s) s32max = fmaxf(s32max, dot32(c));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s32max = fmaxf(s32max, __shfl_xor(s32max, off));
  const float floor32 = s32max - 1.1920929e-7f * ((float)(k + 4) * cdev + 3.f) * sqrtf(xnorm2) * 1.001f - 1e-30f;
  double xn = 0.0;
  for (int t = 0; t < k; ++t) xn += (double)xrow[t] * (double)xrow[t];
  double bestv = DBL_MAX;
  int besti = INT_MAX;
  for (int c = lane; c < n; c += kWave) {
    if (!(dot_lead(c) >= floor_s)) continue;
    if (!(dot32(c) >= floor32)) continue;
    const float* cr = centers + (int64_t)c * k;
    double dot = 0.0, cn = 0.0;
    for (int t = 0; t < k; ++t) {
      dot += (double)xrow[t] * (double)cr[t];
      cn += (double)cr[t] * (double)cr[t];
    }
    double den = sqrt(xn) * sqrt(cn);
    den = den > 1e-8 ? den : 1e-8;
    const double d = 1.0 - dot / den;
    if (d < bestv) { bestv = d; besti = c; }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const double ov = __shfl_xor(bestv, off);
    const int oi = __shfl_xor(besti, off);
    if (ov < bestv || (ov == bestv && oi < besti)) { bestv = ov; besti = oi; }
  }
  // a row without a single comparable distance (NaN or infinite entries) goes to centre 0, where the
  // callers' trainer sends it (examples/my_kmeans.py:92-94 turns such distances into 1 before the
  // arg-min); the label must be a valid index whatever the data
  return besti == INT_MAX ? 0 : besti;
}

// PW = false: labels of the nearest centre (KMeans.predict).  PW = true: the distance matrix itself
// (pairwise_distance), dist[row * ldd + centre], from the same scores.  The squared L2 distance
// does not change when one vector is subtracted from both arguments, and fl(v - mu) carries a
// relative error of 2^-24 of the difference itself, so for L2 both modes first subtract the mean of
// the centres from every x and centre: data far from the origin would otherwise lose most of the
// expanded form's bits to cancellation (and send most rows to the exact re-evaluation).
template <int S, int NB, bool PW>
__global__ __launch_bounds__(256) void predict_split_kernel(const float* __restrict__ x,
                                                            const float* __restrict__ centers,
                                                            int64_t* __restrict__ lab64,
                                                            uint8_t* __restrict__ lab8, int64_t m,
                                                            int n, int k, int metric, int n_pad,
                                                            float* __restrict__ dist, int64_t ldd) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int n_ct = n_pad >> 5;                                   // 32-centre tiles
  bf16x8* ap = reinterpret_cast<bf16x8*>(smem_raw);              // [3][n_ct][S][64]
  float* bias = reinterpret_cast<float*>(smem_raw + (size_t)3 * n_ct * S * 64 * 16);   // [n_pad]
  float* inv = bias + n_pad;                                     // [n_pad] 1 / |c| (cosine) or 1
  int* cmax_bits = reinterpret_cast<int*>(inv + n_pad);
  float* xs = reinterpret_cast<float*>(cmax_bits + 4) + (threadIdx.x >> 6) * 16 * S;   // one row of x per wave
  float* mu = reinterpret_cast<float*>(cmax_bits + 4) + 4 * 16 * S;                    // [16 S]
  constexpr int kTrPitch = 36;
  float* tr = mu + 16 * S + (threadIdx.x >> 6) * 32 * kTrPitch;                        // PW only
  const bool cosine = metric == F2CGT_METRIC_COSINE;
  if (threadIdx.x == 0) { cmax_bits[0] = 0; cmax_bits[1] = 0; cmax_bits[2] = 0; cmax_bits[3] = 0x7f800000; }
  // Staging works on items (centre, chunk of 8 dimensions) = one half-operand, four items per
  // thread with their loads issued together: first the sums of squares of the chunks, then, once
  // the norms are known, the pieces.  Dimensions from k on and centres from n on read as zeros.
  const bool cvec = (k % 8 == 0) && ((reinterpret_cast<uintptr_t>(centers) & 15) == 0);
  // L2: mu[t] = mean of the centres in dimension t, subtracted from every centre and every x (the
  // distances do not change, the cancellation of the expanded form does).  It is used only when it
  // matters, |mu|^2 above twice the summed variance of the centres (otherwise, and for cosine, mu
  // is zero and the subtraction of the hot loop is skipped): cmax_bits[3] != 0 says so for L2.
  const bool centred = !cosine;
  if (!centred) {
    if (threadIdx.x < 16 * S) mu[threadIdx.x] = 0.f;
    __syncthreads();
  } else {
    float* psum = reinterpret_cast<float*>(smem_raw);            // [4][64] sums, [4][64] sums of squares
    float* psq = psum + 256;                                     // (overwritten by the pieces later)
    const int t = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if (cvec) {
      // a lane sums a float4 column of every 16th row, sixteen loads in flight; the four row groups of
      // a wave are added with shuffles
      const int col = t & 15, part = threadIdx.x >> 4;
      float4 a4 = make_float4(0.f, 0.f, 0.f, 0.f), q4 = make_float4(0.f, 0.f, 0.f, 0.f);
      auto add = [&](const float4& v) {
        a4.x += v.x; a4.y += v.y; a4.z += v.z; a4.w += v.w;
        q4.x = __fmaf_rn(v.x, v.x, q4.x); q4.y = __fmaf_rn(v.y, v.y, q4.y);
        q4.z = __fmaf_rn(v.z, v.z, q4.z); q4.w = __fmaf_rn(v.w, v.w, q4.w);
      };
      if (4 * col < k) {
        const float* base = centers + 4 * col;
        int c = part;
        for (; c + 16 * 15 < n; c += 16 * 16) {
          float4 v[16];
#pragma unroll
          for (int u = 0; u < 16; ++u) v[u] = *reinterpret_cast<const float4*>(base + (int64_t)(c + 16 * u) * k);
#pragma unroll
          for (int u = 0; u < 16; ++u) add(v[u]);
        }
        for (; c < n; c += 16) add(*reinterpret_cast<const float4*>(base + (int64_t)c * k));
      }
#pragma unroll
      for (int off = 16; off <= 32; off <<= 1) {
        a4.x += __shfl_xor(a4.x, off); a4.y += __shfl_xor(a4.y, off);
        a4.z += __shfl_xor(a4.z, off); a4.w += __shfl_xor(a4.w, off);
        q4.x += __shfl_xor(q4.x, off); q4.y += __shfl_xor(q4.y, off);
        q4.z += __shfl_xor(q4.z, off); q4.w += __shfl_xor(q4.w, off);
      }
      if (t < 16) {
        *reinterpret_cast<float4*>(psum + wv * 64 + 4 * t) = a4;
        *reinterpret_cast<float4*>(psq + wv * 64 + 4 * t) = q4;
      }
    } else {
      float sum = 0.f, sq = 0.f;
      if (t < k)
        for (int c = wv; c < n; c += 4) {
          const float v = centers[(int64_t)c * k + t];
          sum += v;
          sq = __fmaf_rn(v, v, sq);
        }
      psum[wv * 64 + t] = sum;
      psq[wv * 64 + t] = sq;
    }
    __syncthreads();
    if (threadIdx.x < 64) {                                      // the first wave, all of it
      const float mt = ((psum[t] + psum[64 + t]) + (psum[128 + t] + psum[192 + t])) / (float)n;
      const float st = ((psq[t] + psq[64 + t]) + (psq[128 + t] + psq[192 + t])) / (float)n;
      float m2 = mt * mt, var = st - mt * mt;                    // dimensions from k on hold zeros
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
        m2 += __shfl_xor(m2, off);
        var += __shfl_xor(var, off);
      }
      const bool use = m2 > 2.f * (var > 0.f ? var : 0.f);
      if (t < 16 * S) mu[t] = use ? mt : 0.f;
      if (t == 0) cmax_bits[3] = use ? 1 : 0;
    }
    __syncthreads();
  }
  auto load8 = [&](int c, int ch, float (&v)[8]) {
    const bool in = c < n && 8 * ch < k;
    const float* cr = centers + (in ? (int64_t)c * k + 8 * ch : 0);
    if (cvec) {
      const float4 u = reinterpret_cast<const float4*>(cr)[0], w = reinterpret_cast<const float4*>(cr)[1];
      v[0] = u.x; v[1] = u.y; v[2] = u.z; v[3] = u.w; v[4] = w.x; v[5] = w.y; v[6] = w.z; v[7] = w.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = in ? v[e] : 0.f;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (in && 8 * ch + e < k) ? cr[e] : 0.f;
    }
    if (centred) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (in && 8 * ch + e < k) ? v[e] - mu[8 * ch + e] : 0.f;
    }
  };
  constexpr int kChunks = 2 * S;
  const int n_items = n_pad * kChunks;
  double* partial = reinterpret_cast<double*>(smem_raw);        // [n_pad][2 S], overwritten by the pieces later
  for (int i0 = threadIdx.x; i0 < n_items; i0 += blockDim.x * 4) {
    float v[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int it = i0 + u * blockDim.x;
      load8(it < n_items ? it / kChunks : n, it % kChunks, v[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int it = i0 + u * blockDim.x;
      double sq = 0.0;                       // fp64: 1 / |c| must be good to a rounding or two
#pragma unroll
      for (int e = 0; e < 8; ++e) sq += (double)v[u][e] * (double)v[u][e];
      if (it < n_items) partial[it] = sq;
    }
  }
  __syncthreads();
  for (int jj = threadIdx.x; jj < n_pad; jj += blockDim.x) {
    double cn64 = 0.0;
#pragma unroll
    for (int ch = 0; ch < kChunks; ++ch) cn64 += partial[jj * kChunks + ch];
    const float cn = (float)cn64;
    float sc = 1.f;
    if (cosine) sc = (float)(1.0 / sqrt(cn64 > 1e-60 ? cn64 : 1e-60));
    inv[jj] = sc;
    bias[jj] = jj >= n ? INFINITY : (cosine ? 0.f : cn);
    if (jj < n && !cosine) atomicMax(cmax_bits, __float_as_int(cn));
    if (jj < n && cosine && !(cn > 1e-12f)) atomicOr(cmax_bits + 1, 1);   // a centre without a direction
    if (PW && jj < n && cosine) atomicMin(cmax_bits + 3, __float_as_int(cn));
  }
  __syncthreads();
  // Cosine assignment: argmin_c -x . c^ = argmin_c -x . (c^ - m) for any m, and with m the mean of
  // the normalised centres c^ the operands of the matrix core shrink to the spread of the centres'
  // directions: what data far from the origin leaves of the evaluation's resolution goes to the
  // differences between centres.  Used when |m| > 1/2; mu[] then holds m (zeros otherwise).
  if (!PW && cosine) {
    float* psum = reinterpret_cast<float*>(smem_raw);            // [4][64]
    const int t = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const bool degenerate = cmax_bits[1] != 0;
    if (cvec) {
      // as for the L2 mean: a float4 column of every 16th row per lane, sixteen loads in flight
      const int col = t & 15, part = threadIdx.x >> 4;
      float4 a4 = make_float4(0.f, 0.f, 0.f, 0.f);
      if (!degenerate && 4 * col < k) {
        const float* base = centers + 4 * col;
        int c = part;
        for (; c + 16 * 15 < n; c += 16 * 16) {
          float4 v[16];
#pragma unroll
          for (int u = 0; u < 16; ++u) v[u] = *reinterpret_cast<const float4*>(base + (int64_t)(c + 16 * u) * k);
#pragma unroll
          for (int u = 0; u < 16; ++u) {
            const float sc = inv[c + 16 * u];
            a4.x = __fmaf_rn(v[u].x, sc, a4.x); a4.y = __fmaf_rn(v[u].y, sc, a4.y);
            a4.z = __fmaf_rn(v[u].z, sc, a4.z); a4.w = __fmaf_rn(v[u].w, sc, a4.w);
          }
        }
        for (; c < n; c += 16) {
          const float4 v = *reinterpret_cast<const float4*>(base + (int64_t)c * k);
          const float sc = inv[c];
          a4.x = __fmaf_rn(v.x, sc, a4.x); a4.y = __fmaf_rn(v.y, sc, a4.y);
          a4.z = __fmaf_rn(v.z, sc, a4.z); a4.w = __fmaf_rn(v.w, sc, a4.w);
        }
      }
#pragma unroll
      for (int off = 16; off <= 32; off <<= 1) {
        a4.x += __shfl_xor(a4.x, off); a4.y += __shfl_xor(a4.y, off);
        a4.z += __shfl_xor(a4.z, off); a4.w += __shfl_xor(a4.w, off);
      }
      if (t < 16) *reinterpret_cast<float4*>(psum + wv * 64 + 4 * t) = a4;
    } else {
      float sum = 0.f;
      if (!degenerate && t < k)
        for (int c = wv; c < n; c += 4) sum = __fmaf_rn(centers[(int64_t)c * k + t], inv[c], sum);
      psum[wv * 64 + t] = sum;
    }
    __syncthreads();
    if (threadIdx.x < 64) {
      const float mt = ((psum[t] + psum[64 + t]) + (psum[128 + t] + psum[192 + t])) / (float)n;
      float m2 = mt * mt;
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) m2 += __shfl_xor(m2, off);
      const bool use = !degenerate && m2 > 0.25f;
      if (t < 16 * S) mu[t] = use ? mt : 0.f;
      if (t == 0) cmax_bits[3] = use ? 1 : 0;
    }
    __syncthreads();
  }
  float dev2max = 0.f;
  for (int i0 = threadIdx.x; i0 < n_items; i0 += blockDim.x * 4) {
    float v[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int it = i0 + u * blockDim.x;
      load8(it < n_items ? it / kChunks : n, it % kChunks, v[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int it = i0 + u * blockDim.x;
      if (it >= n_items) break;
      const int c = it / kChunks, ch = it % kChunks;
      const float sc = inv[c];
      bf16x8 p0, p1, p2;
      float dev2 = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float val = v[u][e] * sc;
        if (cosine) val = (c < n && 8 * ch + e < k) ? val - mu[8 * ch + e] : 0.f;
        dev2 = __fmaf_rn(val, val, dev2);
        __bf16 a0, a1, a2;
        split3(val, a0, a1, a2);
        p0[e] = a0; p1[e] = a1; p2[e] = a2;
      }
      dev2max = fmaxf(dev2max, dev2);                            // largest 8-dimension share of |c^ - m|^2
      // chunk ch of centre c is lane (c % 32) + 32 (ch % 2) of step ch / 2 of tile c / 32
      const int at = ((c >> 5) * S + (ch >> 1)) * 64 + (ch & 1) * 32 + (c & 31);
      ap[at] = p0;
      ap[n_ct * S * 64 + at] = p1;
      ap[2 * n_ct * S * 64 + at] = p2;
    }
  }
  if (cosine) {                                                  // one LDS atomic per wave
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) dev2max = fmaxf(dev2max, __shfl_xor(dev2max, off));
    if ((threadIdx.x & 63) == 0) atomicMax(cmax_bits, __float_as_int(dev2max));
  }
  __syncthreads();
  const float cmax = __int_as_float(cmax_bits[0]);
  const bool use_mu = centred && __builtin_amdgcn_readfirstlane(cmax_bits[3]) != 0;
  const bool plain_cosine = cmax_bits[1] != 0;   // degenerate centres: no candidate filter for cosine
  // cosine: upper bound of |c^ - m| over the centres (1 without the mean; never above 2)
  float cdev = 1.f;
  if (!PW && cosine && !plain_cosine && cmax_bits[3] == 1) {
    cdev = sqrtf((float)kChunks * cmax) * 1.0001f;
    cdev = cdev < 2.f ? cdev : 2.f;
  }
  cdev = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(cdev)));
  const float cmin_norm = sqrtf(__int_as_float(cmax_bits[3]));   // PW, cosine: smallest |c|

  const int lane = threadIdx.x & 63;
  const int j = lane & 31;
  const int g = lane >> 5;
  constexpr int kGroupRows = 32 * NB;
  const int64_t n_groups = (m + kGroupRows - 1) / kGroupRows;
  // Error bound of one score in units of 2^-24 (|x|^2 + max |c|^2), which is >= 2 |x||c| = P and
  // >= |c|^2: each of the S leading instructions cuts its 17 addends at 2^-22 of the largest
  // (<= P): 68 S; the small pairs (2^-8 P and below) together stay below 4; the bias sum k + 1;
  // its addition 2; the dropped pairs (2^-24 P each way) 2; the rounding of x - mu and c - mu 4
  // (L2: 2^-22 (|x|^2 + |c|^2)); 3 spare.  Doubled for the two scores of a gap.
  const float unit = 5.9604645e-8f * (float)(2 * (68 * S + k + 16));
  const float xscale = cosine ? -1.f : -2.f;
  const bool vec4 = (k % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
  // A workgroup owns a contiguous share of the row groups and its four waves draw from it through
  // a counter in LDS: a wave held up by exact re-evaluations simply takes fewer groups.
  const int64_t per_wg = (n_groups + gridDim.x - 1) / gridDim.x;
  const int64_t wg_lo = (int64_t)blockIdx.x * per_wg;
  const int64_t wg_hi = wg_lo + per_wg < n_groups ? wg_lo + per_wg : n_groups;
  for (;;) {
    int draw = 0;
    if (lane == 0) draw = atomicAdd(cmax_bits + 2, 1);
    const int64_t grp = wg_lo + __builtin_amdgcn_readfirstlane(draw);
    if (grp >= wg_hi) break;
    bf16x8 xp[NB][S][3];
    float xn[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int64_t row = grp * kGroupRows + 32 * b + j;
      const bool valid = row < m;
      float sum = 0.f;
#pragma unroll
      for (int st = 0; st < S; ++st) {
        const int kk0 = 16 * st + 8 * g;
        float q[8];
        if (vec4) {
          const bool in = valid && kk0 < k;                   // loads always issued, from row 0 when idle
          const float4* xp4 = reinterpret_cast<const float4*>(x + (in ? row * k + kk0 : 0));
          const float4 u = xp4[0], w = xp4[1];
          q[0] = u.x; q[1] = u.y; q[2] = u.z; q[3] = u.w; q[4] = w.x; q[5] = w.y; q[6] = w.z; q[7] = w.w;
#pragma unroll
          for (int e = 0; e < 8; ++e) q[e] = in ? q[e] : 0.f;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) q[e] = (valid && kk0 + e < k) ? x[row * k + kk0 + e] : 0.f;
        }
        if (use_mu) {
#pragma unroll
          for (int e = 0; e < 8; ++e) q[e] = (valid && kk0 + e < k) ? q[e] - mu[kk0 + e] : 0.f;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          sum += q[e] * q[e];
          __bf16 a0, a1, a2;
          split3(q[e] * xscale, a0, a1, a2);
          xp[b][st][0][e] = a0; xp[b][st][1][e] = a1; xp[b][st][2][e] = a2;
        }
      }
      sum += __shfl_xor(sum, 32);
      xn[b] = sum;
    }

    float best[NB], second[NB];
    int bv[NB], bct[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) { best[b] = INFINITY; second[b] = INFINITY; bv[b] = 0; bct[b] = 0; }
    for (int ct = 0; ct < n_ct; ++ct) {
      floatx16 bz;
      const float* bp = bias + ct * 32 + 4 * g;
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const float4 t4 = *reinterpret_cast<const float4*>(bp + 8 * v4);
        bz[4 * v4] = t4.x; bz[4 * v4 + 1] = t4.y; bz[4 * v4 + 2] = t4.z; bz[4 * v4 + 3] = t4.w;
      }
      bf16x8 a[3][S];
#pragma unroll
      for (int q = 0; q < 3; ++q)
#pragma unroll
        for (int st = 0; st < S; ++st) a[q][st] = ap[(q * n_ct + ct) * S * 64 + st * 64 + lane];
      floatx16 acc[NB];
      // Piece pairs (x piece, centre piece).  The matrix core aligns the 16 products and C of an
      // instruction to the largest of them and keeps about 24 bits below it (measured: a unit
      // product next to +-2^24 survives, next to +-2^28 it does not), so the small pairs are
      // summed first, from zero, the leading pair last, and the bias, as large as the whole dot
      // product, is added on the vector ALU: the leading products are then cut at 2^-22 of their
      // own size, not of |c|^2 plus the running sum.
      constexpr int px[6] = {2, 0, 1, 1, 0, 0};
      constexpr int pc[6] = {0, 2, 1, 0, 1, 0};
      floatx16 zero;
#pragma unroll
      for (int v = 0; v < 16; ++v) zero[v] = 0.f;
#pragma unroll
      for (int b = 0; b < NB; ++b) acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[pc[0]][0], xp[b][0][px[0]], zero, 0, 0, 0);
#pragma unroll
      for (int term = 0; term < 6; ++term)
#pragma unroll
        for (int st = 0; st < S; ++st) {
          if (term == 0 && st == 0) continue;
#pragma unroll
          for (int b = 0; b < NB; ++b)
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[pc[term]][st], xp[b][st][px[term]], acc[b], 0, 0, 0);
        }
      if constexpr (PW) {
        // Distances of this 32-centre tile.  L2: |x|^2 + |c|^2 - 2 x.c (of the centred vectors) loses
        // what the two have in common, so an entry below an eighth of |x|^2 + |c|^2 (three bits gone)
        // is evaluated again as sum((x - c)^2); cosine needs that only near the clamp of |x||c|.
        const bool vst = (ldd % 4 == 0) && ((reinterpret_cast<uintptr_t>(dist) & 15) == 0);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          const bool valid = grp * kGroupRows + 32 * b + j < m;
          float dv[16];
          bool redo = false;
          if (!cosine) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              dv[v] = (acc[b][v] + bz[v]) + xn[b];
              redo = redo || (dv[v] < 0.125f * (xn[b] + bz[v]));
            }
          } else {
            const float nx = sqrtf(xn[b]);
            const float rx = 1.f / (nx > 1e-30f ? nx : 1e-30f);
#pragma unroll
            for (int v = 0; v < 16; ++v) dv[v] = __fmaf_rn(acc[b][v], rx, 1.f);
            // the reference form clamps |x||c| at 1e-8 from below: rows that can reach the clamp
            redo = plain_cosine || !(xn[b] > 1e-12f) || !(nx * cmin_norm > 2e-8f);
          }
          if (__ballot(valid && redo)) {
            // every lane evaluates its own flagged entries in the unexpanded fp32 form, one per trip
            // of a loop that exists once in the code (the entry's slot is a lane-varying index)
            uint32_t fm = 0;
#pragma unroll
            for (int v = 0; v < 16; ++v)
              if (valid && (cosine ? redo : (dv[v] < 0.125f * (xn[b] + bz[v])))) fm |= 1u << v;
            const float* xr = x + (grp * kGroupRows + 32 * b + j) * k;
#pragma nounroll
            while (__ballot(fm != 0)) {
              const int vl = fm ? __ffs((int)fm) - 1 : 0;
              const int cc = ct * 32 + 8 * (vl >> 2) + 4 * g + (vl & 3);
              const bool on = fm != 0 && cc < n;
              fm &= fm - 1;
              float s0 = 0.f, s1 = 0.f, s2 = 0.f;
              if (on) {
                const float* yr = centers + (int64_t)cc * k;
                auto term = [&](float xv, float yv) {
                  if (cosine) {
                    s0 = __fmaf_rn(xv, yv, s0);
                    s1 = __fmaf_rn(xv, xv, s1);
                    s2 = __fmaf_rn(yv, yv, s2);
                  } else {
                    const float d = xv - yv;
                    s0 = __fmaf_rn(d, d, s0);
                  }
                };
                if (vec4 && cvec) {        // eight dimensions per trip, their loads issued together
                  for (int t = 0; t < k; t += 8) {
                    const float4 xa = *reinterpret_cast<const float4*>(xr + t), xb = *reinterpret_cast<const float4*>(xr + t + 4);
                    const float4 ya = *reinterpret_cast<const float4*>(yr + t), yb = *reinterpret_cast<const float4*>(yr + t + 4);
                    term(xa.x, ya.x); term(xa.y, ya.y); term(xa.z, ya.z); term(xa.w, ya.w);
                    term(xb.x, yb.x); term(xb.y, yb.y); term(xb.z, yb.z); term(xb.w, yb.w);
                  }
                } else {
                  for (int t = 0; t < k; ++t) term(xr[t], yr[t]);
                }
                if (cosine) {
                  float den = sqrtf(s1) * sqrtf(s2);
                  den = den > 1e-8f ? den : 1e-8f;
                  s0 = 1.f - s0 / den;
                }
              }
#pragma unroll
              for (int v = 0; v < 16; ++v) dv[v] = (on && vl == v) ? s0 : dv[v];
            }
          }
          // A lane holds four 16-byte pieces of its row's 128-byte segment, every other one: stored
          // from here, an instruction would write half of each 32-byte sector.  The wave's LDS tile
          // (32 rows, pitch 36 floats: conflict-free both ways) turns the segment around so that
          // eight lanes store the 128 contiguous bytes of a row and an instruction covers eight rows.
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *reinterpret_cast<float4*>(tr + j * kTrPitch + 8 * q + 4 * g) =
                make_float4(dv[4 * q], dv[4 * q + 1], dv[4 * q + 2], dv[4 * q + 3]);
          __builtin_amdgcn_wave_barrier();
          const int c0 = ct * 32 + 4 * (lane & 7);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int rr = 8 * i + (lane >> 3);
            const float4 o4 = *reinterpret_cast<const float4*>(tr + rr * kTrPitch + 4 * (lane & 7));
            const int64_t orow_i = grp * kGroupRows + 32 * b + rr;
            if (orow_i < m) {
              float* o = dist + orow_i * ldd + c0;
              if (vst && c0 + 3 < n) {
                store_nt4(o, o4.x, o4.y, o4.z, o4.w);
              } else {
                if (c0 < n) o[0] = o4.x;
                if (c0 + 1 < n) o[1] = o4.y;
                if (c0 + 2 < n) o[2] = o4.z;
                if (c0 + 3 < n) o[3] = o4.w;
              }
            }
          }
        }
      } else {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[b][v] += bz[v];
          argmin_update(acc[b], ct * 32, best[b], second[b], bv[b], bct[b]);
        }
      }
    }
    if constexpr (PW) continue;
    int besti[NB];
    uint64_t todo[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const bool valid = grp * kGroupRows + 32 * b + j < m;
      int bi = bct[b] + 8 * (bv[b] >> 2) + 4 * g + (bv[b] & 3);
      float bs = best[b], sd = second[b];
      {  // merge the two halves of the wave (same x row, disjoint centres)
        const float ob = __shfl_xor(bs, 32);
        const float os = __shfl_xor(sd, 32);
        const int oi = __shfl_xor(bi, 32);
        if (ob < bs || (ob == bs && oi < bi)) {
          sd = fminf(bs, os);
          bs = ob;
          bi = oi;
        } else {
          sd = fminf(sd, ob);
        }
      }
      // cosine: the evaluation's share shrinks with the operands, the rounding of c / |c| (norm in
      // fp64, one rounding for 1 / |c|, one for the product, one for - m: 3 units, doubled) does not
      const float scale = cosine ? sqrtf(xn[b]) * (cdev + 3.5762787e-7f / unit) : xn[b] + cmax;
      besti[b] = bi;
      todo[b] = __ballot(valid && g == 0 && !((sd - bs) > unit * scale + kTinyGap));
    }
    // exact re-evaluation of the flagged rows: one copy of the code, whichever tile the row is in
#pragma nounroll
    for (int b = 0; b < NB; ++b) {
      uint64_t td = todo[0];
#pragma unroll
      for (int q = 1; q < NB; ++q) td = b == q ? todo[q] : td;
      while (td) {
        const int src = __ffsll((unsigned long long)td) - 1;
        td &= td - 1;
        const int64_t rrow = grp * kGroupRows + 32 * b + (src & 31);
        int exact;
        if (!cosine) {
          exact = exact_argmin_row_l2_pieces<S>(x + rrow * k, xs, ap, n, n_ct, k, lane, mu, cmax, centers);
          if (exact < 0) exact = exact_argmin_row(x + rrow * k, centers, n, k, metric, lane);   // the original row decides
        }
        else if (plain_cosine) exact = exact_argmin_row(x + rrow * k, centers, n, k, metric, lane);
        else exact = exact_argmin_row_cosine_pieces<S>(x + rrow * k, xs, ap, centers, n, n_ct, k, lane, cdev);
#pragma unroll
        for (int q = 0; q < NB; ++q) besti[q] = (b == q && lane == src) ? exact : besti[q];
      }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int64_t row = grp * kGroupRows + 32 * b + j;
      if (row < m && g == 0) {
        if (lab64) lab64[row] = besti[b];
        if (lab8) lab8[row] = (uint8_t)besti[b];
      }
    }
  }
}

// ---- pairwise distance --------------------------------------------------------------------
// 128 x 128 output tile per 256-thread workgroup, 8 x 8 per thread: per staged k step a thread
// reads 8 + 8 values from LDS (four 16-byte reads) for 64 fused multiply-adds, so the vector
// ALUs, not LDS, set the pace.  L2 is the unexpanded sum of squared differences.
constexpr int kTile = 128;  // rows of x and of y per workgroup
constexpr int kChunk = 16;  // k dimensions staged per pass

__global__ __launch_bounds__(256) void pairwise_kernel(const float* __restrict__ x,
                                                       const float* __restrict__ y,
                                                       float* __restrict__ dist, int64_t m, int64_t n,
                                                       int k, int metric) {
  __shared__ __align__(16) float xs[kChunk][kTile + 4];
  __shared__ __align__(16) float ys[kChunk][kTile + 4];
  const int tx = threadIdx.x & 15;  // 8 y rows each
  const int ty = threadIdx.x >> 4;  // 8 x rows each
  const bool cosine = metric == F2CGT_METRIC_COSINE;
  const int64_t n_tiles_n = (n + kTile - 1) / kTile;
  const int64_t n_tiles = ((m + kTile - 1) / kTile) * n_tiles_n;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t i0 = (tile / n_tiles_n) * kTile;
    const int64_t j0 = (tile % n_tiles_n) * kTile;
    float acc[8][8], xn[8], yn[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      xn[a] = 0.f;
      yn[a] = 0.f;
#pragma unroll
      for (int b = 0; b < 8; ++b) acc[a][b] = 0.f;
    }
    for (int k0 = 0; k0 < k; k0 += kChunk) {
      __syncthreads();
      for (int t = threadIdx.x; t < kTile * kChunk; t += 256) {
        const int r = t / kChunk, c = t % kChunk;
        const bool kin = k0 + c < k;
        xs[c][r] = (kin && i0 + r < m) ? x[(i0 + r) * k + k0 + c] : 0.f;
        ys[c][r] = (kin && j0 + r < n) ? y[(j0 + r) * k + k0 + c] : 0.f;
      }
      __syncthreads();
#pragma unroll 4
      for (int c = 0; c < kChunk; ++c) {
        float xv[8], yv[8];
        const float4 xa = *reinterpret_cast<const float4*>(&xs[c][ty * 8]);
        const float4 xb = *reinterpret_cast<const float4*>(&xs[c][ty * 8 + 4]);
        // a thread's 8 y rows are two groups of 4, 64 apart, so that the 16 threads of a row of the
        // tile store 256 contiguous bytes per instruction (8 consecutive ones would be 16 of every 32)
        const float4 ya = *reinterpret_cast<const float4*>(&ys[c][tx * 4]);
        const float4 yb = *reinterpret_cast<const float4*>(&ys[c][64 + tx * 4]);
        xv[0] = xa.x; xv[1] = xa.y; xv[2] = xa.z; xv[3] = xa.w; xv[4] = xb.x; xv[5] = xb.y; xv[6] = xb.z; xv[7] = xb.w;
        yv[0] = ya.x; yv[1] = ya.y; yv[2] = ya.z; yv[3] = ya.w; yv[4] = yb.x; yv[5] = yb.y; yv[6] = yb.z; yv[7] = yb.w;
        if (cosine) {
#pragma unroll
          for (int a = 0; a < 8; ++a) {
            xn[a] = __fmaf_rn(xv[a], xv[a], xn[a]);
            yn[a] = __fmaf_rn(yv[a], yv[a], yn[a]);
#pragma unroll
            for (int b = 0; b < 8; ++b) acc[a][b] = __fmaf_rn(xv[a], yv[b], acc[a][b]);
          }
        } else {
#pragma unroll
          for (int a = 0; a < 8; ++a)
#pragma unroll
            for (int b = 0; b < 8; ++b) {
              const float d = xv[a] - yv[b];
              acc[a][b] = __fmaf_rn(d, d, acc[a][b]);
            }
        }
      }
    }
    const bool full = j0 + kTile <= n && n % 4 == 0 && ((reinterpret_cast<uintptr_t>(dist) & 15) == 0);
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      const int64_t i = i0 + ty * 8 + a;
      if (i >= m) continue;
      float v[8];
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        v[b] = acc[a][b];
        if (cosine) {
          float den = sqrtf(xn[a]) * sqrtf(yn[b]);
          den = den > 1e-8f ? den : 1e-8f;
          v[b] = 1.f - v[b] / den;
        }
      }
      float* o = dist + i * n + j0 + tx * 4;       // columns j0 + 4 tx + (0..3) and + 64
      if (full) {
        store_nt4(o, v[0], v[1], v[2], v[3]);
        store_nt4(o + 64, v[4], v[5], v[6], v[7]);
      } else {
#pragma unroll
        for (int b = 0; b < 8; ++b) {
          const int col = tx * 4 + (b & 3) + (b >> 2) * 64;
          if (j0 + col < n) dist[i * n + j0 + col] = v[b];
        }
      }
    }
  }
}

// ---- any dimension, any number of centres: vector-ALU tiles with a running arg-min ----------------
// The assignment for shapes the matrix-core kernels do not take (more than 64 dimensions, or centres that do
// not fit their LDS layout).  A 256-thread workgroup owns 128 rows of x and walks the centres in tiles of 128
// with the 8 x 8 register tiles of pairwise_kernel (unexpanded sum of squared differences, or the cosine
// distance); instead of writing the distances a thread keeps, for each of its 8 rows, the smallest and the
// second smallest score and the centre of the smallest (first minimum: strict compares in rising centre order),
// and the 16 threads of a row combine theirs at the end.  fp32 sums of k terms are good to about k ulp, so a
// row whose two best scores are closer than that is decided again by exact_argmin_row (float64, one wave per
// such row), as is a row without a finite score.
__global__ __launch_bounds__(256) void predict_tiled_kernel(const float* __restrict__ x,
                                                            const float* __restrict__ centers,
                                                            int64_t* __restrict__ lab64,
                                                            uint8_t* __restrict__ lab8, int64_t m, int n, int k,
                                                            int metric) {
  __shared__ __align__(16) float xs[kChunk][kTile + 4];
  __shared__ __align__(16) float ys[kChunk][kTile + 4];
  __shared__ int s_again[kTile];
  __shared__ int s_count;
  const int tx = threadIdx.x & 15;  // 8 centres of a tile each
  const int ty = threadIdx.x >> 4;  // 8 rows each
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool cosine = metric == F2CGT_METRIC_COSINE;
  const float tol = (float)(k + 8) * 2.4e-7f;
  const int64_t row_tiles = (m + kTile - 1) / kTile;
  for (int64_t rt = blockIdx.x; rt < row_tiles; rt += gridDim.x) {
    const int64_t i0 = rt * kTile;
    float best[8], second[8];
    int arg[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      best[a] = INFINITY;
      second[a] = INFINITY;
      arg[a] = 0;
    }
    if (threadIdx.x == 0) s_count = 0;
    for (int j0 = 0; j0 < n; j0 += kTile) {
      float acc[8][8], xn[8], yn[8];
#pragma unroll
      for (int a = 0; a < 8; ++a) {
        xn[a] = 0.f;
        yn[a] = 0.f;
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[a][b] = 0.f;
      }
      for (int k0 = 0; k0 < k; k0 += kChunk) {
        __syncthreads();
        for (int t = threadIdx.x; t < kTile * kChunk; t += 256) {
          const int r = t / kChunk, c = t % kChunk;
          const bool kin = k0 + c < k;
          xs[c][r] = (kin && i0 + r < m) ? x[(i0 + r) * k + k0 + c] : 0.f;
          ys[c][r] = (kin && j0 + r < n) ? centers[(int64_t)(j0 + r) * k + k0 + c] : 0.f;
        }
        __syncthreads();
#pragma unroll 4
        for (int c = 0; c < kChunk; ++c) {
          float xv[8], yv[8];
          const float4 xa = *reinterpret_cast<const float4*>(&xs[c][ty * 8]);
          const float4 xb = *reinterpret_cast<const float4*>(&xs[c][ty * 8 + 4]);
          const float4 ya = *reinterpret_cast<const float4*>(&ys[c][tx * 4]);
          const float4 yb = *reinterpret_cast<const float4*>(&ys[c][64 + tx * 4]);
          xv[0] = xa.x; xv[1] = xa.y; xv[2] = xa.z; xv[3] = xa.w; xv[4] = xb.x; xv[5] = xb.y; xv[6] = xb.z; xv[7] = xb.w;
          yv[0] = ya.x; yv[1] = ya.y; yv[2] = ya.z; yv[3] = ya.w; yv[4] = yb.x; yv[5] = yb.y; yv[6] = yb.z; yv[7] = yb.w;
          if (cosine) {
#pragma unroll
            for (int a = 0; a < 8; ++a) {
              xn[a] = __fmaf_rn(xv[a], xv[a], xn[a]);
              yn[a] = __fmaf_rn(yv[a], yv[a], yn[a]);
#pragma unroll
              for (int b = 0; b < 8; ++b) acc[a][b] = __fmaf_rn(xv[a], yv[b], acc[a][b]);
            }
          } else {
#pragma unroll
            for (int a = 0; a < 8; ++a)
#pragma unroll
              for (int b = 0; b < 8; ++b) {
                const float d = xv[a] - yv[b];
                acc[a][b] = __fmaf_rn(d, d, acc[a][b]);
              }
          }
        }
      }
      // the tile's scores into the running (best, second, centre) of the thread's rows, centres in rising order
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const int col = j0 + tx * 4 + (b & 3) + (b >> 2) * 64;
#pragma unroll
        for (int a = 0; a < 8; ++a) {
          float v = acc[a][b];
          if (cosine) {
            float den = sqrtf(xn[a]) * sqrtf(yn[b]);
            den = den > 1e-8f ? den : 1e-8f;
            v = 1.f - v / den;
          }
          if (col >= n) v = INFINITY;
          const bool lt = v < best[a];
          second[a] = __builtin_amdgcn_fmed3f(best[a], second[a], v);
          arg[a] = lt ? col : arg[a];
          best[a] = lt ? v : best[a];
        }
      }
    }
    // the 16 threads of a row (consecutive lanes) combine: smallest score, lowest centre among equals
#pragma unroll
    for (int a = 0; a < 8; ++a) {
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) {
        const float ob = __shfl_xor(best[a], off), os = __shfl_xor(second[a], off);
        const int oa = __shfl_xor(arg[a], off);
        const bool take = ob < best[a] || (ob == best[a] && oa < arg[a]);
        const float hi = take ? best[a] : ob;          // the larger of the two smallest
        second[a] = fminf(fminf(second[a], os), hi);
        arg[a] = take ? oa : arg[a];
        best[a] = take ? ob : best[a];
      }
    }
    __syncthreads();   // s_count cleared, staging no longer read
    if (tx == 0) {
#pragma unroll
      for (int a = 0; a < 8; ++a) {
        const int64_t i = i0 + ty * 8 + a;
        if (i >= m) continue;
        // NaN compares false everywhere: a row of NaN keeps best = inf and is decided by the exact form
        const bool close = !(second[a] - best[a] > tol * (cosine ? 1.f : (fabsf(best[a]) + fabsf(second[a]))));
        if (close || !(best[a] < INFINITY)) {
          s_again[atomicAdd(&s_count, 1)] = ty * 8 + a;
        } else {
          if (lab64) lab64[i] = arg[a];
          if (lab8) lab8[i] = (uint8_t)arg[a];
        }
      }
    }
    __syncthreads();
    const int again = s_count;
    for (int f = wave; f < again; f += 4) {
      const int64_t i = i0 + s_again[f];
      const int lab = exact_argmin_row(x + i * k, centers, n, k, metric, lane);
      if (lane == 0) {
        if (lab64) lab64[i] = lab;
        if (lab8) lab8[i] = (uint8_t)lab;
      }
    }
    __syncthreads();   // s_again read before the next row tile clears the count
  }
}

template <int KH>
int launch_mfma(const float* x, const float* centers, int64_t* l64, uint8_t* l8, int64_t m, int n,
                int k, int metric, int n_pad, size_t lds, hipStream_t st) {
  auto kern = predict_mfma_kernel<KH>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "kmeans_predict: cannot reserve %zu B of LDS", lds);
  }
  // The tiles are dealt round-robin to a grid that must be resident all at once (a workgroup
  // that starts late does its whole share after the others have finished), so size the grid
  // from the occupancy the registers and LDS of this instantiation really allow.
  static thread_local size_t cached_lds = 0;   // per instantiation (KH) and thread
  static thread_local int cached_per_cu = 0;
  if (cached_per_cu == 0 || cached_lds != lds) {
    int v = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, reinterpret_cast<const void*>(kern), 256, lds) !=
            hipSuccess || v < 1)
      v = 1;
    cached_per_cu = v;
    cached_lds = lds;
  }
  const int per_cu = cached_per_cu;
  int64_t need = ceil_div(ceil_div(m, 32), 4);
  int64_t cap = (int64_t)num_cus() * per_cu;
  const int grid = (int)(need < cap ? need : cap);
  kern<<<grid, 256, lds, st>>>(x, centers, l64, l8, m, n, k, metric, n_pad);
  return launch_status("kmeans_predict");
}

template <int S, int NB, bool PW = false>
int launch_split(const float* x, const float* centers, int64_t* l64, uint8_t* l8, int64_t m, int n, int k,
                 int metric, int n_pad, size_t lds, hipStream_t st, float* dist = nullptr, int64_t ldd = 0) {
  auto kern = predict_split_kernel<S, NB, PW>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "kmeans_predict: cannot reserve %zu B of LDS", lds);
  }
  // resident grid, as for the fp32 kernel
  static thread_local size_t cached_lds = 0;
  static thread_local int cached_per_cu = 0;
  if (cached_per_cu == 0 || cached_lds != lds) {
    int v = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, reinterpret_cast<const void*>(kern), 256, lds) !=
            hipSuccess || v < 1)
      v = 1;
    cached_per_cu = v;
    cached_lds = lds;
  }
  const int64_t need = ceil_div(ceil_div(m, 32 * NB), 4);
  const int64_t cap = (int64_t)num_cus() * cached_per_cu;
  kern<<<(int)(need < cap ? need : cap), 256, lds, st>>>(x, centers, l64, l8, m, n, k, metric, n_pad, dist, ldd);
  return launch_status(PW ? "pairwise_distance" : "kmeans_predict");
}

}  // namespace
}  // namespace f2cgt

using namespace f2cgt;

extern "C" int f2cgt_pairwise_distance(const float* x, const float* y, float* dist, int64_t m,
                                       int64_t n, int64_t k, int metric, void* stream) {
  F2CGT_REQUIRE(m >= 0 && n >= 0 && k >= 0, F2CGT_E_INVALID, "pairwise_distance: negative size");
  F2CGT_REQUIRE(k < (1 << 24), F2CGT_E_UNSUPPORTED, "pairwise_distance: k too large");
  F2CGT_REQUIRE(metric == F2CGT_METRIC_L2 || metric == F2CGT_METRIC_COSINE, F2CGT_E_INVALID,
                "pairwise_distance: unknown metric %d", metric);
  if (m * n == 0) return 0;
  F2CGT_REQUIRE(dist && (k == 0 || (x && y)), F2CGT_E_INVALID, "pairwise_distance: null buffer");
  {  // matrix-core path: 9..64 dimensions; y goes through LDS in chunks of up to 96 KB of operands
    const int steps = (int)ceil_div(k, 16);
    if (k > 8 && steps <= 4) {
      const int64_t per32 = (int64_t)3 * steps * 64 * 16 + 2 * 32 * 4;          // bytes per 32 rows of y
      const int64_t turn = 4 * 32 * 36 * 4;                                     // the waves' output tiles
      int64_t chunk = ((96 * 1024 - 16 - 5 * 16 * steps * 4 - turn) / per32) * 32;
      chunk = chunk > 512 ? 512 : chunk;
      for (int64_t c0 = 0; c0 < n; c0 += chunk) {
        const int nn = (int)(n - c0 < chunk ? n - c0 : chunk);
        const int n_pad32 = (int)ceil_div(nn, 32) * 32;
        const size_t lds = (size_t)3 * (n_pad32 / 32) * steps * 64 * 16 + (size_t)2 * n_pad32 * 4 + 16 +
                           (size_t)5 * 16 * steps * 4 + (size_t)turn;
        const float* yc = y + c0 * k;
        float* dc = dist + c0;
        hipStream_t st = as_stream(stream);
        int rc;
        switch (steps) {
          case 1: rc = launch_split<1, 2, true>(x, yc, nullptr, nullptr, m, nn, (int)k, metric, n_pad32, lds, st, dc, n); break;
          case 2: rc = launch_split<2, 2, true>(x, yc, nullptr, nullptr, m, nn, (int)k, metric, n_pad32, lds, st, dc, n); break;
          case 3: rc = launch_split<3, 2, true>(x, yc, nullptr, nullptr, m, nn, (int)k, metric, n_pad32, lds, st, dc, n); break;
          default: rc = launch_split<4, 2, true>(x, yc, nullptr, nullptr, m, nn, (int)k, metric, n_pad32, lds, st, dc, n); break;
        }
        if (rc != 0) return rc;
      }
      return 0;
    }
  }
  const int64_t tiles = ceil_div(m, kTile) * ceil_div(n, kTile);
  const int64_t cap = (int64_t)num_cus() * 8;
  pairwise_kernel<<<(int)(tiles < cap ? tiles : cap), 256, 0, as_stream(stream)>>>(x, y, dist, m, n,
                                                                                  (int)k, metric);
  return launch_status("pairwise_distance");
}

extern "C" int f2cgt_kmeans_predict(const float* x, const float* centers, int64_t* labels_i64,
                                    uint8_t* labels_u8, int64_t m, int64_t n, int64_t k, int metric,
                                    void* stream) {
  F2CGT_REQUIRE(m >= 0 && n > 0 && k > 0, F2CGT_E_INVALID,
                "kmeans_predict: need m >= 0, n > 0 centres, k > 0 dimensions");
  F2CGT_REQUIRE(n <= 65536 && k < (1 << 20), F2CGT_E_UNSUPPORTED, "kmeans_predict: n or k too large");
  F2CGT_REQUIRE(metric == F2CGT_METRIC_L2 || metric == F2CGT_METRIC_COSINE, F2CGT_E_INVALID,
                "kmeans_predict: unknown metric %d", metric);
  F2CGT_REQUIRE(labels_u8 == nullptr || n <= 256, F2CGT_E_INVALID,
                "kmeans_predict: uint8 labels need n <= 256 centres");
  if (m == 0) return 0;
  F2CGT_REQUIRE(x && centers && (labels_i64 || labels_u8), F2CGT_E_INVALID,
                "kmeans_predict: null buffer");
  hipStream_t st = as_stream(stream);
  {  // split-bf16 path: up to 64 dimensions, operand pieces and biases within 96 KB of LDS
    const int steps = (int)ceil_div(k, 16);
    const int n_pad32 = (int)ceil_div(n, 32) * 32;
    const size_t lds = (size_t)3 * (n_pad32 / 32) * steps * 64 * 16 + (size_t)2 * n_pad32 * 4 + 16 +
                       (size_t)5 * 16 * steps * 4;
    if (steps <= 4 && lds <= 96 * 1024) {
      switch (steps) {
        case 1: return launch_split<1, 2>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad32, lds, st);
        case 2: return launch_split<2, 2>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad32, lds, st);
        case 3: return launch_split<3, 2>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad32, lds, st);
        default: return launch_split<4, 2>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad32, lds, st);
      }
    }
  }
  const int khalf = (int)((k + 1) / 2);
  int kh = pow2_ceil(khalf);
  if (kh < 4) kh = 4;
  const int n_pad = (int)ceil_div(n, 64) * 64;  // two 32-centre tiles per step
  const size_t lds = ((size_t)2 * kh * n_pad + 2 * (size_t)n_pad + 4) * sizeof(float);
  if (kh <= 32 && lds <= 96 * 1024) {
    switch (kh) {
      case 4: return launch_mfma<4>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad, lds, st);
      case 8: return launch_mfma<8>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad, lds, st);
      case 16: return launch_mfma<16>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad, lds, st);
      default: return launch_mfma<32>(x, centers, labels_i64, labels_u8, m, (int)n, (int)k, metric, n_pad, lds, st);
    }
  }
  if (m >= 64) {   // tiles of 128 rows (a handful of rows: one wave per row, exact, below)
    const int64_t tiles = ceil_div(m, (int64_t)kTile);
    const int64_t cap = (int64_t)num_cus() * 4;
    predict_tiled_kernel<<<(int)(tiles < cap ? tiles : cap), 256, 0, st>>>(x, centers, labels_i64, labels_u8, m,
                                                                         (int)n, (int)k, metric);
    return launch_status("kmeans_predict");
  }
  int64_t need = ceil_div(m, 4);
  int64_t cap = (int64_t)num_cus() * 8;
  predict_exact_kernel<<<(int)(need < cap ? need : cap), 256, 0, st>>>(x, centers, labels_i64, labels_u8, m,
                                                                      (int)n, (int)k, metric);
  return launch_status("kmeans_predict");
}
