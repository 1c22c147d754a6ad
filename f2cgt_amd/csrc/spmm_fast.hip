// Row-block kernels for the fused decompress + mean aggregation.
//
// The per-row skeleton in spmm.hip walks indptr -> indices -> code row -> store as a
// chain of dependent HBM round trips per destination row; with 2-15 edges per row that
// chain, not bandwidth, sets the run time.  Here a workgroup owns a block of consecutive
// destination rows and turns the chain into three wide phases, each one coalesced burst
// of independent loads:
//   1. indptr[row0 .. row0+RB]            -> LDS
//   2. indices[e0 .. e1)  (contiguous)    -> LDS (clamped source ids)
//   3. the packed code rows of all edges  -> LDS staging (each lane LB bytes)
//   4. decode + sum in edge order per (row, column chunk) from LDS, IEEE divide by the
//      degree, one non-temporal float4/float4x2 store; the block's output is one
//      contiguous span, written in address order.
// Several workgroups share a CU, so one block's phase 4 overlaps the loads of others.
// Blocks whose edge count exceeds the LDS staging capacity fall back to a direct
// per-row loop inside the same kernel.
#include "spmm_fast.hpp"

#include <cstdlib>
#include <cstring>

namespace f2cgt {
namespace {

constexpr int kBlock = 256;
constexpr int kStageBytes = 18 * 1024;  // LDS staging per workgroup -> 7-8 workgroups per CU
constexpr int kGatherUnroll = 8;

// Rows per block for small launches.  A block is a chain of dependent round trips, so the launch
// time is set by how many of them a CU overlaps: below `target` workgroups the blocks are shrunk to
// (at least) `floor` rows so that the grid does not fall short of a few workgroups per CU.
// Integer-accumulating kernel (128 threads, target 2048), power-law block, 400-byte output rows:
// 16384 rows 7.3 us with 56 rows per block, 5.5 us with 8; 65536 rows 10.4 / 9.5 us with 56 / 32;
// from 2.5e5 rows on the degree-based size is best.  Staged-rows kernel (256 threads, target
// 1024, at least 16 rows): 16384 rows 10.7 / 7.8 / 9.7 us with 8 / 16 / 64 rows per block.
inline int shrink_rows_per_block(int rb, int64_t R, int floor, int step, int target) {
  const int64_t want = R / target;
  int cap = (int)(want > rb ? rb : want) / step * step;
  cap = cap < floor ? floor : cap;
  return rb < cap ? rb : cap;
}

template <int LB> struct word_of;
template <> struct word_of<1> { using type = uint8_t; };
template <> struct word_of<2> { using type = uint16_t; };
template <> struct word_of<4> { using type = uint32_t; };

struct SqBlockArgs {
  const uint8_t* codes;
  const float* table;    // affine: params [2, param_stride]; log domain: codebooks [n_cb, 5]
  int64_t param_stride;  // affine only
  int64_t column_slice;  // log domain only
  int num_codebooks;     // log domain only
  int64_t R, E, N;
  int src_dim, feat_dim;
  int rows_per_block;    // RB
  int edge_cap;          // staging capacity in edges
  int pitch;             // staged bytes per edge (multiple of 4)
  int cp2;               // lanes per row = pow2 >= chunks per row
};

// Per-lane decode state for its fixed column chunk.
template <int BITS, int LB, bool AFFINE>
struct ChunkDecoder {
  static constexpr int PER = 8 / BITS;
  static constexpr int NOUT = LB * PER;
  static constexpr int NCODE = 1 << BITS;
  float mn[AFFINE ? NOUT : 1];
  float sc[AFFINE ? NOUT : 1];
  int lut_base[AFFINE ? 1 : LB];
  const float* lut;

  __device__ void init(const SqBlockArgs& a, int chunk, bool active, const float* lds_lut) {
    lut = lds_lut;
    if (AFFINE) {
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        mn[i] = active ? a.table[chunk * NOUT + i] : 0.f;
        sc[i] = active ? a.table[a.param_stride + chunk * NOUT + i] : 0.f;
      }
    } else {
#pragma unroll
      for (int b = 0; b < LB; ++b) {
        int64_t cb = ((int64_t)(chunk * LB + b) * PER) / a.column_slice;
        cb = cb < a.num_codebooks ? cb : a.num_codebooks - 1;
        lut_base[b] = (int)cb * NCODE;
      }
    }
  }
  __device__ __forceinline__ void add(uint32_t w, float (&acc)[NOUT]) const {
    if (AFFINE) {
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        const float code = (float)((w >> (BITS * i)) & (NCODE - 1));
        acc[i] += __fadd_rn(mn[i], __fmul_rn(code, sc[i]));
      }
    } else {
#pragma unroll
      for (int b = 0; b < LB; ++b) {
        const uint32_t byte = (w >> (8 * b)) & 0xffu;
#pragma unroll
        for (int k = 0; k < PER; ++k) acc[b * PER + k] += lut[lut_base[b] + ((byte >> (BITS * k)) & (NCODE - 1))];
      }
    }
  }
};

template <int NOUT>
__device__ __forceinline__ void store_chunk(float* o, const float (&acc)[NOUT], float deg) {
#pragma unroll
  for (int i = 0; i < NOUT; i += 4)
    store_nt4(o + i, acc[i] / deg, acc[i + 1] / deg, acc[i + 2] / deg, acc[i + 3] / deg);
}

template <int BITS, int LB, bool AFFINE, typename Idx>
__global__ __launch_bounds__(kBlock) void sq_block_kernel(SqBlockArgs a, const Idx* __restrict__ indptr,
                                                          const Idx* __restrict__ indices,
                                                          float* __restrict__ out) {
  using W = typename word_of<LB>::type;
  using Dec = ChunkDecoder<BITS, LB, AFFINE>;
  constexpr int NOUT = Dec::NOUT;
  extern __shared__ __align__(16) unsigned char smem[];
  // layout: [lut floats][RB+1 edge offsets int64][edge_cap ids uint32][edge_cap * pitch bytes]
  float* s_lut = reinterpret_cast<float*>(smem);
  const int lut_floats = AFFINE ? 0 : ((a.num_codebooks * Dec::NCODE + 3) & ~3);
  int64_t* s_ptr = reinterpret_cast<int64_t*>(s_lut + lut_floats);
  uint32_t* s_ids = reinterpret_cast<uint32_t*>(s_ptr + a.rows_per_block + 2);
  unsigned char* s_codes = reinterpret_cast<unsigned char*>(s_ids + a.edge_cap);

  const int t = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * a.rows_per_block;
  const int nrows = (int)((a.R - row0) < a.rows_per_block ? (a.R - row0) : a.rows_per_block);

  // phase 1: row offsets (and the LUT of the log-domain decoder)
  for (int i = t; i <= nrows; i += kBlock) {
    int64_t v = (int64_t)indptr[row0 + i];
    s_ptr[i] = v < 0 ? 0 : (v > a.E ? a.E : v);
  }
  if (!AFFINE) {
    for (int i = t; i < a.num_codebooks * Dec::NCODE; i += kBlock) {
      const float* cb = a.table + (int64_t)(i >> BITS) * 5;
      const uint32_t raw = (uint32_t)(i & (Dec::NCODE - 1));
      float v;
      if (BITS == 1) {
        v = ((float)raw - 0.5f) * (2.f * cb[4]);
      } else {
        const float drange = (float)(1 << (BITS - 1));
        const float k = __fdiv_rn(__fsub_rn(cb[3], cb[2]), drange);
        v = sq_log_decode(BITS < 8 ? (float)raw - drange : (float)(int8_t)raw, k, cb[2]);
      }
      s_lut[i] = v;
    }
  }
  const int chunks = a.feat_dim / NOUT;
  const int chunk = t & (a.cp2 - 1);
  const int slot = t / a.cp2;
  const int nslots = kBlock / a.cp2;
  const bool active = chunk < chunks;
  Dec dec;
  dec.init(a, chunk, active, s_lut);
  __syncthreads();

  const int64_t e0 = s_ptr[0];
  int64_t e1 = s_ptr[nrows];
  e1 = e1 < e0 ? e0 : e1;
  const int64_t ne64 = e1 - e0;

  if (ne64 <= a.edge_cap) {
    const int ne = (int)ne64;
    // phase 2: source ids
    for (int i = t; i < ne; i += kBlock) s_ids[i] = (uint32_t)clamp_idx(indices[e0 + i], a.N);
    __syncthreads();
    // phase 3: gather the packed rows
    if (active) {
      const uint8_t* base = a.codes + chunk * LB;
      for (int e = slot; e < ne; e += nslots * kGatherUnroll) {
        W w[kGatherUnroll];
#pragma unroll
        for (int u = 0; u < kGatherUnroll; ++u) {
          const int ee = e + u * nslots;
          if (ee < ne) w[u] = *reinterpret_cast<const W*>(base + (int64_t)s_ids[ee] * a.src_dim);
        }
#pragma unroll
        for (int u = 0; u < kGatherUnroll; ++u) {
          const int ee = e + u * nslots;
          if (ee < ne) *reinterpret_cast<W*>(s_codes + ee * a.pitch + chunk * LB) = w[u];
        }
      }
    }
    __syncthreads();
    // phase 4: decode + mean, rows in address order
    if (active) {
      for (int r = slot; r < nrows; r += nslots) {
        int b = (int)(s_ptr[r] - e0);
        int e = (int)(s_ptr[r + 1] - e0);
        b = b < 0 ? 0 : (b > ne ? ne : b);
        e = e < b ? b : (e > ne ? ne : e);
        float acc[NOUT];
#pragma unroll
        for (int i = 0; i < NOUT; ++i) acc[i] = 0.f;
        for (int k = b; k < e; ++k)
          dec.add((uint32_t)*reinterpret_cast<const W*>(s_codes + k * a.pitch + chunk * LB), acc);
        const float deg = (float)(e - b == 0 ? 1 : e - b);
        store_chunk<NOUT>(out + (row0 + r) * (int64_t)a.feat_dim + chunk * NOUT, acc, deg);
      }
    }
  } else if (active) {
    // over-capacity block: direct per-row loop
    const uint8_t* base = a.codes + chunk * LB;
    for (int r = slot; r < nrows; r += nslots) {
      int64_t b = s_ptr[r], e = s_ptr[r + 1];
      e = e < b ? b : e;
      float acc[NOUT];
#pragma unroll
      for (int i = 0; i < NOUT; ++i) acc[i] = 0.f;
      for (int64_t k = b; k < e; ++k) {
        const int64_t s = clamp_idx(indices[k], a.N);
        dec.add((uint32_t)*reinterpret_cast<const W*>(base + s * a.src_dim), acc);
      }
      const float deg = (float)(e - b == 0 ? 1 : e - b);
      store_chunk<NOUT>(out + (row0 + r) * (int64_t)a.feat_dim + chunk * NOUT, acc, deg);
    }
  }
}

template <int BITS, int LB, bool AFFINE>
int launch_sq_block(SqBlockArgs a, const void* indptr, const void* indices, int idx_dtype, float* out,
                    hipStream_t st, const char* what) {
  constexpr int NOUT = LB * (8 / BITS);
  const int chunks = a.feat_dim / NOUT;
  a.cp2 = pow2_ceil(chunks);
  // a row's chunks must fit one workgroup: with no lane group left the kernel's loops would not advance
  if (chunks < 1 || a.cp2 > kBlock) return fail(F2CGT_E_UNSUPPORTED, "%s: %d columns exceed the row-block kernel", what, a.feat_dim);
  a.pitch = (chunks * LB + 3) & ~3;
  const int lut_bytes = AFFINE ? 0 : (((a.num_codebooks << BITS) + 3) & ~3) * 4;
  a.edge_cap = kStageBytes / (a.pitch + 4);
  if (a.edge_cap > 1024) a.edge_cap = 1024;
  const double avg_deg = a.R > 0 ? (double)a.E / (double)a.R : 1.0;
  int rb = (int)(0.7 * a.edge_cap / (avg_deg > 0.5 ? avg_deg : 0.5));
  int rb2 = 4;
  while (rb2 * 2 <= rb && rb2 < 64) rb2 *= 2;
  const int min_rows = kBlock / a.cp2;  // at least one row per lane group
  a.rows_per_block = rb2 < min_rows ? min_rows : rb2;
  const size_t lds = (size_t)lut_bytes + (size_t)(a.rows_per_block + 2) * 8 + (size_t)a.edge_cap * 4 +
                     (size_t)a.edge_cap * a.pitch;
  const int64_t grid = ceil_div(a.R, a.rows_per_block);
  if (grid > 0x7fffffffll) return fail(F2CGT_E_UNSUPPORTED, "%s: too many row blocks", what);
  if (plan_only()) {
    plan_record("sq_block_kernel", grid, kBlock, (int64_t)lds, a.rows_per_block, kBlock / a.cp2, a.edge_cap);
    return 0;
  }
  if (idx_dtype == F2CGT_DT_I32)
    sq_block_kernel<BITS, LB, AFFINE, int32_t><<<(unsigned)grid, kBlock, lds, st>>>(
        a, static_cast<const int32_t*>(indptr), static_cast<const int32_t*>(indices), out);
  else
    sq_block_kernel<BITS, LB, AFFINE, int64_t><<<(unsigned)grid, kBlock, lds, st>>>(
        a, static_cast<const int64_t*>(indptr), static_cast<const int64_t*>(indices), out);
  return launch_status(what);
}


// ---- affine SQ, 4- and 8-bit codes: integer accumulation in LDS ----------------------------
// sum_e (min + c_e * scale) / deg == min + scale * (sum_e c_e) / deg, and the code sum is an
// exact integer.  The block keeps integer accumulators in LDS with the codes of a dword spread
// over fields wide enough that no field can carry into its neighbour:
//     4-bit codes, every row of the block <= 17 edges : 8-bit fields, 2 words per code dword
//     4-bit codes, <= 4369 edges per row              : 16-bit fields, 4 words per code dword
//     8-bit codes, <= 257 edges per row               : 16-bit fields, 2 words per code dword
// The gather is edge-parallel: a lane takes 8 bytes of an edge's code row with one (byte-granular,
// the hardware handles unaligned global loads) 64-bit load, splits them into fields with a few
// mask/shift operations and adds them with LDS atomics -- no per-row loop, no divergence, and
// the instruction count per edge is what bounds this kernel, not HBM.  The float work (convert,
// * 1/deg, * scale, + min) runs once per output with the column parameters held in registers.
// The result differs from "decode, then sum in fp32" by a few ulp of the summands (it is the
// closer of the two to the exact mean) and is identical to the decode for rows with one neighbour.
// A block with a row above the widest field capacity takes the direct per-output loop instead.
struct AccArgs {
  const uint8_t* codes;
  const float* params;
  int64_t param_stride;
  int64_t R, E, N;
  int src_dim, feat_dim;
  int rows_per_block;  // destination rows per workgroup
#ifdef F2CGT_EXPERIMENTS
  int64_t n_first;     // workgroups [0, n_first) take rows_per_block rows, the ones after them rows_tail
  int rows_tail;
#endif
  int sub_rows;        // rows that go through the accumulators at a time
  int wide_rows;       // ... in the layout with 4 words per code dword: sub_rows, or half of it when the LDS was sized for the narrow one
  int acc_words;       // words of the accumulator area at the start of the workgroup's LDS
  int edge_batch;
  int eff_bytes;     // leading bytes of a code row that hold output columns
  int lanes;         // 8-byte gather lanes per edge
  int lane_shift;    // log2 of the lane-group size (pow2 >= lanes)
  int pitch_n;       // accumulator words per row with 2 words per code dword
  int pitch_w;       // ... with 4 words per code dword (4-bit codes, 16-bit fields)
  int f4_per_row;    // feat_dim / 4
  int fin_group;     // finalize: lanes per row (min(f4_per_row, block))
  int fin_slots;     // finalize: rows per pass
  uint32_t fin_magic;  // ceil(2^16 / fin_group)
  int nt_out;        // output larger than the last-level cache: non-temporal stores
#ifdef F2CGT_EXPERIMENTS
  unsigned long long* trace;   // 8 words per workgroup: time stamps of its phases (100 MHz) and where it ran
#endif
};

#ifdef F2CGT_EXPERIMENTS
unsigned long long* g_acc_trace = nullptr;
#define ACC_STAMP(a, slot)                                                                  \
  do {                                                                                      \
    if ((a).trace && threadIdx.x == 0) (a).trace[(size_t)blockIdx.x * 8 + (slot)] = wall_clock64(); \
  } while (0)
#else
#define ACC_STAMP(a, slot) do {} while (0)
#endif
// A wave is given its scalar registers in units of 16 plus 16 more (measured: a kernel of 84 runs 7 waves per
// SIMD, one of 104 runs 6, one of 78 runs 8, out of 800 per SIMD).  The stamps cost about ten scalar registers;
// the stamped build is held to the 80 of the shipped one so that it keeps the same 32 workgroups per CU.
#ifdef F2CGT_EXPERIMENTS
#define F2CGT_SGPR_AS_SHIPPED __attribute__((amdgpu_num_sgpr(80)))
#else
#define F2CGT_SGPR_AS_SHIPPED
#endif

template <int TB, int BITS>
__device__ __forceinline__ void acc_direct_block(const AccArgs& a, const int* s_ptr, int64_t e0, int64_t row0,
                                              int nrows, const int64_t* idx64, const int32_t* idx32,
                                              float* __restrict__ out) {
  constexpr int PER = 8 / BITS;
  const int items = nrows * a.feat_dim;
  for (int it = threadIdx.x; it < items; it += TB) {
    const int r = it / a.feat_dim, col = it - r * a.feat_dim;
    const int64_t b = e0 + s_ptr[r], e = e0 + s_ptr[r + 1];
    uint64_t tot = 0;
    for (int64_t k = b; k < e; ++k) {
      const int64_t id = idx64 ? clamp_idx(idx64[k], a.N) : clamp_idx(idx32[k], a.N);
      const uint32_t byte = a.codes[id * a.src_dim + col / PER];
      tot += (byte >> (BITS * (col % PER))) & ((1u << BITS) - 1u);
    }
    const int64_t deg = e - b;
    const float rdeg = __builtin_amdgcn_rcpf((float)(deg > 1 ? deg : 1));
    const float v = __fadd_rn(a.params[col], __fmul_rn((float)tot * rdeg, a.params[a.param_stride + col]));
    out[(row0 + r) * (int64_t)a.feat_dim + col] = deg <= 0 ? 0.f : v;
  }
}

// ---- building blocks of the integer-accumulating kernel ----
// NW = accumulator words per code dword (see the table above).

template <int TB>
__device__ __forceinline__ void acc_zero(uint32_t* s_acc, int words) {
  for (int i = threadIdx.x; i < words >> 2; i += TB)
    reinterpret_cast<uint4*>(s_acc)[i] = make_uint4(0u, 0u, 0u, 0u);
}

// s_edge[i] = {source row id, local row} for the edges [eb, eb + nb) of the block (positions are
// relative to the block's first edge).  The ids are written edge-parallel; the local row of an
// edge is written by the thread of that row (rows [0, nr) whose range is ptr[r] .. ptr[r + 1]).
template <int TB, typename Idx>
__device__ __forceinline__ void acc_tag(const AccArgs& a, const int* ptr, int nr, int eb, int nb, int64_t e0,
                                        const Idx* __restrict__ indices, uint2* s_edge) {
  uint32_t* flat = reinterpret_cast<uint32_t*>(s_edge);
  for (int i = threadIdx.x; i < nb; i += TB)
    flat[2 * i] = (uint32_t)clamp_idx(indices[e0 + eb + i], a.N);
  for (int r = threadIdx.x; r < nr; r += TB) {
    int b = ptr[r] - eb, e = ptr[r + 1] - eb;
    b = b < 0 ? 0 : b;
    e = e > nb ? nb : e;
    for (int k = b; k < e; ++k) flat[2 * k + 1] = (uint32_t)r;
  }
}

// Adds the code fields of the tagged edges s_edge[i0 .. i1) to the accumulators; an edge of local
// row y goes to accumulator row y - row_base.
// CHUNK: a lane group takes a contiguous share of the edges instead of every gslots-th one, so that the
// groups of one instruction work on edges (and, from a handful of edges per row on, on rows) far apart:
// neighbouring edges of one long row add to the same accumulator words, and LDS atomics to one address
// are served one after the other.
template <int TB, int BITS, int NW, bool CHUNK = false>
__device__ __forceinline__ void acc_gather(const AccArgs& a, uint32_t* s_acc, const uint2* s_edge, int i0, int i1,
                                           int row_base, int pitch) {
  constexpr uint32_t M = NW == 4 ? 0x000f000fu : (BITS == 4 ? 0x0f0f0f0fu : 0x00ff00ffu);
  constexpr int S = BITS == 4 ? 4 : 8;  // shift between the words of one code dword
  const int t = threadIdx.x;
  const int lanes = a.lanes;
  // lane j of a group covers row bytes [8j, 8j+8); the last lane's load is moved back so that it
  // ends with the row's useful bytes, and shifted so that everything past them reads as 0
  const int j = t & ((1 << a.lane_shift) - 1);
  const int gslot = t >> a.lane_shift;
  const int gslots = TB >> a.lane_shift;
  const bool lane_on = j < lanes;
  const int want_off = lane_on ? 8 * j : 0;
  const int off = want_off < a.eff_bytes - 8 ? want_off : a.eff_bytes - 8;
  const int sh = (want_off - off) * 8;
  uint32_t* accj = s_acc + j - row_base * pitch;
  constexpr int U = 4;
  if (!lane_on) return;
  uint32_t keep = 0;
  const int per = CHUNK ? (i1 - i0 + gslots - 1) / gslots : 0;
  const int first_e = CHUNK ? i0 + gslot * per : i0 + gslot;
  const int last_e = CHUNK ? ((first_e + per) < i1 ? (first_e + per) : i1) : i1;   // one past this group's last edge
  const int su = CHUNK ? 1 : gslots;                                               // from one load of a trip to the next
  for (int e = first_e; e < last_e; e += su * U) {
    uint2 ed[U];
    uint64_t w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int ee = e + u * su;
      ee = ee < last_e ? ee : last_e - 1;
      ed[u] = s_edge[ee];
      __builtin_memcpy(&w[u], a.codes + ((uint64_t)ed[u].x * (uint32_t)a.src_dim + (uint32_t)off), 8);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // The unconditional use keeps every load up here, issued back to back; a load whose only
      // use sits in the branch below is moved into it by the compiler and waited for on its own.
      keep ^= (uint32_t)w[u];
      if (u == 0 || e + u * su < last_e) {
        const uint64_t v = w[u] >> sh;
        const uint32_t d0 = (uint32_t)v, d1 = (uint32_t)(v >> 32);
        uint32_t* acc = accj + (int)ed[u].y * pitch;
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          atomicAdd(acc + k * lanes, (d0 >> (S * k)) & M);
          atomicAdd(acc + (NW + k) * lanes, (d1 >> (S * k)) & M);
        }
      }
    }
  }
  if (keep == 0x9e3779b9u && a.eff_bytes < 0) s_acc[0] = keep;  // never true; gives `keep` a use
}

// Means of the rows [rb, rb + nr) of the block from the accumulator rows [0, nr): a lane keeps
// one float4 column group (its parameters in registers) and walks the rows.
// min / scale of a lane's first column group, fetched when the kernel starts: the loads would
// otherwise sit behind the last barrier of a block, one more round trip in its dependent chain.
struct FinParams {
  float mn[4], sc[4];
};

// HALF != 0: rows of 4 k + 2 columns.  They start at multiples of 8 bytes only and end with a group of two columns:
// that group's parameters are fetched column by column (nothing is read past the row's last column), the 16-byte
// stores go to any dword, and the last group stores its two columns alone.  HALF is 1 for cached and 2 for streamed
// stores, fixed when the kernel is chosen: with both forms of the under-aligned store behind one run-time test the
// compiler folds them into one and the streamed form is lost.
template <int HALF = 0>
__device__ __forceinline__ FinParams acc_fin_params(const AccArgs& a) {
  FinParams p;
  const int t = threadIdx.x;
  const int g = (int)(((uint32_t)t * a.fin_magic) >> 16);
  const int l = t - g * a.fin_group;
  const int c4 = (g < a.fin_slots && l < a.f4_per_row) ? l : 0;
  if (HALF == 0 || c4 * 4 + 4 <= a.feat_dim) {   // four consecutive parameters: one load each for min and scale
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p.mn[i] = a.params[c4 * 4 + i];
      p.sc[i] = a.params[a.param_stride + c4 * 4 + i];
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = c4 * 4 + i >= a.feat_dim ? a.feat_dim - 1 : c4 * 4 + i;
      p.mn[i] = a.params[col];
      p.sc[i] = a.params[a.param_stride + col];
    }
  }
  return p;
}

template <int TB, int BITS, int NW, int HALF = 0>
__device__ __forceinline__ void acc_finalize(const AccArgs& a, const FinParams& first, const uint32_t* s_acc,
                                             const float* s_rdeg, int64_t row0, int rb, int nr, int pitch,
                                             float* __restrict__ out) {
  const int t = threadIdx.x;
  const int lanes = a.lanes;
  const int g = (int)(((uint32_t)t * a.fin_magic) >> 16);
  const int l = t - g * a.fin_group;
  if (g >= a.fin_slots) return;
  for (int c4 = l; c4 < a.f4_per_row; c4 += a.fin_group) {
    float mn[4], sc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      mn[i] = first.mn[i];
      sc[i] = first.sc[i];
    }
    if (c4 != l) {
      if (HALF == 0 || c4 * 4 + 4 <= a.feat_dim) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          mn[i] = a.params[c4 * 4 + i];
          sc[i] = a.params[a.param_stride + c4 * 4 + i];
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int col = c4 * 4 + i >= a.feat_dim ? a.feat_dim - 1 : c4 * 4 + i;
          mn[i] = a.params[col];
          sc[i] = a.params[a.param_stride + col];
        }
      }
    }
    const bool half_group = HALF != 0 && c4 * 4 + 2 == a.feat_dim;
    const int d = BITS == 4 ? (c4 >> 1) : c4;     // code dword that holds these 4 columns
    const int fsh = BITS == 4 ? (c4 & 1) * 16 : 0;
    const uint32_t* accd = s_acc + ((d & 1) * NW) * lanes + (d >> 1);
    float* o = out + ((row0 + rb) * (int64_t)a.feat_dim + c4 * 4);
    for (int r = g; r < nr; r += a.fin_slots) {
      const uint32_t* ar = accd + r * pitch;
      float s0, s1, s2, s3;
      if (NW == 4) {
        s0 = (float)((ar[0] >> fsh) & 0xffffu);
        s1 = (float)((ar[lanes] >> fsh) & 0xffffu);
        s2 = (float)((ar[2 * lanes] >> fsh) & 0xffffu);
        s3 = (float)((ar[3 * lanes] >> fsh) & 0xffffu);
      } else if (BITS == 4) {
        const uint32_t w0 = ar[0] >> fsh, w1 = ar[lanes] >> fsh;
        s0 = (float)(w0 & 0xffu);
        s1 = (float)(w1 & 0xffu);
        s2 = (float)((w0 >> 8) & 0xffu);
        s3 = (float)((w1 >> 8) & 0xffu);
      } else {
        const uint32_t w0 = ar[0], w1 = ar[lanes];
        s0 = (float)(w0 & 0xffffu);
        s1 = (float)(w1 & 0xffffu);
        s2 = (float)(w0 >> 16);
        s3 = (float)(w1 >> 16);
      }
      const float rdeg = s_rdeg[rb + r];  // 0 marks an empty row, rcp(1) == 1 exactly
      float v0 = __fadd_rn(mn[0], __fmul_rn(s0 * rdeg, sc[0]));
      float v1 = __fadd_rn(mn[1], __fmul_rn(s1 * rdeg, sc[1]));
      float v2 = __fadd_rn(mn[2], __fmul_rn(s2 * rdeg, sc[2]));
      float v3 = __fadd_rn(mn[3], __fmul_rn(s3 * rdeg, sc[3]));
      if (rdeg == 0.f) v0 = v1 = v2 = v3 = 0.f;
      // plain stores: rows are not cache-line multiples in general, and the L2 merges the partial
      // lines that neighbouring waves write before they go to HBM
      if constexpr (HALF != 0) {
        float* dst = o + (int64_t)r * a.feat_dim;
        if (half_group) {
          if constexpr (HALF == 2) store_nt2(dst, v0, v1);
          else *reinterpret_cast<float2*>(dst) = make_float2(v0, v1);
        } else {
          if constexpr (HALF == 2) store_nt4_align8(dst, v0, v1, v2, v3);
          else store4_align8(dst, v0, v1, v2, v3);
        }
      } else {
        if (a.nt_out) store_nt4(o + (int64_t)r * a.feat_dim, v0, v1, v2, v3);
        else *reinterpret_cast<float4*>(o + (int64_t)r * a.feat_dim) = make_float4(v0, v1, v2, v3);
      }
    }
  }
}

// All rows of the block, `sub` rows at a time through the accumulators.
template <int TB, int BITS, int NW, typename Idx, bool CHUNK = false, int HALF = 0>
__device__ __forceinline__ void acc_block(const AccArgs& a, const FinParams& first, uint32_t* s_acc, const int* s_ptr,
                                          const float* s_rdeg, uint2* s_edge, int64_t e0, int64_t row0, int nrows,
                                          const Idx* __restrict__ indices, float* __restrict__ out) {
  const int pitch = NW == 4 ? a.pitch_w : a.pitch_n;
  const int sub = NW == 4 ? a.wide_rows : a.sub_rows;
  const int ne = s_ptr[nrows];
  if (ne <= a.edge_batch) {
    // common case: every edge of the block is tagged once, up front
    acc_tag<TB>(a, s_ptr, nrows, 0, ne, e0, indices, s_edge);
    acc_zero<TB>(s_acc, (nrows < sub ? nrows : sub) * pitch);
    __syncthreads();
    ACC_STAMP(a, 2);
    for (int sb = 0; sb < nrows; sb += sub) {
      const int nr = (nrows - sb) < sub ? (nrows - sb) : sub;
      acc_gather<TB, BITS, NW, CHUNK>(a, s_acc, s_edge, s_ptr[sb], s_ptr[sb + nr], sb, pitch);
      __syncthreads();
      if (sb == 0) ACC_STAMP(a, 3);
      acc_finalize<TB, BITS, NW, HALF>(a, first, s_acc, s_rdeg, row0, sb, nr, pitch, out);
      if (sb + sub < nrows) {
        __syncthreads();
        acc_zero<TB>(s_acc, sub * pitch);
        __syncthreads();
      }
    }
  } else {
    for (int sb = 0; sb < nrows; sb += sub) {
      const int nr = (nrows - sb) < sub ? (nrows - sb) : sub;
      const int* ptr = s_ptr + sb;
      if (sb) __syncthreads();
      acc_zero<TB>(s_acc, nr * pitch);
      for (int eb = ptr[0]; eb < ptr[nr]; eb += a.edge_batch) {
        const int nb = (ptr[nr] - eb) < a.edge_batch ? (ptr[nr] - eb) : a.edge_batch;
        if (eb != ptr[0]) __syncthreads();
        acc_tag<TB>(a, ptr, nr, eb, nb, e0, indices, s_edge);
        __syncthreads();
        acc_gather<TB, BITS, NW, CHUNK>(a, s_acc, s_edge, 0, nb, 0, pitch);
      }
      __syncthreads();
      acc_finalize<TB, BITS, NW, HALF>(a, first, s_acc, s_rdeg, row0, sb, nr, pitch, out);
    }
  }
}

template <int TB, int BITS, typename Idx, bool CHUNK = false, int HALF = 0>
__global__ __launch_bounds__(TB) void sq_affine_acc_kernel(AccArgs a, const Idx* __restrict__ indptr,
                                                               const Idx* __restrict__ indices,
                                                               float* __restrict__ out) {
  constexpr int CAP_N = BITS == 4 ? 17 : 257;     // edges per row: 2 accumulator words per code dword
  constexpr int CAP_W = BITS == 4 ? 4369 : 257;   // 4 words per code dword (4-bit codes only)
  extern __shared__ __align__(16) unsigned char smem[];
  uint32_t* s_acc = reinterpret_cast<uint32_t*>(smem);                         // [sub_rows][pitch_n] or [wide_rows][pitch_w]
  int* s_ptr = reinterpret_cast<int*>(s_acc + a.acc_words);                    // [RB + 1]
  float* s_rdeg = reinterpret_cast<float*>(s_ptr + a.rows_per_block + 4);      // [RB]
  uint32_t* s_wflag = reinterpret_cast<uint32_t*>(s_rdeg + a.rows_per_block);  // [waves]
  uint2* s_edge = reinterpret_cast<uint2*>(s_wflag + 4);          // [edge_batch]

  const int t = threadIdx.x;
  ACC_STAMP(a, 0);
#ifdef F2CGT_EXPERIMENTS
  const bool tail_block = (int64_t)blockIdx.x >= a.n_first;
  const int row_cap = tail_block ? a.rows_tail : a.rows_per_block;
  const int64_t row0 = tail_block ? a.n_first * a.rows_per_block + ((int64_t)blockIdx.x - a.n_first) * a.rows_tail
                                  : (int64_t)blockIdx.x * a.rows_per_block;
#else
  const int row_cap = a.rows_per_block;
  const int64_t row0 = (int64_t)blockIdx.x * a.rows_per_block;
#endif
  const int nrows = (int)((a.R - row0) < row_cap ? (a.R - row0) : row_cap);
  const FinParams first = acc_fin_params<HALF>(a);
  int64_t e0 = (int64_t)indptr[row0];
  e0 = e0 < 0 ? 0 : (e0 > a.E ? a.E : e0);
  uint32_t level = 0;
  for (int i = t; i <= nrows; i += TB) {
    int64_t v = (int64_t)indptr[row0 + i];
    v = v < e0 ? e0 : (v > a.E ? a.E : v);
    const int p = (int)(v - e0 > 0x7fffffff ? 0x7fffffff : v - e0);
    s_ptr[i] = p;
    if (i < nrows) {
      int64_t v2 = (int64_t)indptr[row0 + i + 1];
      v2 = v2 < e0 ? e0 : (v2 > a.E ? a.E : v2);
      const int deg = (int)(v2 - e0 > 0x7fffffff ? 0x7fffffff : v2 - e0) - p;
      s_rdeg[i] = deg > 0 ? __builtin_amdgcn_rcpf((float)deg) : 0.f;
      level |= (deg > CAP_N ? 1u : 0u) | (deg > CAP_W ? 2u : 0u);
    }
  }
  {
    const uint32_t wl = (__ballot(level & 1u) ? 1u : 0u) | (__ballot(level & 2u) ? 2u : 0u);
    if ((t & (kWave - 1)) == 0) s_wflag[t / kWave] = wl;
  }
  __syncthreads();
  ACC_STAMP(a, 1);
  uint32_t block_level = 0;
#pragma unroll
  for (int w = 0; w < TB / kWave; ++w) block_level |= s_wflag[w];
  if (block_level & 2u) {
    const bool is64 = sizeof(Idx) == 8;
    acc_direct_block<TB, BITS>(a, s_ptr, e0, row0, nrows,
                           is64 ? reinterpret_cast<const int64_t*>(indices) : nullptr,
                           is64 ? nullptr : reinterpret_cast<const int32_t*>(indices), out);
    return;
  }
  if (BITS == 4 && (block_level & 1u))
    acc_block<TB, BITS, 4, Idx, CHUNK, HALF>(a, first, s_acc, s_ptr, s_rdeg, s_edge, e0, row0, nrows, indices, out);
  else
    acc_block<TB, BITS, 2, Idx, CHUNK, HALF>(a, first, s_acc, s_ptr, s_rdeg, s_edge, e0, row0, nrows, indices, out);
  ACC_STAMP(a, 4);
#ifdef F2CGT_EXPERIMENTS
  if (a.trace && threadIdx.x == 0) {
    a.trace[(size_t)blockIdx.x * 8 + 5] = __builtin_amdgcn_s_getreg((31 << 11) | 4);    // HW_ID
    a.trace[(size_t)blockIdx.x * 8 + 6] = __builtin_amdgcn_s_getreg((31 << 11) | 20);   // XCC_ID
  }
#endif
}

#ifdef F2CGT_EXPERIMENTS
// ---- persistent form (measured, not adopted) ---------------------------------------------------
// A block's life is a chain of dependent memory round trips (indptr -> indices -> code rows) before
// its first store, and with 2-10 edges per row the launch is over after two or three such chains per
// workgroup slot.  Here a workgroup walks the blocks blk, blk + grid, ... and fetches the row
// offsets and the source ids of its next block into registers while the current one gathers and
// stores, so only the code-row fetch of every block after the first stays on the critical path.
// The barriers order LDS traffic only (a workgroup-scope fence on the whole address space would
// drain the loads in flight at every barrier).  On the 2.5e5-row power-law block it ran at 24.4 us
// against 23.1 us for one workgroup per block: the hardware already starts a new workgroup the
// moment a slot frees, and 13-14 of them per CU overlap their chains as well as the prefetch does.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int TB, int BITS, typename Idx>
__global__ __launch_bounds__(TB) void sq_affine_acc_pkernel(AccArgs a, const Idx* __restrict__ indptr,
                                                            const Idx* __restrict__ indices,
                                                            float* __restrict__ out) {
  constexpr int CAP_N = BITS == 4 ? 17 : 257;
  constexpr int CAP_W = BITS == 4 ? 4369 : 257;
  constexpr int NID = 2;   // prefetched source ids per thread: edge_batch = NID * TB
  extern __shared__ __align__(16) unsigned char smem[];
  uint32_t* s_acc = reinterpret_cast<uint32_t*>(smem);                         // [sub_rows][pitch_n] or [wide_rows][pitch_w]
  int* s_ptr = reinterpret_cast<int*>(s_acc + a.acc_words);                    // [RB + 1]
  float* s_rdeg = reinterpret_cast<float*>(s_ptr + a.rows_per_block + 4);      // [RB]
  uint32_t* s_wflag = reinterpret_cast<uint32_t*>(s_rdeg + a.rows_per_block);  // [waves]
  uint2* s_edge = reinterpret_cast<uint2*>(s_wflag + 4);                       // [edge_batch]

  const int t = threadIdx.x;
  const int rb = a.rows_per_block;       // rb + 1 <= TB: one row offset per thread
  const int64_t nblocks = (a.R + rb - 1) / rb;
  const FinParams first = acc_fin_params(a);
  const int64_t e_last = a.E > 0 ? a.E - 1 : 0;

  // row offsets of a block, one per thread, plus its first and last offset for everybody
  Idx p_lo = 0, p_hi = 0, p_e0 = 0, p_end = 0;
  auto fetch_ptr = [&](int64_t blk) {
    const int64_t row0 = blk * rb;
    const int nr = (int)((a.R - row0) < rb ? (a.R - row0) : rb);
    const int i = t <= nr ? t : nr;
    p_lo = indptr[row0 + i];
    p_hi = indptr[row0 + (i < nr ? i + 1 : nr)];
    p_e0 = indptr[row0];
    p_end = indptr[row0 + nr];
  };
  Idx ids[NID];
#pragma unroll
  for (int j = 0; j < NID; ++j) ids[j] = 0;
  bool ids_ready = false;   // ids[] hold the first edges of the block about to start

  int64_t blk = blockIdx.x;
  if (blk < nblocks) fetch_ptr(blk);
  for (; blk < nblocks; blk += gridDim.x) {
    const int64_t row0 = blk * rb;
    const int nrows = (int)((a.R - row0) < rb ? (a.R - row0) : rb);
    int64_t e0 = (int64_t)p_e0;
    e0 = e0 < 0 ? 0 : (e0 > a.E ? a.E : e0);
    uint32_t level = 0;
    if (t <= nrows) {
      int64_t v = (int64_t)p_lo;
      v = v < e0 ? e0 : (v > a.E ? a.E : v);
      const int p = (int)(v - e0 > 0x7fffffff ? 0x7fffffff : v - e0);
      s_ptr[t] = p;
      if (t < nrows) {
        int64_t v2 = (int64_t)p_hi;
        v2 = v2 < e0 ? e0 : (v2 > a.E ? a.E : v2);
        const int deg = (int)(v2 - e0 > 0x7fffffff ? 0x7fffffff : v2 - e0) - p;
        s_rdeg[t] = deg > 0 ? __builtin_amdgcn_rcpf((float)deg) : 0.f;
        level = (deg > CAP_N ? 1u : 0u) | (deg > CAP_W ? 2u : 0u);
      }
    }
    {
      const uint32_t wl = (__ballot(level & 1u) ? 1u : 0u) | (__ballot(level & 2u) ? 2u : 0u);
      if ((t & (kWave - 1)) == 0) s_wflag[t / kWave] = wl;
    }
    // the row offsets of the next block start their trip now
    const int64_t next = blk + gridDim.x;
    const bool has_next = next < nblocks;
    if (has_next) fetch_ptr(next);
    lds_barrier();
    uint32_t block_level = 0;
#pragma unroll
    for (int w = 0; w < TB / kWave; ++w) block_level |= s_wflag[w];
    const int ne = s_ptr[nrows];
    const bool simple = block_level == 0 && ne <= a.edge_batch && nrows <= a.sub_rows;
    if (simple) {
      // every edge of the block is tagged once; the ids come from the registers when they were prefetched
      uint32_t* flat = reinterpret_cast<uint32_t*>(s_edge);
#pragma unroll
      for (int j = 0; j < NID; ++j) {
        const int i = t + j * TB;
        if (i < ne) {
          const Idx raw = ids_ready ? ids[j] : indices[e0 + i];
          flat[2 * i] = (uint32_t)clamp_idx(raw, a.N);
        }
      }
      if (t < nrows) {
        const int b = s_ptr[t], e = s_ptr[t + 1];
        for (int k = b; k < e; ++k) flat[2 * k + 1] = (uint32_t)t;
      }
      acc_zero<TB>(s_acc, nrows * a.pitch_n);
      lds_barrier();
      acc_gather<TB, BITS, 2>(a, s_acc, s_edge, 0, ne, 0, a.pitch_n);
    } else {
      lds_barrier();   // (keeps the barrier count of the two branches equal)
    }
    // the source ids of the next block: its offsets have had the gather to arrive
    ids_ready = false;
    if (has_next) {
      int64_t e0n = (int64_t)p_e0, e1n = (int64_t)p_end;
      e0n = e0n < 0 ? 0 : (e0n > a.E ? a.E : e0n);
      e1n = e1n < e0n ? e0n : (e1n > a.E ? a.E : e1n);
      if (e1n - e0n <= a.edge_batch) {
        ids_ready = true;
#pragma unroll
        for (int j = 0; j < NID; ++j) {
          int64_t at = e0n + t + j * TB;
          at = at > e_last ? e_last : at;
          ids[j] = indices[at];
        }
      }
    }
    if (simple) {
      lds_barrier();
      acc_finalize<TB, BITS, 2>(a, first, s_acc, s_rdeg, row0, 0, nrows, a.pitch_n, out);
    } else if (block_level & 2u) {
      const bool is64 = sizeof(Idx) == 8;
      acc_direct_block<TB, BITS>(a, s_ptr, e0, row0, nrows,
                                 is64 ? reinterpret_cast<const int64_t*>(indices) : nullptr,
                                 is64 ? nullptr : reinterpret_cast<const int32_t*>(indices), out);
    } else if (BITS == 4 && (block_level & 1u)) {
      acc_block<TB, BITS, 4, Idx>(a, first, s_acc, s_ptr, s_rdeg, s_edge, e0, row0, nrows, indices, out);
    } else {
      acc_block<TB, BITS, 2, Idx>(a, first, s_acc, s_ptr, s_rdeg, s_edge, e0, row0, nrows, indices, out);
    }
    lds_barrier();   // the block's LDS is reused by the next one
  }
}

#endif  // F2CGT_EXPERIMENTS

#ifdef F2CGT_EXPERIMENTS
static bool acc_persistent_enabled() {   // F2CGT_ACC_PERSIST=1 selects the persistent form
  const char* v = getenv("F2CGT_ACC_PERSIST");
  return v != nullptr && v[0] == '1';
}
#endif

template <int TB, int BITS>
int launch_acc_tb(AccArgs a, size_t lds, int64_t grid, const void* indptr, const void* indices, int idx_dtype,
                  float* out, hipStream_t st, const char* what) {
  a.fin_group = a.f4_per_row < TB ? a.f4_per_row : TB;
  a.fin_slots = TB / a.fin_group;
  a.fin_magic = (uint32_t)((65536 + a.fin_group - 1) / a.fin_group);
  a.nt_out = stream_output(a.R * (int64_t)a.feat_dim * 4, (int64_t)a.feat_dim * 4,
                           a.R > 0 ? (double)a.E / (double)a.R : 0.0) ? 1 : 0;
#ifdef F2CGT_EXPERIMENTS
  a.trace = g_acc_trace;
  if (const char* v = getenv("F2CGT_ACC_RESIDENT")) {   // at most this many workgroups per CU, by padding the LDS request
    const int n = atoi(v);
    if (n >= 1 && n <= 32) {
      const size_t want = (size_t)(160 * 1024 / n / 1280) * 1280;
      if (want > lds) lds = want;
    }
  }
#endif
  if (plan_only()) {
    plan_record("sq_affine_acc_kernel", grid, TB, (int64_t)lds, a.rows_per_block, a.fin_slots, TB >> a.lane_shift,
                a.sub_rows, a.edge_batch);
    return 0;
  }
#ifdef F2CGT_EXPERIMENTS
  if (a.rows_per_block + 1 <= TB && a.edge_batch == 2 * TB && a.feat_dim % 4 == 0 && acc_persistent_enabled()) {
    // as many workgroups as the device holds at once (LDS bound), each walking blocks grid apart
    int64_t per_cu = lds > 0 ? (int64_t)(160 * 1024) / (int64_t)lds : 16;
    per_cu = per_cu > 2048 / TB ? 2048 / TB : (per_cu < 1 ? 1 : per_cu);
    int64_t pgrid = per_cu * num_cus();
    pgrid = pgrid > grid ? grid : pgrid;
    if (idx_dtype == F2CGT_DT_I32)
      sq_affine_acc_pkernel<TB, BITS, int32_t><<<(unsigned)pgrid, TB, lds, st>>>(
          a, static_cast<const int32_t*>(indptr), static_cast<const int32_t*>(indices), out);
    else
      sq_affine_acc_pkernel<TB, BITS, int64_t><<<(unsigned)pgrid, TB, lds, st>>>(
          a, static_cast<const int64_t*>(indptr), static_cast<const int64_t*>(indices), out);
    return launch_status(what);
  }
#endif
  // contiguous shares of the edges per lane group from six edges per row on (see acc_gather)
  bool chunk = a.R > 0 && (double)a.E >= 6.0 * (double)a.R;
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_ACC_CHUNK")) chunk = atoi(v) != 0;
#endif
  const int half = a.feat_dim % 4 == 0 ? 0 : (a.nt_out ? 2 : 1);   // 4 k + 2 columns: cached or streamed stores
#define F2CGT_ACC_GO(I, C, H)                                                   \
  sq_affine_acc_kernel<TB, BITS, I, C, H><<<(unsigned)grid, TB, lds, st>>>(     \
      a, static_cast<const I*>(indptr), static_cast<const I*>(indices), out)
#define F2CGT_ACC_HALF(I, C)                                                    \
  do {                                                                          \
    if (half == 0) F2CGT_ACC_GO(I, C, 0);                                       \
    else if (half == 1) F2CGT_ACC_GO(I, C, 1);                                  \
    else F2CGT_ACC_GO(I, C, 2);                                                 \
  } while (0)
#define F2CGT_ACC_IDX(I)                                                        \
  do {                                                                          \
    if (chunk) F2CGT_ACC_HALF(I, true);                                         \
    else F2CGT_ACC_HALF(I, false);                                              \
  } while (0)
  if (idx_dtype == F2CGT_DT_I32) F2CGT_ACC_IDX(int32_t);
  else F2CGT_ACC_IDX(int64_t);
#undef F2CGT_ACC_IDX
#undef F2CGT_ACC_HALF
#undef F2CGT_ACC_GO
  return launch_status(what);
}

// Block geometry for TB-thread workgroups, then the launch.
template <int TB, int BITS>
int launch_acc_sized(AccArgs a, double dg, size_t acc_row, const void* indptr, const void* indices, int idx_dtype,
                     float* out, hipStream_t st, const char* what) {
  a.edge_batch = 2 * TB;
  int sub = ((int)(TB / dg) + 4) / 8 * 8;  // ~one edge per thread and sub-block, multiple of 8 rows
  sub = sub < 8 ? 8 : (sub > 64 ? 64 : sub);
  // Eight rows of 11-20 edges leave a 128-thread workgroup with less than an edge per thread; sixteen
  // measured 8-22 % faster there (11 edges per row, 128 columns: 65 -> 51 us at 4 bit, 66 -> 58 at 8 bit;
  // 14: 57 -> 49 and 60 -> 52; 20: 93 -> 90 and level), and level above.
  if (sub < 16 && dg <= 20.0) sub = 16;
  while (sub > 8 && sub * acc_row > 24 * 1024) sub -= 8;
  int rb = sub * (int)(0.6 * a.edge_batch / (dg * sub));
  rb = rb < sub ? sub : (rb > 256 ? 256 / sub * sub : rb);
  {
    const int small = shrink_rows_per_block(rb, a.R, 8, 8, 2048);
    if (small < rb) {
      rb = small;
      sub = sub > rb ? rb : sub;
      rb = rb / sub * sub;
    }
  }
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_ACC_RB")) {   // rows per block, a multiple of 8
    const int want = atoi(v);
    if (want >= 8) { sub = want / 8 * 8; rb = sub; }
  }
  if (const char* v = getenv("F2CGT_ACC_SUB")) {   // rows through the accumulators at a time; F2CGT_ACC_RB then a multiple of it
    const int want = atoi(v);
    const char* r = getenv("F2CGT_ACC_RB");
    if (want >= 8 && r) { sub = want / 8 * 8; rb = atoi(r) / sub * sub; if (rb < sub) rb = sub; }
  }
#endif
  a.rows_per_block = rb;
  a.sub_rows = sub;
  a.wide_rows = acc_row >= (size_t)a.pitch_w * 4 ? sub : sub >> 1;
  a.acc_words = (int)(sub * acc_row / 4);
  const size_t lds = sub * acc_row + (size_t)(rb + 4) * 4 + (size_t)rb * 4 + 16 + (size_t)a.edge_batch * 8 + 16;
  int64_t grid = ceil_div(a.R, rb);
#ifdef F2CGT_EXPERIMENTS
  a.n_first = grid;
  a.rows_tail = rb;
  if (const char* v = getenv("F2CGT_ACC_TAIL")) {   // "<n_first>:<rows_tail>"
    const long long nf = atoll(v);
    const char* c = strchr(v, ':');
    const int rt = c ? atoi(c + 1) / 8 * 8 : 0;
    if (nf > 0 && nf < grid && rt >= 8 && rt <= rb) {
      a.n_first = nf;
      a.rows_tail = rt;
      grid = nf + ceil_div(a.R - nf * rb, rt);
    }
  }
#endif
  if (grid > 0x7fffffffll) return fail(F2CGT_E_UNSUPPORTED, "%s: too many row blocks", what);
  return launch_acc_tb<TB, BITS>(a, lds, grid, indptr, indices, idx_dtype, out, st, what);
}

template <int BITS>
int launch_acc(AccArgs a, const void* indptr, const void* indices, int idx_dtype, float* out, hipStream_t st,
               const char* what) {
  a.eff_bytes = (int)ceil_div(a.feat_dim, 8 / BITS);
  a.lanes = (int)ceil_div(a.eff_bytes, 8);
  const int lanes2 = pow2_ceil(a.lanes);
  a.lane_shift = 0;
  while ((1 << a.lane_shift) < lanes2) ++a.lane_shift;
  // rows of the accumulator array start lanes2 banks apart so that the lane groups of a wave,
  // which mostly work on neighbouring rows, spread over all 32 banks
  const int skew = lanes2 % 32;
  a.pitch_n = ((4 * a.lanes + 31) / 32 * 32 + skew + 3) & ~3;
  a.pitch_w = ((8 * a.lanes + 31) / 32 * 32 + skew + 3) & ~3;
#ifdef F2CGT_EXPERIMENTS
  if (getenv("F2CGT_ACC_PITCH")) {   // rows packed: the 64 banks spread them as long as the pitch is not a multiple of 16 words
    a.pitch_n = 4 * a.lanes + ((4 * a.lanes) % 16 == 0 ? 4 : 0);
    a.pitch_w = 8 * a.lanes + ((8 * a.lanes) % 16 == 0 ? 4 : 0);
  }
#endif
  a.f4_per_row = (a.feat_dim + 3) / 4;
  const double avg_deg = a.R > 0 ? (double)a.E / (double)a.R : 1.0;
  const double dg = avg_deg > 0.5 ? avg_deg : 0.5;
  // Sized for the narrow layout, the accumulators take the wide one (4-bit codes, a row of more than 17
  // edges in the block) on half the rows at a time, so it must fit twice into the narrow one.  From nine
  // edges per row on average such blocks are the rule: the accumulators are then sized for the wide layout
  // and a block stays one pass (18 / 20 / 25 edges per row, 128 columns: 87 / 91 / 88 us in two passes).
  bool expect_wide = BITS == 4 && dg >= 9.0;
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_ACC_WIDE_FULL")) expect_wide = BITS == 4 && atoi(v) != 0;
#endif
  const size_t acc_row = expect_wide ? (size_t)(a.pitch_w > a.pitch_n ? a.pitch_w : a.pitch_n) * 4
                                     : (size_t)(a.pitch_n * 2 > a.pitch_w ? a.pitch_n : (a.pitch_w + 1) / 2) * 4;
  // 128-thread workgroups: more, smaller blocks in flight per CU overlap the dependent
  // indptr -> indices -> code-row loads of one block with the output stores of others
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_ACC_TB")) {   // workgroup size for an A/B: 64 or 256
    if (atoi(v) == 64) return launch_acc_sized<64, BITS>(a, dg, acc_row, indptr, indices, idx_dtype, out, st, what);
    if (atoi(v) == 256) return launch_acc_sized<256, BITS>(a, dg, acc_row, indptr, indices, idx_dtype, out, st, what);
  }
#endif
  return launch_acc_sized<128, BITS>(a, dg, acc_row, indptr, indices, idx_dtype, out, st, what);
}


// ---- log-domain (LUT) and 1-/2-bit affine SQ: staged rows, sequential fp32 sums ------------
// Same block phases as above with 128- or 256-thread workgroups, but the decode is not linear in the
// code, so the sums stay in fp32 and in edge order: the code rows of the block's edges are staged
// in LDS by the edge-parallel 8-byte gather, then a lane that owns one float4 column group (LUT
// bases or affine parameters in registers) walks its rows' edges from LDS.  The mean is the
// correctly rounded quotient (reciprocal refined by FMAs), i.e. what `sum / deg` gives.
struct RowsArgs {
  const uint8_t* codes;
  const float* table;    // affine: params [2, param_stride]; log domain: codebooks [n_cb, 5]
  int64_t param_stride;
  int64_t column_slice;
  int num_codebooks;
  int64_t R, E, N;
  int src_dim, feat_dim;
  int rows_per_block, edge_cap;
  int eff_bytes, pitch;  // useful bytes of a code row; staged bytes per edge (multiple of 8)
  int lanes, lane_shift;
  int f4_per_row, fin_group, fin_slots;
  uint32_t fin_magic;
  int nt_out;            // output larger than the last-level cache: non-temporal stores
};


__device__ __forceinline__ float mean_of(float sum, float d, float r) {
  const float q = sum * r;
  return __fmaf_rn(__fmaf_rn(-q, d, sum), r, q);
}

// HALF: 0, or 1 / 2 for output rows at any multiple of 8 bytes, possibly with a last group of two columns (rows of
// 4 k + 2 columns), written with cached / streamed stores (see acc_fin_params).  4- and 8-bit rows always take 1 or 2:
// with the store form fixed at compile time the row loop came out 3-5 % faster at 100-256 columns and 17-19 % at 600
// (3e6 edges, 10 per row, 4 bit: 97.8 -> 93.7 us at 128 columns, 592 -> 489 us at 600); 1- and 2-bit rows measured
// level to 2 % slower and keep the run-time test.
template <int BITS, bool AFFINE, typename Idx, int TB, int HALF = 0>
__global__ __launch_bounds__(TB) void sq_rows_kernel(RowsArgs a, const Idx* __restrict__ indptr,
                                                             const Idx* __restrict__ indices,
                                                             float* __restrict__ out) {
  constexpr int NK = (64 + TB - 1) / TB;   // rows of a block (at most 64) per thread in the sorting steps
  constexpr int PER = 8 / BITS;
  constexpr int NCODE = 1 << BITS;
  constexpr uint32_t MASK = NCODE - 1;
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_lut = reinterpret_cast<float*>(smem);
  const int lut_floats = AFFINE ? 0 : ((a.num_codebooks * NCODE + 3) & ~3);
  int* s_ptr = reinterpret_cast<int*>(s_lut + lut_floats);                       // [RB + 1] (+3 pad)
  int* s_cnt = s_ptr + a.rows_per_block + 4;                                     // [16] rows per degree class
  int* s_order = s_cnt + 16;                                                     // [RB] rows, heaviest first
  uint32_t* s_ids = reinterpret_cast<uint32_t*>(s_order + a.rows_per_block);     // [edge_cap]
  unsigned char* s_codes = reinterpret_cast<unsigned char*>(s_ids + a.edge_cap); // [edge_cap][pitch]

  const int t = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * a.rows_per_block;
  const int nrows = (int)((a.R - row0) < a.rows_per_block ? (a.R - row0) : a.rows_per_block);
  int64_t e0 = (int64_t)indptr[row0];
  e0 = e0 < 0 ? 0 : (e0 > a.E ? a.E : e0);
  for (int i = t; i <= nrows; i += TB) {
    int64_t v = (int64_t)indptr[row0 + i];
    v = v < e0 ? e0 : (v > a.E ? a.E : v);
    s_ptr[i] = (int)(v - e0 > 0x7fffffff ? 0x7fffffff : v - e0);
  }
  if (t < 16) s_cnt[t] = 0;
  if (!AFFINE) {
    for (int i = t; i < a.num_codebooks * NCODE; i += TB) {
      const float* cb = a.table + (int64_t)(i >> BITS) * 5;
      const uint32_t raw = (uint32_t)(i & MASK);
      float v;
      if (BITS == 1) {
        v = ((float)raw - 0.5f) * (2.f * cb[4]);
      } else {
        const float drange = (float)(1 << (BITS - 1));
        const float k = __fdiv_rn(__fsub_rn(cb[3], cb[2]), drange);
        v = sq_log_decode(BITS < 8 ? (float)raw - drange : (float)(int8_t)raw, k, cb[2]);
      }
      s_lut[i] = v;
    }
  }
  __syncthreads();
  const int ne = s_ptr[nrows];
  const bool staged = ne <= a.edge_cap;

  // Rows are visited heaviest first (counting sort on min(degree, 15)), so the lanes of a wave,
  // which each walk one row's edges, loop about equally long instead of all waiting for the
  // longest row of an arbitrary group.
  int my_class[NK], my_rank[NK];
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int r = t + k * TB;
    my_class[k] = my_rank[k] = 0;
    if (r < nrows) {
      const int d = s_ptr[r + 1] - s_ptr[r];
      my_class[k] = d < 0 ? 0 : (d > 15 ? 15 : d);
      my_rank[k] = atomicAdd(&s_cnt[my_class[k]], 1);
    }
  }
  if (staged)
    for (int i = t; i < ne; i += TB) s_ids[i] = (uint32_t)clamp_idx(indices[e0 + i], a.N);
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int r = t + k * TB;
    if (r < nrows) {
      int before = 0;
      for (int c = 15; c > my_class[k]; --c) before += s_cnt[c];
      s_order[before + my_rank[k]] = r;
    }
  }
  if (staged) {
    // gather: lane j of a group stages row bytes [8j, 8j+8) of its edge (see acc_gather)
    const int j = t & ((1 << a.lane_shift) - 1);
    const int gslot = t >> a.lane_shift;
    const int gslots = TB >> a.lane_shift;
    if (j < a.lanes) {
      const int off = 8 * j < a.eff_bytes - 8 ? 8 * j : a.eff_bytes - 8;
      const int sh = (8 * j - off) * 8;
      constexpr int U = 4;
      uint32_t keep = 0;
      for (int e = gslot; e < ne; e += gslots * U) {
        uint64_t w[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          int ee = e + u * gslots;
          ee = ee < ne ? ee : ne - 1;
          __builtin_memcpy(&w[u], a.codes + ((uint64_t)s_ids[ee] * (uint32_t)a.src_dim + (uint32_t)off), 8);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          keep ^= (uint32_t)w[u];  // keeps the loads together ahead of the conditional stores
          if (u == 0 || e + u * gslots < ne)
            *reinterpret_cast<uint64_t*>(s_codes + (e + u * gslots) * a.pitch + 8 * j) = w[u] >> sh;
        }
      }
      if (keep == 0x9e3779b9u && a.eff_bytes < 0) s_ids[0] = keep;  // never true; gives `keep` a use
    }
  }
  __syncthreads();

  // decode + sum: a lane keeps one float4 column group and walks the rows
  const int g = (int)(((uint32_t)t * a.fin_magic) >> 16);
  const int l = t - g * a.fin_group;
  if (g >= a.fin_slots) return;
  for (int c4 = l; c4 < a.f4_per_row; c4 += a.fin_group) {
    float mn[4], sc[4];
    int lb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // a last group of two columns takes the last column's parameters for the two it has not
      const int col = HALF != 0 && c4 * 4 + i >= a.feat_dim ? a.feat_dim - 1 : c4 * 4 + i;
      if (AFFINE) {
        mn[i] = a.table[col];
        sc[i] = a.table[a.param_stride + col];
        lb[i] = 0;
      } else {
        int64_t cb = ((int64_t)(col / PER) * PER) / a.column_slice;  // codebook of the packed byte
        cb = cb < a.num_codebooks ? cb : a.num_codebooks - 1;
        lb[i] = (int)cb * NCODE;
        mn[i] = sc[i] = 0.f;
      }
    }
    // position of this group's code bits inside a row
    const int boff = BITS == 8 ? 4 * c4 : (BITS == 4 ? 2 * c4 : (BITS == 2 ? c4 : (c4 >> 1)));
    const int bsh = BITS == 1 ? (c4 & 1) * 4 : 0;
    const unsigned char* sp = s_codes + boff;
    const uint8_t* gp = a.codes + boff;
    float* o = out + (row0 * (int64_t)a.feat_dim + c4 * 4);
    // Rows of 4 k + 2 columns start at multiples of 8 bytes only and end with a group of two columns: the 16-byte
    // stores go to any dword, the last group stores its two columns alone and, unstaged, reads only their bytes.
    const bool half_group = HALF != 0 && c4 * 4 + 2 == a.feat_dim;
    for (int ri = g; ri < nrows; ri += a.fin_slots) {
      const int r = s_order[ri];
      const int b = s_ptr[r], e = s_ptr[r + 1];
      float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
      // two edges per trip (the second clamped to the first and masked at a row's odd end): the
      // staged reads and the eight LUT reads of a trip are independent, which halves the chain of
      // LDS round trips per row
      for (int k = b; k < e; k += 2) {
        const bool two = k + 1 < e;
        const int k1 = two ? k + 1 : k;
        uint32_t w, x;
        if (staged) {
          if (BITS == 8) {
            w = *reinterpret_cast<const uint32_t*>(sp + k * a.pitch);
            x = *reinterpret_cast<const uint32_t*>(sp + k1 * a.pitch);
          } else if (BITS == 4) {
            w = *reinterpret_cast<const uint16_t*>(sp + k * a.pitch);
            x = *reinterpret_cast<const uint16_t*>(sp + k1 * a.pitch);
          } else {
            w = sp[k * a.pitch];
            x = sp[k1 * a.pitch];
          }
        } else {
          const uint8_t* src = gp + (uint64_t)clamp_idx(indices[e0 + k], a.N) * (uint32_t)a.src_dim;
          const uint8_t* sr1 = gp + (uint64_t)clamp_idx(indices[e0 + k1], a.N) * (uint32_t)a.src_dim;
          if (BITS >= 4 && half_group) {
            if (BITS == 8) { uint16_t h0, h1; __builtin_memcpy(&h0, src, 2); __builtin_memcpy(&h1, sr1, 2); w = h0; x = h1; }
            else { w = *src; x = *sr1; }
          }
          else if (BITS == 8) { __builtin_memcpy(&w, src, 4); __builtin_memcpy(&x, sr1, 4); }
          else if (BITS == 4) { uint16_t h0, h1; __builtin_memcpy(&h0, src, 2); __builtin_memcpy(&h1, sr1, 2); w = h0; x = h1; }
          else { w = *src; x = *sr1; }
        }
        w >>= bsh;
        x >>= bsh;
        float v[4], u[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t cw = (w >> (BITS * i)) & MASK, cx = (x >> (BITS * i)) & MASK;
          if (AFFINE) {
            v[i] = __fadd_rn(mn[i], __fmul_rn((float)cw, sc[i]));
            u[i] = __fadd_rn(mn[i], __fmul_rn((float)cx, sc[i]));
          } else {
            v[i] = s_lut[lb[i] + cw];
            u[i] = s_lut[lb[i] + cx];
          }
        }
        s0 += v[0]; s1 += v[1]; s2 += v[2]; s3 += v[3];
        if (two) { s0 += u[0]; s1 += u[1]; s2 += u[2]; s3 += u[3]; }
      }
      const int deg = e - b;
      if (deg > 1) {
        const float d = (float)deg;
        float rc = __builtin_amdgcn_rcpf(d);
        rc = __fmaf_rn(__fmaf_rn(-d, rc, 1.f), rc, rc);
        s0 = mean_of(s0, d, rc); s1 = mean_of(s1, d, rc); s2 = mean_of(s2, d, rc); s3 = mean_of(s3, d, rc);
      }
      if constexpr (HALF != 0) {
        float* dst = o + (int64_t)r * a.feat_dim;
        if (half_group) {
          if constexpr (HALF == 2) store_nt2(dst, s0, s1);
          else *reinterpret_cast<float2*>(dst) = make_float2(s0, s1);
        } else {
          if constexpr (HALF == 2) store_nt4_align8(dst, s0, s1, s2, s3);
          else store4_align8(dst, s0, s1, s2, s3);
        }
      } else {
        if (a.nt_out) store_nt4(o + (int64_t)r * a.feat_dim, s0, s1, s2, s3);
        else *reinterpret_cast<float4*>(o + (int64_t)r * a.feat_dim) = make_float4(s0, s1, s2, s3);
      }
    }
  }
}

template <int BITS, bool AFFINE>
int launch_sq_rows(RowsArgs a, const void* indptr, const void* indices, int idx_dtype, float* out, hipStream_t st,
                   const char* what) {
  // 4- and 8-bit rows: 256 threads walk the same staged rows (twice the lanes in the decode + sum
  // phase, which sets this kernel's time: 35.7 -> 31.9 us and 43.9 -> 34.8 us on the 2.5e5-row
  // power-law block; 512 threads: 36.6 and 41.6); 1- and 2-bit rows are faster with 128 (27.7 against
  // 30.8 us), 64 lose everywhere
  constexpr int TB = BITS >= 4 ? 256 : 128;
  a.eff_bytes = (int)ceil_div(a.feat_dim, 8 / BITS);
  a.pitch = (a.eff_bytes + 7) & ~7;
  a.lanes = a.pitch / 8;
  const int lanes2 = pow2_ceil(a.lanes);
  a.lane_shift = 0;
  while ((1 << a.lane_shift) < lanes2) ++a.lane_shift;
  a.f4_per_row = (a.feat_dim + 3) / 4;
  a.fin_group = a.f4_per_row < TB ? a.f4_per_row : TB;
  a.fin_slots = TB / a.fin_group;
  a.fin_magic = (uint32_t)((65536 + a.fin_group - 1) / a.fin_group);
  a.nt_out = stream_output(a.R * (int64_t)a.feat_dim * 4, (int64_t)a.feat_dim * 4,
                           a.R > 0 ? (double)a.E / (double)a.R : 0.0) ? 1 : 0;
  const size_t lut_bytes = AFFINE ? 0 : (size_t)(((a.num_codebooks << BITS) + 3) & ~3) * 4;
  const double avg_deg = a.R > 0 ? (double)a.E / (double)a.R : 1.0;
  const double dg = avg_deg > 0.5 ? avg_deg : 0.5;
  int cap = (int)((20 * 1024) / (a.pitch + 4));
  cap = cap > 2 * TB ? 2 * TB : cap;
  {
    // Eight rows of the average length have to fit the staging, or every block reads its code rows unstaged
    // (3e6 edges, 128 columns: 4-bit rows 75 us at 30 edges per row and 139 us at 40; 2-bit rows 60 and 132 us).
    // The staging grows to hold them, up to 28 KB: 40 edges per row then take 100 and 87 us.  More than that
    // leaves too few workgroups per CU (8-bit rows at 30 edges per row: 211 us staged in 36 KB against 140 us
    // unstaged), and such launches keep the 20 KB and read unstaged.
    const int want = (int)(8.0 * dg * 1.1) + 8;
    int most = (int)((28 * 1024) / (a.pitch + 4));
    most = most > 1024 ? 1024 : most;
    if (want > cap && want <= most) cap = want;
  }
  a.edge_cap = (cap < 8 ? 8 : cap) & ~1;  // even: keeps the staging 8-byte aligned
  int rb = ((int)(0.6 * a.edge_cap / dg) + 4) / 8 * 8;
  rb = rb < 8 ? 8 : (rb > 64 ? 64 : rb);
  rb = shrink_rows_per_block(rb, a.R, 16, 8, 1024);
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_ROWS_RB")) {
    const int want = atoi(v);
    if (want >= 8 && want <= 64) rb = want / 8 * 8;
  }
#endif
  a.rows_per_block = rb;
  // Sparse graphs reach the 64-row limit with most of the staging empty (2.5e5-row power-law block:
  // 143 of 340 edge slots used, seven blocks per CU).  The staging is then cut to 1 / 0.6 of the
  // edges the block's rows are expected to have, which is what the row count above was derived from
  // when it was not clipped: ten blocks per CU, 31.0 -> 29.2 us on that graph.  (A block with more
  // edges than slots reads its code rows unstaged, as before.)
  {
    int need = ((int)(rb * dg / 0.6) + 15) & ~15;
    need = need < 64 ? 64 : need;
    if (need < a.edge_cap) a.edge_cap = need;
  }
  const size_t lds = lut_bytes + (size_t)(rb + 4) * 4 + 64 + (size_t)rb * 4 + (size_t)a.edge_cap * 4 +
                     (size_t)a.edge_cap * a.pitch + 16;
  const int64_t grid = ceil_div(a.R, rb);
  if (grid > 0x7fffffffll) return fail(F2CGT_E_UNSUPPORTED, "%s: too many row blocks", what);
  if (plan_only()) {
    plan_record("sq_rows_kernel", grid, TB, (int64_t)lds, a.rows_per_block, a.fin_slots, TB >> a.lane_shift,
                a.edge_cap);
    return 0;
  }
  const int half = (a.feat_dim % 4 == 0 && BITS < 4) ? 0 : (a.nt_out ? 2 : 1);
#define F2CGT_ROWS_GO(I, H)                                                      \
  sq_rows_kernel<BITS, AFFINE, I, TB, H><<<(unsigned)grid, TB, lds, st>>>(       \
      a, static_cast<const I*>(indptr), static_cast<const I*>(indices), out)
#define F2CGT_ROWS_IDX(I)                                                        \
  do {                                                                           \
    if constexpr (BITS < 4) {                                                    \
      if (half == 0) F2CGT_ROWS_GO(I, 0);                                        \
    }                                                                            \
    if (half == 1) F2CGT_ROWS_GO(I, 1);                                          \
    else if (half == 2) F2CGT_ROWS_GO(I, 2);                                     \
  } while (0)
  if (idx_dtype == F2CGT_DT_I32) F2CGT_ROWS_IDX(int32_t);
  else F2CGT_ROWS_IDX(int64_t);
#undef F2CGT_ROWS_IDX
#undef F2CGT_ROWS_GO
  return launch_status(what);
}


// ---- two-table hybrid (8-bit affine SQ rows + VQ rows), row-block form ----------------------
// Same structure as sq_affine_acc_kernel<8>: SQ edges are gathered edge-parallel (32-bit lanes
// over the 4-byte chunks of the code row) into 16-bit integer field accumulators in LDS.  The
// (rare, by construction of the two-level scheme) VQ edges are added per output in edge order by
// the lane that owns the output, reading the code byte and the codebook entry through L2, so the
// 128 KB codebook does not pin the kernel to one workgroup per CU.
//   out = (n_sq * min + scale * sum_sq(code) + sum_vq(codebook entry)) / deg
struct HybArgs {
  const int32_t* row_map;
  const uint8_t* sq_codes;
  const float* sq_params;
  int64_t param_stride;
  const uint8_t* vq_codes;
  const float* vq_codebooks;
  int64_t R, E, N, n_sq, n_vq;
  int feat_dim, n_cb, K, w;
  int rows_per_block, edge_batch;
  int chunks, ch2;   // 4-column chunks per row; gather lanes per edge = pow2 >= chunks
  uint32_t magic;
  uint32_t w_magic;  // ceil(2^32 / w), 0 for w == 1: column / w as one multiply
#ifdef F2CGT_EXPERIMENTS
  unsigned long long* trace;   // 8 words per workgroup: time stamps of its phases (100 MHz) and where it ran
  int hot_rows;                // F2CGT_HYB_HOT: the first so many rows of the SQ table are copied to LDS by every workgroup
  int hot_off;                 // where in the workgroup's LDS
#endif
};

constexpr uint32_t kVqFlag = 0x80000000u;

// CH: the number of 4-column chunks per row when it is known at compile time (32 for 128 columns,
// the common width: the accumulator offsets of the gather then fold into the instructions), else 0.
template <typename Idx, int VEC, int TB, int CH = 0>
__global__ __launch_bounds__(TB) F2CGT_SGPR_AS_SHIPPED void hybrid_acc_kernel(HybArgs a, const Idx* __restrict__ indptr,
                                                            const Idx* __restrict__ indices,
                                                            float* __restrict__ out) {
  constexpr int LIMIT = 257;
  const int chunks = CH ? CH : a.chunks;
  const int ch2 = CH ? CH : a.ch2;   // CH is a power of two
  extern __shared__ __align__(16) unsigned char smem[];
  // integer accumulators: [RB][plane 0: bytes 0,2 | plane 1: bytes 1,3][chunk], rows 8 words apart
  // in bank space so that the lane groups of a wave (different rows) spread over all 32 banks
  const int acc_pitch = 2 * chunks + 8;
  uint32_t* s_acc = reinterpret_cast<uint32_t*>(smem);
  float* s_par = reinterpret_cast<float*>(s_acc + (size_t)a.rows_per_block * acc_pitch);  // [chunks][8]
  int* s_ptr = reinterpret_cast<int*>(s_par + (size_t)chunks * 8);         // [RB + 1]
  int* s_nvq = s_ptr + a.rows_per_block + 4;                                 // [RB] VQ edges per row
  uint32_t* s_mask = reinterpret_cast<uint32_t*>(s_nvq + a.rows_per_block);  // [RB][2] which of a row's first 64 edges are not in the accumulators
  uint32_t* s_row = s_mask + 2 * a.rows_per_block;                           // [edge_batch] table row | flag
  uint16_t* s_erow = reinterpret_cast<uint16_t*>(s_row + a.edge_batch);      // [edge_batch] local row

  const int t = threadIdx.x;
#ifdef F2CGT_EXPERIMENTS
  if (a.trace == reinterpret_cast<unsigned long long*>(1)) return;   // the launch alone: what dispatching the grid costs
#endif
  ACC_STAMP(a, 0);
  const int64_t row0 = (int64_t)blockIdx.x * a.rows_per_block;
  const int nrows = (int)((a.R - row0) < a.rows_per_block ? (a.R - row0) : a.rows_per_block);
  // The column parameters are requested ahead of the row offsets, so that the two fetches of this
  // phase share one round trip (issued behind the offsets' wait they made it two).
  constexpr int NP = CH ? (CH * 4 + TB - 1) / TB : 1;
  float par_min[NP], par_scale[NP];
  if (CH) {
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int i = t + p * TB;
      const int ic = i < CH * 4 ? i : CH * 4 - 1;
      par_min[p] = a.sq_params[ic];
      par_scale[p] = a.sq_params[a.param_stride + ic];
    }
  }
  int64_t e0 = (int64_t)indptr[row0];
  e0 = e0 < 0 ? 0 : (e0 > a.E ? a.E : e0);
  // The source ids of the block's first PRE * TB edges are requested as soon as the block's first
  // edge is known, next to the row offsets, and their row-map entries behind them, ahead of the
  // barrier: the chain offsets -> ids -> row map of a block is then two round trips instead of
  // three.  How many of these edges the block really has is known only after the barrier; a
  // position beyond the edge array reads its last entry instead (nothing is read when it is empty).
  constexpr int PRE = 2;
  int64_t pre_id[PRE];
#pragma unroll
  for (int p = 0; p < PRE; ++p) pre_id[p] = 0;
  if (a.E > 0) {   // one block around all of them: the loads go out back to back
#pragma unroll
    for (int p = 0; p < PRE; ++p) {
      int64_t at = e0 + t + p * TB;
      at = at < a.E ? at : a.E - 1;
      pre_id[p] = (int64_t)indices[at];
    }
  }
  for (int i = t; i <= nrows; i += TB) {
    int64_t v = (int64_t)indptr[row0 + i];
    v = v < e0 ? e0 : (v > a.E ? a.E : v);
    s_ptr[i] = (int)(v - e0 > 0x7fffffff ? 0x7fffffff : v - e0);
  }
  int32_t pre_map[PRE];
#pragma unroll
  for (int p = 0; p < PRE; ++p) pre_map[p] = 0;
  if (a.E > 0) {   // edges imply source rows
#pragma unroll
    for (int p = 0; p < PRE; ++p) pre_map[p] = a.row_map[clamp_idx(pre_id[p], a.N)];
  }
#ifdef F2CGT_EXPERIMENTS
  // Measured variant: the hottest source rows (the first hot_rows rows of the SQ table, where the synthetic
  // workloads keep them) are copied into the workgroup's LDS, and edges that name them are gathered from there.
  if (VEC == 4 && a.hot_rows > 0) {
    typedef uint32_t u32x4h __attribute__((ext_vector_type(4)));
    const int pieces = a.hot_rows * (CH ? CH : a.feat_dim >> 2) / 4;   // 16-byte pieces, at most 8 per lane
    const u32x4h* src = reinterpret_cast<const u32x4h*>(a.sq_codes);
    u32x4h hv[8];
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int i = t + p * TB;
      hv[p] = src[i < pieces ? i : pieces - 1];
    }
    u32x4h* dst = reinterpret_cast<u32x4h*>(smem + a.hot_off);
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int i = t + p * TB;
      if (i < pieces) dst[i] = hv[p];
    }
  }
#endif
  {   // all rows of the block's accumulator area, 16 bytes per lane (rows_per_block is a multiple of 8)
    uint4* z = reinterpret_cast<uint4*>(s_acc);
    const int n4 = (a.rows_per_block * acc_pitch) >> 2;
    for (int i = t; i < n4; i += TB) z[i] = make_uint4(0u, 0u, 0u, 0u);
  }
  for (int i = t; i < nrows; i += TB) {
    s_nvq[i] = 0;
    s_mask[2 * i] = 0u;
    s_mask[2 * i + 1] = 0u;
  }
  if (CH) {
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int i = t + p * TB;
      if (i < CH * 4) {
        const int c4 = i >> 2, q = i & 3;
        s_par[c4 * 8 + q] = par_min[p];
        s_par[c4 * 8 + 4 + q] = par_scale[p];
      }
    }
  } else {
    for (int i = t; i < a.feat_dim; i += TB) {
      const int c4 = i >> 2, q = i & 3;
      s_par[c4 * 8 + q] = a.sq_params[i];
      s_par[c4 * 8 + 4 + q] = a.sq_params[a.param_stride + i];
    }
  }
  __syncthreads();
  ACC_STAMP(a, 1);
  const int ne = s_ptr[nrows];
  const uint32_t* codes32 = reinterpret_cast<const uint32_t*>(a.sq_codes);
  const int dwords_per_row = CH ? CH : a.feat_dim >> 2;   // CH chunks are CH dwords of 8-bit codes

  // Blocks of eight rows find an edge's row by comparing its position with the seven inner row starts
  // (read once, the same in every lane) instead of a search with one LDS round trip per step.
  const bool eight = a.rows_per_block == 8;
  int start_of[8];
#pragma unroll
  for (int k = 1; k < 8; ++k) start_of[k] = eight ? s_ptr[k < nrows ? k : nrows] : 0;
  // rows longer than the field capacity are summed directly in the epilogue (flag: all edges "VQ-like")
  for (int eb = 0; eb < ne; eb += a.edge_batch) {
    const int nb = (ne - eb) < a.edge_batch ? (ne - eb) : a.edge_batch;
    if (eb) __syncthreads();
    for (int i = t; i < nb; i += TB) {
      int64_t m;
      if (eb == 0 && i < PRE * TB) {
        m = (int64_t)(i < TB ? pre_map[0] : pre_map[1]);
      } else {
        const int64_t id = clamp_idx(indices[e0 + eb + i], a.N);
        m = (int64_t)a.row_map[id];
      }
      uint32_t v;
      if (m >= 0) {
        v = (uint32_t)(m < a.n_sq ? m : a.n_sq - 1);
      } else {
        const int64_t r = -m - 1;
        v = (uint32_t)(r < a.n_vq ? r : a.n_vq - 1) | kVqFlag;
      }
      // the edge's destination row: the last r with s_ptr[r] <= position (empty rows share a
      // start and are skipped that way); the same number of steps in every lane
      const int pos = eb + i;
      int lo = 0;
      if (eight) {
#pragma unroll
        for (int k = 1; k < 8; ++k) lo += start_of[k] <= pos ? 1 : 0;
      } else {
        int hi = nrows;
        while (hi - lo > 1) {
          const int mid = (lo + hi) >> 1;
          if (s_ptr[mid] <= pos) lo = mid; else hi = mid;
        }
      }
      const int first = s_ptr[lo];
      if (s_ptr[lo + 1] - first > LIMIT) v |= 0x40000000u;   // rows beyond the field capacity stay out of the accumulators
      if (v >> 30) {   // added in the epilogue, in edge order: counted, and marked among the row's first 64 edges
        atomicAdd(s_nvq + lo, 1);
        const int bit = pos - first;
        if (bit >= 0 && bit < 64) atomicOr(s_mask + 2 * lo + (bit >> 5), 1u << (bit & 31));
      }
      s_row[i] = v;
      s_erow[i] = (uint16_t)lo;
    }
    __syncthreads();
    if (eb == 0) ACC_STAMP(a, 2);
    if (VEC == 4) {
      // a lane takes 16 bytes (4 chunks) of an edge's code row: chunks / 4 lanes per edge
      const int lanes = ch2 >> 2;
      const int j = t & (lanes - 1);
      const int gslot = t / lanes;
      const int gslots = TB / lanes;
      constexpr int U = 4;
      // lane j of the lanes that share an edge loads dwords 4j .. 4j+3 with one 16-byte access (the
      // lanes of an edge cover its 128-byte line once; four strided dword loads per lane kept
      // hitting lines still in flight and stalled the L1) and adds dword 4j+c to accumulator word
      // c*q + j (q = chunks / 4), so every atomic instruction touches q consecutive words per edge
      const int per = (nb + gslots - 1) / gslots;
      const int e_begin = gslot * per;
      const int e_end = (e_begin + per) < nb ? (e_begin + per) : nb;
      const int q = chunks >> 2;   // dwords per lane stride (chunks is a multiple of 4 here)
      const bool lane_on = j < q;
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      // every lane always loads: a lane without a row to fetch (an edge that is added in the epilogue,
      // a lane beyond the row's chunks) reads the first 16 bytes of row 0, which the table has
      const uint32_t* lane_codes = codes32 + (lane_on ? 4 * j : 0);
      for (int e = e_begin; e < e_end; e += U) {
        u32x4 w[U];
        uint32_t row[U], er[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          int ee = e + u;
          ee = ee < e_end ? ee : e_end - 1;
          row[u] = s_row[ee];
          er[u] = s_erow[ee];
          uint32_t r = (row[u] >> 30) == 0 ? row[u] : 0u;
#ifdef F2CGT_EXPERIMENTS
          if (a.hot_rows > 0 && r < (uint32_t)a.hot_rows) r = 0u;   // comes from LDS below; the load reads row 0
#endif
          w[u] = *reinterpret_cast<const u32x4*>(lane_codes + (uint64_t)r * (uint32_t)dwords_per_row);
        }
        // the four loads are issued together and waited for together, whatever the adds below use
#pragma unroll
        for (int u = 0; u < U; ++u) asm volatile("" : "+v"(w[u]));
#ifdef F2CGT_EXPERIMENTS
        if (a.hot_rows > 0) {
#pragma unroll
          for (int u = 0; u < U; ++u) {
            if ((row[u] >> 30) == 0 && row[u] < (uint32_t)a.hot_rows)
              w[u] = *reinterpret_cast<const u32x4*>(smem + a.hot_off + (size_t)row[u] * (dwords_per_row * 4) +
                                                     (lane_on ? 16 * j : 0));
          }
        }
#endif
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int ee = e + u;
          if (ee < e_end && lane_on && (row[u] >> 30) == 0) {
            uint32_t* acc = s_acc + er[u] * acc_pitch + j;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              // bytes 0 and 2, then bytes 1 and 3, each widened to a 16-bit field
              atomicAdd(acc + c * q, __builtin_amdgcn_perm(0u, w[u][c], 0x0c020c00u));
              atomicAdd(acc + chunks + c * q, __builtin_amdgcn_perm(0u, w[u][c], 0x0c030c01u));
            }
          }
        }
      }
    } else {
    const int j = t & (ch2 - 1);
    const int gslot = t / ch2;
    const int gslots = TB / ch2;
    constexpr int U = 4;
    for (int e = gslot; e < nb; e += gslots * U) {
      uint32_t w[U], row[U], er[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        int ee = e + u * gslots;
        ee = ee < nb ? ee : nb - 1;
        row[u] = s_row[ee];
        er[u] = s_erow[ee];
        w[u] = 0;
        if (j < chunks && (row[u] >> 30) == 0) w[u] = codes32[(int64_t)row[u] * dwords_per_row + j];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int ee = e + u * gslots;
        if (ee < nb && j < chunks && (row[u] >> 30) == 0) {
          uint32_t* acc = s_acc + er[u] * acc_pitch + j;
          atomicAdd(acc, __builtin_amdgcn_perm(0u, w[u], 0x0c020c00u));
          atomicAdd(acc + chunks, __builtin_amdgcn_perm(0u, w[u], 0x0c030c01u));
        }
      }
    }
    }
  }
  __syncthreads();
  ACC_STAMP(a, 3);
  // finalize: lane <-> one float4 of the block's contiguous output span
  const int items = nrows * chunks;
  float* ob = out + row0 * (int64_t)a.feat_dim;
  for (int it = t; it < items; it += TB) {
    const int r = CH ? it / CH : (int)__umulhi((uint32_t)it, a.magic);
    const int c4 = it - r * chunks;
    uint2 q;
    // (the 16-byte gather stores dword c4 of a row at word (c4 % 4) * chunks / 4 + c4 / 4)
    const int pos = VEC == 4 ? (c4 & 3) * (chunks >> 2) + (c4 >> 2) : c4;
    q.x = s_acc[r * acc_pitch + pos];
    q.y = s_acc[r * acc_pitch + chunks + pos];
    const int b = s_ptr[r], e = s_ptr[r + 1];
    const int deg = e - b;
    const int nvq = s_nvq[r];
    const float nsq = (float)(deg - nvq);
    const float4 mn = *reinterpret_cast<const float4*>(s_par + c4 * 8);
    const float4 sc = *reinterpret_cast<const float4*>(s_par + c4 * 8 + 4);
    float v0 = __fadd_rn(__fmul_rn(nsq, mn.x), __fmul_rn((float)(q.x & 0xffffu), sc.x));
    float v1 = __fadd_rn(__fmul_rn(nsq, mn.y), __fmul_rn((float)(q.y & 0xffffu), sc.y));
    float v2 = __fadd_rn(__fmul_rn(nsq, mn.z), __fmul_rn((float)(q.x >> 16), sc.z));
    float v3 = __fadd_rn(__fmul_rn(nsq, mn.w), __fmul_rn((float)(q.y >> 16), sc.w));
    if (nvq > 0) {  // the row's remaining edges, in edge order, straight from the tables
      const int col = c4 * 4;
      const int sub = a.w_magic ? (int)__umulhi((uint32_t)col, a.w_magic) : col;
      const int off = col - sub * a.w;
      const bool in_lds = ne <= a.edge_batch;  // one batch: s_row still describes every edge of the block
      auto add_edge = [&](int64_t m) {
        if (m >= 0) {
          const int64_t row = m < a.n_sq ? m : a.n_sq - 1;
          const uint32_t wv = codes32[row * dwords_per_row + c4];
          v0 += __fadd_rn(mn.x, __fmul_rn((float)(wv & 0xffu), sc.x));
          v1 += __fadd_rn(mn.y, __fmul_rn((float)((wv >> 8) & 0xffu), sc.y));
          v2 += __fadd_rn(mn.z, __fmul_rn((float)((wv >> 16) & 0xffu), sc.z));
          v3 += __fadd_rn(mn.w, __fmul_rn((float)(wv >> 24), sc.w));
        } else {
          int64_t row = -m - 1;
          row = row < a.n_vq ? row : a.n_vq - 1;
          int code = a.vq_codes[row * a.n_cb + sub];
          code = code < a.K ? code : a.K - 1;
          const float4 x = *reinterpret_cast<const float4*>(a.vq_codebooks + ((int64_t)sub * a.K + code) * a.w + off);
          v0 += x.x; v1 += x.y; v2 += x.z; v3 += x.w;
        }
      };
      if (in_lds && deg <= 64) {
        // only the marked edges (one or two of a dozen, typically), lowest first
        uint64_t mask = (uint64_t)s_mask[2 * r] | ((uint64_t)s_mask[2 * r + 1] << 32);
        while (mask) {
          const uint32_t v = s_row[b + __builtin_ctzll(mask)];
          mask &= mask - 1;
          add_edge((v & kVqFlag) ? -(int64_t)(v & 0x3fffffffu) - 1 : (int64_t)(v & 0x3fffffffu));
        }
      } else {
        for (int k = b; k < e; ++k) {
          int64_t m;
          if (in_lds) {
            const uint32_t v = s_row[k];
            if ((v >> 30) == 0) continue;  // SQ edge already in the integer accumulators
            m = (v & kVqFlag) ? -(int64_t)(v & 0x3fffffffu) - 1 : (int64_t)(v & 0x3fffffffu);
          } else {
            const int64_t id = clamp_idx(indices[e0 + k], a.N);
            m = (int64_t)a.row_map[id];
            if (m >= 0 && deg <= LIMIT) continue;
          }
          add_edge(m);
        }
      }
    }
    if (deg > 1) {
      const float d = (float)deg;
      const float rdeg = __builtin_amdgcn_rcpf(d);
      v0 *= rdeg; v1 *= rdeg; v2 *= rdeg; v3 *= rdeg;
    }
    if (deg <= 0) v0 = v1 = v2 = v3 = 0.f;
    store_nt4(ob + (int64_t)it * 4, v0, v1, v2, v3);
  }
  ACC_STAMP(a, 4);
#ifdef F2CGT_EXPERIMENTS
  if (a.trace && threadIdx.x == 0) {
    a.trace[(size_t)blockIdx.x * 8 + 5] = __builtin_amdgcn_s_getreg((31 << 11) | 4);    // HW_ID
    a.trace[(size_t)blockIdx.x * 8 + 6] = __builtin_amdgcn_s_getreg((31 << 11) | 20);   // XCC_ID
  }
#endif
}

}  // namespace

// The staged-rows kernel keeps at least eight edges of `pitch + 4` bytes in its 20 KB of staging.
static bool sq_rows_pitch_ok(int feat_dim, int target_bits) {
  return (((int64_t)feat_dim * target_bits + 63) / 64) * 8 + 4 <= 2048;
}

bool sq_block_eligible(const void* codes, const float* out, int64_t N, int64_t src_dim, int feat_dim,
                       int target_bits, int64_t lut_entries) {
  if ((target_bits == 1 || target_bits == 2 || target_bits == 4 || target_bits == 8) && feat_dim % 2 == 0 &&
      (int64_t)feat_dim * target_bits >= 64 &&
      src_dim >= 8 && feat_dim <= 4096 && sq_rows_pitch_ok(feat_dim, target_bits) && aligned(out, 16) &&
      N < (1ll << 32) && src_dim < (1ll << 24) && src_dim * (8 / target_bits) >= feat_dim &&
      lut_entries * 4 <= 16 * 1024)
    return true;  // staged-rows kernel (any row pitch up to 2 KB, float4 column groups)
  int lb, nout;
  switch (target_bits) {
    case 8: lb = 4; nout = 4; break;
    case 4: lb = 2; nout = 4; break;
    case 2: lb = 1; nout = 4; break;
    case 1: lb = 1; nout = 8; break;
    default: return false;
  }
  if (feat_dim < nout || feat_dim % nout != 0) return false;
  if (feat_dim / nout > kBlock) return false;
  if (src_dim % lb != 0 || !aligned(codes, lb) || !aligned(out, 16)) return false;
  if (src_dim * (8 / target_bits) < feat_dim) return false;
  if (N >= (1ll << 32) || src_dim >= (1ll << 24)) return false;
  if (lut_entries * 4 > 16 * 1024) return false;
  return true;
}

int sq_block_run(bool affine, const uint8_t* codes, const float* table, int64_t param_stride,
                 int64_t column_slice, int num_codebooks, const void* indptr, const void* indices,
                 int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int64_t src_dim, int feat_dim,
                 int target_bits, hipStream_t st, const char* what) {
  // the 128-thread staged-rows kernel (degree-ordered rows) covers every shape with float4 column
  // groups; the 256-thread block kernel below stays for the remaining ones
  if (feat_dim % 2 == 0 && (int64_t)feat_dim * target_bits >= 64 && src_dim >= 8 && feat_dim <= 4096 &&
      sq_rows_pitch_ok(feat_dim, target_bits)) {
    RowsArgs r{};
    r.codes = codes; r.table = table; r.param_stride = param_stride; r.column_slice = column_slice;
    r.num_codebooks = num_codebooks; r.R = R; r.E = E; r.N = N; r.src_dim = (int)src_dim; r.feat_dim = feat_dim;
#define F2CGT_ROWS(B)                                                                             \
  return affine ? launch_sq_rows<B, true>(r, indptr, indices, idx_dtype, out, st, what)           \
                : launch_sq_rows<B, false>(r, indptr, indices, idx_dtype, out, st, what)
    switch (target_bits) {
      case 8: F2CGT_ROWS(8);
      case 4: F2CGT_ROWS(4);
      case 2: F2CGT_ROWS(2);
      default: F2CGT_ROWS(1);
    }
#undef F2CGT_ROWS
  }
  SqBlockArgs a{};
  a.codes = codes;
  a.table = table;
  a.param_stride = param_stride;
  a.column_slice = column_slice;
  a.num_codebooks = num_codebooks;
  a.R = R; a.E = E; a.N = N;
  a.src_dim = (int)src_dim;
  a.feat_dim = feat_dim;
#define F2CGT_GO(B, L)                                                                              \
  return affine ? launch_sq_block<B, L, true>(a, indptr, indices, idx_dtype, out, st, what)        \
                : launch_sq_block<B, L, false>(a, indptr, indices, idx_dtype, out, st, what)
  switch (target_bits) {
    case 8: F2CGT_GO(8, 4);
    case 4: F2CGT_GO(4, 2);
    case 2: F2CGT_GO(2, 1);
    default: F2CGT_GO(1, 1);
  }
#undef F2CGT_GO
}

bool sq_affine_acc_eligible(const void* codes, const float* out, int64_t N, int64_t src_dim, int feat_dim,
                            int target_bits) {
  if (target_bits != 4 && target_bits != 8) return false;
  if (codes == nullptr || !aligned(out, 16)) return false;
  if (feat_dim % 2 != 0 || feat_dim > 4096) return false;
  if (feat_dim * target_bits < 64) return false;  // a gather lane loads 8 bytes of the row
  if (src_dim < 8 || src_dim >= (1ll << 20) || src_dim * (8 / target_bits) < feat_dim) return false;
  if (N < 1 || N >= (1ll << 32)) return false;
  const int lanes = (int)ceil_div(ceil_div(feat_dim, 8 / target_bits), 8);
  if (pow2_ceil(lanes) > 128) return false;
  if ((size_t)(8 * lanes + 64) * 4 * 4 > 24 * 1024) return false;  // 8 rows of the wide layout
  return true;
}

int sq_affine_acc_run(const uint8_t* codes, const float* params, int64_t param_stride, const void* indptr,
                      const void* indices, int idx_dtype, float* out, int64_t R, int64_t E, int64_t N,
                      int64_t src_dim, int feat_dim, int target_bits, hipStream_t st, const char* what) {
  AccArgs a{};
  a.codes = codes;
  a.params = params;
  a.param_stride = param_stride;
  a.R = R; a.E = E; a.N = N;
  a.src_dim = (int)src_dim;
  a.feat_dim = feat_dim;
  return target_bits == 4 ? launch_acc<4>(a, indptr, indices, idx_dtype, out, st, what)
                          : launch_acc<8>(a, indptr, indices, idx_dtype, out, st, what);
}

template <int TB>
int launch_hybrid(HybArgs a, const void* indptr, const void* indices, int idx_dtype, float* out, hipStream_t st,
                  const char* what, int edges_per_thread = 4) {
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_HYB_BATCH")) {   // edges of a block that are tagged at a time, per thread
    const int want = atoi(v);
    if (want == 4 || want == 8 || want == 16) edges_per_thread = want;
  }
#endif
  a.edge_batch = edges_per_thread * TB;
  const double avg_deg = a.R > 0 ? (double)a.E / (double)a.R : 1.0;
  const int want = (int)(1.5625 * TB / (avg_deg > 0.5 ? avg_deg : 0.5));   // ~1.5 edges per thread
  int rb = 8;
  while (rb * 2 <= want && rb < 64) rb *= 2;
  const size_t acc_row = (size_t)(2 * a.chunks + 8) * 4;
  while (rb > 8 && rb * acc_row > 16 * 1024) rb /= 2;
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_HYB_RB")) {
    const int want = atoi(v);
    if (want == 8 || want == 16 || want == 32 || want == 64) rb = want;
  }
#endif
  a.rows_per_block = rb;
  size_t lds = rb * acc_row + (size_t)a.chunks * 32 + (size_t)(rb + 4) * 4 + (size_t)rb * 4 + (size_t)rb * 8 +
               (size_t)a.edge_batch * 6 + 16;
#ifdef F2CGT_EXPERIMENTS
  a.trace = g_acc_trace;
  a.hot_rows = 0;
  a.hot_off = 0;
  if (const char* v = getenv("F2CGT_HYB_HOT")) {   // hot rows in LDS: 16-byte gather, at most 8 pieces of 16 bytes per lane
    const int want = atoi(v);
    const bool vec4 = a.feat_dim % 16 == 0 && aligned(a.sq_codes, 16) && a.ch2 >= 4;
    if (want > 0 && vec4 && (int64_t)want <= a.n_sq && (int64_t)want * a.feat_dim <= (int64_t)8 * TB * 16) {
      a.hot_rows = want;
      a.hot_off = (int)((lds + 15) & ~(size_t)15);
      lds = (size_t)a.hot_off + (size_t)want * a.feat_dim;
    }
  }
#endif
  const int64_t grid = ceil_div(a.R, rb);
  if (grid > 0x7fffffffll) return fail(F2CGT_E_UNSUPPORTED, "%s: too many row blocks", what);
  const bool vec4 = a.feat_dim % 16 == 0 && aligned(a.sq_codes, 16) && a.ch2 >= 4;
  if (plan_only()) {
    plan_record("hybrid_acc_kernel", grid, TB, (int64_t)lds, a.rows_per_block, vec4 ? TB / (a.ch2 >> 2) : TB / a.ch2,
                vec4 ? 4 : 1, a.edge_batch);
    return 0;
  }
  const int32_t* ip32 = static_cast<const int32_t*>(indptr);
  const int32_t* ix32 = static_cast<const int32_t*>(indices);
  const int64_t* ip64 = static_cast<const int64_t*>(indptr);
  const int64_t* ix64 = static_cast<const int64_t*>(indices);
  if (idx_dtype == F2CGT_DT_I32) {
    if (vec4 && a.chunks == 32) hybrid_acc_kernel<int32_t, 4, TB, 32><<<(unsigned)grid, TB, lds, st>>>(a, ip32, ix32, out);
    else if (vec4) hybrid_acc_kernel<int32_t, 4, TB><<<(unsigned)grid, TB, lds, st>>>(a, ip32, ix32, out);
    else hybrid_acc_kernel<int32_t, 1, TB><<<(unsigned)grid, TB, lds, st>>>(a, ip32, ix32, out);
  } else {
    if (vec4 && a.chunks == 32) hybrid_acc_kernel<int64_t, 4, TB, 32><<<(unsigned)grid, TB, lds, st>>>(a, ip64, ix64, out);
    else if (vec4) hybrid_acc_kernel<int64_t, 4, TB><<<(unsigned)grid, TB, lds, st>>>(a, ip64, ix64, out);
    else hybrid_acc_kernel<int64_t, 1, TB><<<(unsigned)grid, TB, lds, st>>>(a, ip64, ix64, out);
  }
  return launch_status(what);
}

bool hybrid_acc_eligible(const void* sq_codes, const float* vq_codebooks, const float* out, int64_t N,
                         int64_t n_sq, int64_t n_vq, int feat_dim, int w) {
  if (!aligned(sq_codes, 4) || !aligned(out, 16) || !aligned(vq_codebooks, 16)) return false;
  // (feat_dim 4 is one chunk per row: its reciprocal 2^32 does not fit the 32-bit multiplier)
  if (feat_dim < 8 || feat_dim % 4 != 0 || feat_dim > 1024 || w % 4 != 0) return false;
  if (N >= (1ll << 32) || n_sq >= (1ll << 30) || n_vq >= (1ll << 30)) return false;
  return true;
}

int hybrid_acc_run(const int32_t* row_map, const uint8_t* sq_codes, const float* sq_params, int64_t param_stride,
                   const uint8_t* vq_codes, const float* vq_codebooks, const void* indptr, const void* indices,
                   int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int64_t n_sq, int64_t n_vq,
                   int feat_dim, int n_cb, int K, int w, hipStream_t st, const char* what) {
  HybArgs a{};
  a.row_map = row_map; a.sq_codes = sq_codes; a.sq_params = sq_params; a.param_stride = param_stride;
  a.vq_codes = vq_codes; a.vq_codebooks = vq_codebooks;
  a.R = R; a.E = E; a.N = N; a.n_sq = n_sq; a.n_vq = n_vq;
  a.feat_dim = feat_dim; a.n_cb = n_cb; a.K = K; a.w = w;
  a.w_magic = w > 1 ? (uint32_t)((0x100000000ull + (uint64_t)w - 1) / (uint64_t)w) : 0u;
  a.chunks = feat_dim / 4;
  a.ch2 = pow2_ceil(a.chunks);
  a.magic = (uint32_t)((0x100000000ull + a.chunks - 1) / a.chunks);
  // One wave per workgroup (8 rows at 12 edges per row) for rows of up to 128 columns and up to 32 edges:
  // the phases of a block are dependent memory round trips, and many small blocks per CU overlap
  // them better than few large ones, without a barrier between waves (C4: 334 -> 313 us; 128
  // threads and 16 rows: 318; twice the rows per block at either size: 332-344).  Against the
  // 256-thread form on 2e7-node tables, 64 / 128 columns: 2 edges per row 145 / 228 against 148 / 243 us,
  // 5: 192 / 298 against 196 / 309, 20: 289 / 179 against 439 / 220, 32: 247 / 163 against 697 / 325;
  // above 32 edges per row eight rows no longer fit one batch of 256 edges (48: 752 / 585 against
  // 663 / 311), and at 256 columns the 256-thread form is level or ahead from 5 edges per row on.
  const double avg_deg = R > 0 ? (double)E / (double)R : 0.0;
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_HYB_TB")) {   // workgroup size for an A/B: 64, 128 or 256
    if (atoi(v) == 64) return launch_hybrid<64>(a, indptr, indices, idx_dtype, out, st, what);
    if (atoi(v) == 128) return launch_hybrid<128>(a, indptr, indices, idx_dtype, out, st, what);
    if (atoi(v) == 256) return launch_hybrid<256>(a, indptr, indices, idx_dtype, out, st, what);
  }
#endif
  // Beyond that: the smallest workgroup whose edge batch still holds eight rows of the average length, so that
  // a block is tagged and gathered in one go (us for 1.2e7 edges, 128 columns, 256 threads x 4 edges against the
  // choice below: 40 edges per row 318 -> 175, 64: 310 -> 181, 80: 342 -> 264, 128: 359 -> 284, 200: 655 -> 357;
  // 256 columns: 40: 166 -> 149, 200: 587 -> 271; 64 columns, 2.4e7 edges: 100: 608 -> 394, 200: 971 -> 510).
  // The limits are exact fits for rows of one length, which an edge count that is a multiple of the row count
  // gives away (a sampled block with a fixed fanout); ragged rows get a quarter of slack, since a block over its
  // batch takes several rounds (rows capped at 40 with 28.2 on average: 166 us with 256-edge batches, twice the
  // time per edge of its neighbours).
  const double fit = (R > 0 && E % R == 0) ? 1.0 : 0.8;
  if (a.ch2 <= 32) {
    if (avg_deg <= 32.0 * fit) return launch_hybrid<64>(a, indptr, indices, idx_dtype, out, st, what);
    if (avg_deg <= 64.0 * fit) return launch_hybrid<128>(a, indptr, indices, idx_dtype, out, st, what);
    if (avg_deg <= 128.0 * fit) return launch_hybrid<128>(a, indptr, indices, idx_dtype, out, st, what, 8);
    if (a.ch2 <= 16) return launch_hybrid<128>(a, indptr, indices, idx_dtype, out, st, what, 16);
    return launch_hybrid<256>(a, indptr, indices, idx_dtype, out, st, what, 8);
  }
  // wider rows: 128 threads below 6 edges per row (2: 676 against 756 us, 5: 360 against 382) and from 24 to 64
  if (avg_deg <= 6.0 || (avg_deg > 24.0 && avg_deg <= 64.0 * fit))
    return launch_hybrid<128>(a, indptr, indices, idx_dtype, out, st, what);
  if (avg_deg > 128.0 * fit) return launch_hybrid<256>(a, indptr, indices, idx_dtype, out, st, what, 8);
  return launch_hybrid<256>(a, indptr, indices, idx_dtype, out, st, what);
}

}  // namespace f2cgt

#ifdef F2CGT_EXPERIMENTS
// Experiments build only: device buffer of 8 x 64-bit words per workgroup that sq_affine_acc_kernel
// fills with the time stamps of its phases; nullptr switches it off.
extern "C" void f2cgt_experiment_set_acc_trace(unsigned long long* device_buffer) { f2cgt::g_acc_trace = device_buffer; }
#endif
