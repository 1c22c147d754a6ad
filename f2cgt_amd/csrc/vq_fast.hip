// Persistent, software-pipelined kernel for the fused VQ decode + mean aggregation.
//
// One 1024-thread workgroup per CU keeps a 128-column tile of the codebook in LDS, laid out
// [code][128 columns], so the 16 B a lane reads per edge sit at bank offset 4 * (lane % 32):
// the 32 lanes of a row read 512 contiguous bytes of one code's row only when codes agree, and
// otherwise spread over all banks.  A lane owns one float4 of a destination row (32 lanes per
// row) and two rows of a 64-row block, walks the row's edges in order with register
// accumulators, and issues the codebook reads of the next group of edges before the adds of
// the current group.
//
// Everything that comes from HBM is prefetched through registers two iterations ahead, one
// element per lane and stage, and parked in LDS one barrier before it is needed:
//     P  indptr of block b        issued at iteration b-6, in LDS (ring of 8) after b-5
//     I  source id of edge t      issued at b-4 (needs P), stays in the lane's register
//     C  code bytes of edge t     issued at b-2 (needs I), in LDS after b-1
//     compute block b             iteration b
// so the dependent chain indptr -> indices -> codes -> output never stalls a wave.
// Workgroups are bound to a (column tile, row stripe); wide features (D = 768) use six tiles.
#include "spmm_fast.hpp"

#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace f2cgt {
namespace {

constexpr int kThreads = 1024;
constexpr int kRows = 64;        // destination rows per block (kThreads / 16 pieces)
constexpr int kEdgeCap = 1024;   // staged edges per block: one per lane
constexpr int kRing = 8;
constexpr int kGroup = 5;        // edges per register group of the inner loop
constexpr int kXcds = 8;         // accelerator dies (one L2 each) of the MI355X

struct VqArgs {
  const uint8_t* codes;
  const float* codebooks;
  int64_t R, E, N;
  int n_cb, K, w, feat_dim;
  int n_tiles, n_stripes;
  int stripes_per_xcd;  // > 0: the column tiles of a stripe share one XCD (see the kernel)
  int dense_store;      // sparse rows: results go through LDS so that every store instruction is dense
  int own_lg;           // 2: the launch takes the form whose lanes own their columns in groups of four (pair_pos)
  int store_late;       // experiments build only: 9 = the time-stamped form of the wave kernel
  unsigned long long* trace;   // experiments build only: per wave {start, first step, end} in 100 MHz ticks
};

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int BT> struct code_word;
template <> struct code_word<4> { using type = uint32_t; };
template <> struct code_word<8> { using type = u32x2; };
template <> struct code_word<16> { using type = u32x4; };

__device__ __forceinline__ float dpp_swap_pair(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
}

// Correctly rounded a / d from r = RN-refined 1/d (two FMAs after the product).
__device__ __forceinline__ float div_by(float a, float d, float r) {
  const float q = a * r;
  return __fmaf_rn(__fmaf_rn(-q, d, a), r, q);
}

// 1 / n for a row of n >= 2 edges, refined by one Newton step: within an ulp of the exact
// reciprocal, so `sum * mean_scale(n)` is the mean to 2 ulp (relative 2.4e-7), where a correctly
// rounded division costs three more vector instructions per output.
__device__ __forceinline__ float mean_scale(int n) {
  const float d = (float)n;
  const float r = __builtin_amdgcn_rcpf(d);
  return __fmaf_rn(__fmaf_rn(-d, r, 1.f), r, r);
}

template <int BT, typename Idx>
struct VqPipe {
  using CW = typename code_word<BT>::type;
  // register state, two generations per stage
  int64_t Pa, Pb, P0a, P0b;
  int64_t Ia, Ib;
  CW Ca, Cb;
  template <int G> __device__ __forceinline__ int64_t& Pr() { if constexpr (G == 0) return Pa; else return Pb; }
  template <int G> __device__ __forceinline__ int64_t& P0r() { if constexpr (G == 0) return P0a; else return P0b; }
  template <int G> __device__ __forceinline__ int64_t& Ir() { if constexpr (G == 0) return Ia; else return Ib; }
  template <int G> __device__ __forceinline__ CW& Cr() { if constexpr (G == 0) return Ca; else return Cb; }

  const VqArgs& a;
  const Idx* __restrict__ indptr;
  const Idx* __restrict__ indices;
  float* __restrict__ out;
  float* s_cb;
  unsigned char* s_codes;
  int* s_ptr;       // [kRing][kRows + 2]: relative edge offsets, [kRows + 1] = edge count
  int64_t* s_e0;    // [kRing]
  int tile, stripe, t;
  int64_t my_blocks;

  __device__ VqPipe(const VqArgs& a_, const Idx* ip, const Idx* ix, float* o) : a(a_), indptr(ip), indices(ix), out(o) {}

  __device__ __forceinline__ int64_t global_block(int64_t b) const { return stripe + b * a.n_stripes; }
  __device__ __forceinline__ bool valid(int64_t b) const { return b >= 0 && b < my_blocks; }
  __device__ __forceinline__ int rows_of(int64_t b) const {
    const int64_t row0 = global_block(b) * kRows;
    return (int)((a.R - row0) < kRows ? (a.R - row0) : kRows);
  }

  // Block-uniform values read back from LDS are moved to scalar registers so that the stage
  // bookkeeping runs on the scalar unit and only the per-lane load/store remains vector work.
  __device__ __forceinline__ int uniform_ne(int64_t b) const {
    return __builtin_amdgcn_readfirstlane(s_ptr[(int)(b & (kRing - 1)) * (kRows + 2) + kRows + 1]);
  }
  __device__ __forceinline__ int64_t uniform_e0(int64_t b) const {
    const int64_t v = s_e0[b & (kRing - 1)];
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
  }

  template <int PAR>
  __device__ __forceinline__ void iteration(int64_t it) {
    // ---- issue the three prefetch stages ---------------------------------------------------
    // Every wave issues exactly three loads per iteration (lanes without work read a harmless
    // valid address), and nothing here consumes a loaded value at once, so the memory counter
    // waits the compiler inserts are "all but the last few", never a full drain.
    {  // C: code bytes of edge t of block it+2; the id was fetched at it-2 and is clamped only now
      const int ne = valid(it + 2) ? uniform_ne(it + 2) : 0;
      const bool on = ne <= kEdgeCap && t < ne;
      const uint64_t raw = (uint64_t)Ir<PAR>();
      const uint64_t id = raw < (uint64_t)a.N ? raw : (uint64_t)(a.N - 1);
      const uint8_t* src = a.codes + (on ? id * (uint32_t)a.n_cb : 0) + tile * BT;
      Cr<PAR>() = *reinterpret_cast<const CW*>(src);
    }
    {  // I: source id of edge t of block it+4 (raw; ids outside [0, N) read row N-1)
      const bool v = valid(it + 4);
      const int ne = v ? uniform_ne(it + 4) : 0;
      const bool on = ne <= kEdgeCap && t < ne;
      const int64_t e0 = v ? uniform_e0(it + 4) : 0;
      const Idx* src = on ? indices + e0 + t : indptr;
      Ir<PAR>() = (int64_t)*src;
    }
    {  // P: row offsets of block it+6
      const bool v = valid(it + 6);
      const int64_t row0 = v ? global_block(it + 6) * kRows : 0;
      const int nr = v ? rows_of(it + 6) : 0;
      P0r<PAR>() = (int64_t)indptr[row0];
      Pr<PAR>() = (int64_t)indptr[row0 + (t <= nr ? t : 0)];
    }
    // ---- compute block `it` ------------------------------------------------------------------
    if (valid(it)) compute(it);
    __syncthreads();
    // ---- park what was issued one iteration ago ------------------------------------------------
    if (valid(it + 1)) {  // C issued at it-1 lives in the other generation
      const int ne = uniform_ne(it + 1);
      if (ne <= kEdgeCap && t < ne) *reinterpret_cast<CW*>(s_codes + t * BT) = Cr<PAR ^ 1>();
    }
    if (valid(it + 5)) {  // P issued at it-1
      const int slot = (int)((it + 5) & (kRing - 1));
      const int nr = rows_of(it + 5);
      int64_t e0 = P0r<PAR ^ 1>();
      e0 = e0 < 0 ? 0 : (e0 > a.E ? a.E : e0);
      if (t <= nr) {
        int64_t v = Pr<PAR ^ 1>();
        v = v < e0 ? e0 : (v > a.E ? a.E : v);
        const int64_t rel = v - e0;
        const int r32 = rel > 0x3fffffff ? 0x3fffffff : (int)rel;
        s_ptr[slot * (kRows + 2) + t] = r32;
        if (t == nr) s_ptr[slot * (kRows + 2) + kRows + 1] = r32;
      }
      if (t == 0) s_e0[slot] = e0;
    }
    __syncthreads();
  }

  // A lane owns one float4 of a destination row (32 lanes per row: the conflict-free LDS
  // pattern) and takes two rows of the block, 32 apart.
  __device__ __forceinline__ void compute(int64_t b) {
    const int c4 = t & 31;
    const int rs = t >> 5;
    const int slot = (int)(b & (kRing - 1));
    const int* sp = s_ptr + slot * (kRows + 2);
    const int nr = rows_of(b);
    const int tile_cols = (a.feat_dim - tile * 128) >= 128 ? 128 : (a.feat_dim - tile * 128);
    if (c4 * 4 >= tile_cols) return;
    const int ne = __builtin_amdgcn_readfirstlane(sp[kRows + 1]);
    const int byte_idx = (c4 * 4) / a.w;
    const float* cbp = s_cb + c4 * 4;
    const bool staged = ne <= kEdgeCap;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int row = rs + pass * 32;
      if (row >= nr) continue;
      int eb = sp[row], ee = sp[row + 1];
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      int n;
      if (staged) {
        eb = eb > ne ? ne : eb;
        ee = ee > ne ? ne : ee;
        n = ee - eb;
        const unsigned char* cp = s_codes + eb * BT + byte_idx;
        int k = 0;
        for (; k + kGroup <= n; k += kGroup) {
          uint32_t code[kGroup];
          float4 x[kGroup];
#pragma unroll
          for (int u = 0; u < kGroup; ++u) code[u] = cp[u * BT];
          cp += kGroup * BT;
#pragma unroll
          for (int u = 0; u < kGroup; ++u) x[u] = *reinterpret_cast<const float4*>(cbp + code[u] * 128);
#pragma unroll
          for (int u = 0; u < kGroup; ++u) { a0 += x[u].x; a1 += x[u].y; a2 += x[u].z; a3 += x[u].w; }
        }
        for (; k < n; ++k) {
          const uint32_t code = *cp;
          cp += BT;
          const float4 x = *reinterpret_cast<const float4*>(cbp + code * 128);
          a0 += x.x; a1 += x.y; a2 += x.z; a3 += x.w;
        }
      } else {
        // block with more edges than the staging holds: walk the row straight from HBM
        n = ee - eb;
        const int64_t e0 = s_e0[slot];
        for (int k = 0; k < n; ++k) {
          const int64_t id = clamp_idx(indices[e0 + eb + k], a.N);
          const uint32_t code = a.codes[id * a.n_cb + tile * BT + byte_idx];
          const float4 x = *reinterpret_cast<const float4*>(cbp + code * 128);
          a0 += x.x; a1 += x.y; a2 += x.z; a3 += x.w;
        }
      }
      if (n > 1) {
        const float r = mean_scale(n);
        a0 *= r; a1 *= r; a2 *= r; a3 *= r;
      }
      store_nt4(out + (global_block(b) * kRows + row) * (int64_t)a.feat_dim + tile * 128 + c4 * 4, a0, a1, a2, a3);
    }
  }
};

template <int BT, typename Idx>
__global__ __launch_bounds__(kThreads) void vq_pipe_kernel(VqArgs a, const Idx* __restrict__ indptr,
                                                           const Idx* __restrict__ indices,
                                                           float* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char smem[];
  VqPipe<BT, Idx> pipe(a, indptr, indices, out);
  pipe.s_cb = reinterpret_cast<float*>(smem);
  pipe.s_codes = smem + (size_t)a.K * 128 * 4;
  pipe.s_e0 = reinterpret_cast<int64_t*>(pipe.s_codes + kEdgeCap * BT);
  pipe.s_ptr = reinterpret_cast<int*>(pipe.s_e0 + kRing);
  pipe.t = threadIdx.x;
  if (a.stripes_per_xcd > 0) {
    // Workgroup ids are dealt round-robin to the XCDs.  The column tiles of a stripe read the same
    // indptr, indices and code rows, so they are placed on one XCD and share its L2: the rows come
    // from HBM once per stripe instead of once per tile.
    const int xcd = blockIdx.x % kXcds, k = blockIdx.x / kXcds;
    if (k >= a.stripes_per_xcd * a.n_tiles) return;
    pipe.tile = k % a.n_tiles;
    pipe.stripe = xcd * a.stripes_per_xcd + k / a.n_tiles;
  } else {
    pipe.tile = blockIdx.x % a.n_tiles;
    pipe.stripe = blockIdx.x / a.n_tiles;
  }
  const int64_t nblocks = ceil_div(a.R, kRows);
  pipe.my_blocks = pipe.stripe < nblocks ? (nblocks - pipe.stripe + a.n_stripes - 1) / a.n_stripes : 0;
  pipe.Pa = pipe.Pb = pipe.P0a = pipe.P0b = 0;
  pipe.Ia = pipe.Ib = 0;

  // codebook tile -> LDS as [code][piece][8]
  const int tile_cols = (a.feat_dim - pipe.tile * 128) >= 128 ? 128 : (a.feat_dim - pipe.tile * 128);
  stage_codebook_tile<kThreads, false>(pipe.s_cb, a.codebooks, a.K, a.w, pipe.tile, tile_cols);
  for (int i = threadIdx.x; i < kRing * (kRows + 2); i += kThreads) pipe.s_ptr[i] = 0;
  __syncthreads();

  for (int64_t it = -6; it < pipe.my_blocks; it += 2) {
    pipe.template iteration<0>(it);
    pipe.template iteration<1>(it + 1);
  }
}

// ---- wave-granular variant ------------------------------------------------------------------
// Same codebook tile, lane mapping and inner loop, but every wave of the workgroup runs its own
// pipeline, with wave-private staging in LDS.  After the codebook is staged no workgroup barrier
// is left: a wave that waits for its loads does not hold the other fifteen, and the LDS
// operations of one wave execute in order, so its own stage hand-overs need no synchronisation.
// A wave takes chunks of 12 consecutive destination rows from its workgroup's range (dealt through
// a counter in LDS) and walks them as mini-blocks of RPM rows (<= 64 edges: one edge per lane in the
// I and C stages; larger ones are summed straight from HBM).  RPM follows the average degree: 4 up
// to 15 edges per row, and 2 or 1 above, where the lane groups left over in a pass share a row's
// edges and add their partial sums:
//     P  the 13 row offsets of a chunk     one load per chunk, issued while the previous chunk
//                                          starts, parked half a chunk later (two LDS buffers)
//     I  source id of edge `lane`          issued two mini-blocks ahead, stays in the register
//     C  code bytes of edge `lane`         issued one mini-block ahead, parked in LDS when due
// Everything that is the same for all lanes (mini-block bounds, row numbers, base addresses) is
// kept in scalar registers; the vector instructions outside the inner loop are what bounded the
// block-synchronous version of this kernel.
constexpr int kWRows = 4;
constexpr int kWEdges = 64;
constexpr int kWMini = 3;                     // 4-row mini-blocks per chunk
constexpr int kWChunk = kWRows * kWMini;      // rows per chunk
constexpr int kWPtr = 56;                     // ints per offset buffer: [0..12] offsets, [52..53] first edge, [55] of the first buffer: next chunk

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

// TAIL: code rows whose length is no multiple of BT (13 codebooks of 8 columns for 100 features: one tile of 13 code
// bytes).  The BT bytes a lane fetches for its tile then start at any byte of the table, reach into the next row
// (bytes the tile has no columns for) and, for the table's last row or two, past its end: those rows are fetched
// byte by byte.
// EVEN2 (H == 1): feat_dim is even but no multiple of 4 (602 columns).  Output rows then start at multiples of 8
// bytes only and the last column group of the last tile has two columns.  A lane still stores its four values with
// one 16-byte store (global memory takes it at any dword); the lane of the two-column group fetches the previous
// group's last two sums from that group's lane and stores the 16 bytes that end with its own two, so that every lane
// issues the same single store (1191 us with one column per lane, 507 us with two 8-byte stores per lane; 602
// columns, 3e6 edges, 10 per row).  A tile of two columns in all (130 = 128 + 2) stores those alone.  The codebooks
// hold the columns up to the next multiple of 4, since n_cb * w >= feat_dim is a multiple of 8, so the sums are
// formed as for a full group.
// QUAD (H == 2): the two 16-byte halves of a lane's result are exchanged inside lane quads before they are stored,
// so that a store instruction writes whole 64-byte pieces (see the store at the end of a step).
// OWN (H == 2): the binary logarithm of the number of lanes that own the columns of a code together (pair_pos).
template <int BT, int H, int RPM, typename Idx, bool DENSE = false, bool TRACE = false, bool TAIL = false,
          bool EVEN2 = false, bool QUAD = false, int OWN = 0>
__global__ __launch_bounds__(kThreads) void vq_wave_kernel(VqArgs a, const Idx* __restrict__ indptr,
                                                           const Idx* __restrict__ indices,
                                                           float* __restrict__ out) {
  using CW = typename code_word<BT>::type;
  constexpr int kWaves = kThreads / 64;
  constexpr int kMini = kWChunk / RPM;          // mini-blocks (RPM rows each) per chunk
  // TRACE (experiments build): time stamps per wave
  unsigned long long t_start = 0;
  if constexpr (TRACE) t_start = wall_clock64();
  const bool K_FITS_ONE_PASS = a.K * 32 <= 8 * kThreads;
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_cb = reinterpret_cast<float*>(smem);
  const int wave = uni((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  constexpr int kStage = kWEdges * BT > 1024 ? kWEdges * BT : 1024;     // code bytes of a mini-block, or 64 float4
  unsigned char* s_codes = smem + (size_t)a.K * 128 * 4 + (size_t)wave * kStage;
  int* s_ptr = reinterpret_cast<int*>(smem + (size_t)a.K * 128 * 4 + (size_t)kWaves * kStage) + wave * 2 * kWPtr;

  int tile, stripe;
  if (a.stripes_per_xcd > 0) {
    const int xcd = blockIdx.x % kXcds, k = blockIdx.x / kXcds;
    if (k >= a.stripes_per_xcd * a.n_tiles) return;
    tile = k % a.n_tiles;
    stripe = xcd * a.stripes_per_xcd + k / a.n_tiles;
  } else {
    tile = blockIdx.x % a.n_tiles;
    stripe = blockIdx.x / a.n_tiles;
  }
  const int tile_cols_out = (a.feat_dim - tile * 128) >= 128 ? 128 : (a.feat_dim - tile * 128);
  const int tile_cols = EVEN2 ? (tile_cols_out + 3) & ~3 : tile_cols_out;   // columns staged and summed

  // A workgroup owns one contiguous range of rows, cut into chunks of 12 rows.  The waves deal the
  // chunks among themselves through a counter in LDS: wave w starts with chunk w and takes the next
  // free one whenever it starts a chunk (the one after the chunk it is working on, so that its row
  // offsets and source ids are loaded a chunk ahead).  With equal fixed shares the oldest wave of
  // each SIMD, which the hardware serves first, finished 25 % earlier than the youngest and the CU
  // ran its last quarter with ever fewer waves (16 x 8 codebooks: waves 0-3 done at 69 us, 12-15 at
  // 92 us); uneven degrees add to that.  Twelve rows (three 4-row mini-blocks) is the smallest chunk
  // whose offsets can still be requested a chunk ahead with two offset buffers; the tail of a
  // workgroup is one chunk long (16 rows: 79.3 us, 12 rows: 77.8 us at that shape).
  // A launch too small to give every wave a 12-row chunk is cut into one piece per wave instead
  // (nothing is left to deal then, and no wave walks four mini-blocks while others idle).
  const int64_t wg_share = (a.R + a.n_stripes - 1) / a.n_stripes;
  const bool dealt = wg_share >= (int64_t)kWaves * kWChunk;
  const int64_t piece = dealt ? (int64_t)kWChunk : ((wg_share + kWaves - 1) / kWaves + RPM - 1) / RPM * RPM;
  const int64_t rows_per_wg = dealt ? (wg_share + kWChunk - 1) / kWChunk * kWChunk : piece * kWaves;
  const int64_t wg_row0 = (int64_t)stripe * rows_per_wg;
  const int64_t wg_end = wg_row0 + rows_per_wg < a.R ? wg_row0 + rows_per_wg : a.R;
  const int64_t wg_chunks = !dealt ? 0 : (wg_end > wg_row0 ? (wg_end - wg_row0 + kWChunk - 1) / kWChunk : 0);
  // rows of this wave end here: the workgroup's range when chunks are dealt, else the wave's own piece
  const int64_t my_row0 = wg_row0 + (int64_t)wave * piece;
  const int64_t row_end = dealt ? wg_end : (my_row0 + piece < wg_end ? my_row0 + piece : wg_end);
  const bool has_rows = my_row0 < row_end;
  int* s_next = reinterpret_cast<int*>(smem + (size_t)a.K * 128 * 4 + (size_t)kWaves * kStage) + 55;
  auto minis_of = [&](int64_t base) {   // mini-blocks of the chunk that starts at row `base`
    const int64_t left = row_end - base;
    return (int64_t)(((left < kWChunk ? left : (int64_t)kWChunk) + RPM - 1) / RPM);
  };
  int64_t base_cur = my_row0;                              // first row of the chunk being worked on
  int64_t base_next = 0;
  bool have_next = false;
  int par = 0;                                             // offset buffer of the current chunk
  int64_t n_mini = has_rows ? minis_of(base_cur) : 0;      // mini-blocks of the chunks taken so far

  // lanes per row: 32 lanes with one float4 each (H == 1) or 16 lanes with a whole 8-column code
  // each (H == 2); the wave then works on 2 or 4 rows at a time
  constexpr int kLanesPerRow = 32 / H, kRowsPerPass = 64 / kLanesPerRow;
  // A lane beyond the columns of a partial tile takes the tile's last column group again (it
  // computes and stores what that group's own lane does), so that no lane ever skips a store: the
  // number of memory operations of a step is then the same on every path, and the waits in front
  // of the next step's loads can leave this step's stores in flight (see the main loop).
  const int groups = tile_cols / (4 * H);      // column groups of this tile (tile_cols % (4 H) == 0)
  const int c4 = (lane & (kLanesPerRow - 1)) < groups ? (lane & (kLanesPerRow - 1)) : groups - 1;
  const int half = lane / kLanesPerRow;
  // first column of the lane inside the tile; with H == 2 its second float4 lies 4 << own_lg columns on (pair_pos)
  constexpr int own_lg = H == 2 ? OWN : 0;
  const int col0 = H == 2 ? ((c4 >> own_lg) << (3 + own_lg)) + 4 * (c4 & ((1 << own_lg) - 1)) : c4 * 4;
  const int byte_idx = col0 / a.w;
  const float* cbp = s_cb + c4 * 4;
  const int prev_group_lane = (lane & ~(kLanesPerRow - 1)) + (c4 > 0 ? c4 - 1 : 0);   // EVEN2
  const uint8_t* code_base = a.codes + tile * BT;
  const uint32_t n_last = (uint32_t)(a.N - 1);
  // the last source row whose BT bytes for this tile lie inside the table (TAIL only)
  const int64_t tail_room = (int64_t)a.N * a.n_cb - (int64_t)tile * BT - BT;
  const int64_t safe_last = tail_room >= 0 ? tail_room / a.n_cb : -1;
  auto load_codes = [&](uint32_t id) -> CW {
    const uint8_t* src = code_base + (uint64_t)id * (uint32_t)a.n_cb;
    CW c;
    if constexpr (!TAIL) {
      c = *reinterpret_cast<const CW*>(src);
    } else {
      if ((int64_t)id <= safe_last) {
        __builtin_memcpy(&c, src, sizeof(CW));   // any alignment
      } else {
        uint32_t word[BT / 4];
#pragma unroll
        for (int d = 0; d < BT / 4; ++d) word[d] = 0u;
        const int have = a.n_cb - tile * BT;     // code bytes of this tile in a row (< BT here)
#pragma unroll
        for (int b = 0; b < BT; ++b)
          if (b < have) word[b >> 2] |= (uint32_t)src[b] << (8 * (b & 3));
        __builtin_memcpy(&c, word, sizeof(CW));
      }
    }
    return c;
  };

  // loads the row offsets of the chunk that starts at row0, and parks them in offset buffer `which`
  int64_t Preg = 0;
  auto issue_P = [&](int64_t row0) {
    const int64_t left = row_end - row0;
    const int nr = (int)(left < kWChunk ? left : kWChunk);
    Preg = (int64_t)indptr[row0 + (lane < nr ? lane : nr)];
  };
  // With 4-row mini-blocks the four mini-block boundaries of a chunk and its first edge are also
  // kept in scalar registers, one set per offset buffer (read out of the lanes when the offsets
  // are parked), so that the bounds of a mini-block cost no LDS read and no vector instruction in
  // any step; with more mini-blocks per chunk they are read back from LDS.
  constexpr bool SCALAR_BOUNDS = RPM == 4;
  int sb0[4] = {0, 0, 0, 0}, sb1[4] = {0, 0, 0, 0};
  int64_t se0[2] = {0, 0};
  auto park_P = [&](int which) {
    int* buf = s_ptr + which * kWPtr;
    const uint32_t lo = (uint32_t)uni((int)(uint32_t)Preg);
    const uint32_t hi = (uint32_t)uni((int)(uint32_t)((uint64_t)Preg >> 32));
    int64_t e0 = (int64_t)(((uint64_t)hi << 32) | lo);
    e0 = e0 < 0 ? 0 : (e0 > a.E ? a.E : e0);
    int64_t v = Preg;
    v = v < e0 ? e0 : (v > a.E ? a.E : v);
    const int64_t rel = v - e0;
    const int rel32 = rel > 0x3fffffff ? 0x3fffffff : (int)rel;
    if (lane <= kWChunk) buf[lane] = rel32;
    if constexpr (SCALAR_BOUNDS) {
      const int b0 = __builtin_amdgcn_readlane(rel32, 0), b1 = __builtin_amdgcn_readlane(rel32, 4);
      const int b2 = __builtin_amdgcn_readlane(rel32, 8), b3 = __builtin_amdgcn_readlane(rel32, 12);
      if (which) { sb1[0] = b0; sb1[1] = b1; sb1[2] = b2; sb1[3] = b3; se0[1] = e0; }
      else { sb0[0] = b0; sb0[1] = b1; sb0[2] = b2; sb0[3] = b3; se0[0] = e0; }
    } else {
      if (lane == 1) { buf[52] = (int)(uint32_t)e0; buf[53] = (int)(uint32_t)((uint64_t)e0 >> 32); }
    }
  };
  // bounds of mini-block m of the chunk in buffer `which`: first edge (relative to the chunk's e0)
  // and edge count
  auto bounds = [&](int which, int m, int& eb, int& ne) {
    int ee;
    if constexpr (SCALAR_BOUNDS) {
      const int c0 = which ? sb1[0] : sb0[0], c1 = which ? sb1[1] : sb0[1];
      const int c2 = which ? sb1[2] : sb0[2], c3 = which ? sb1[3] : sb0[3];
      eb = m == 0 ? c0 : (m == 1 ? c1 : c2);
      ee = m == 0 ? c1 : (m == 1 ? c2 : c3);
    } else {
      const int* buf = s_ptr + which * kWPtr;
      eb = uni(buf[m * RPM]);
      ee = uni(buf[m * RPM + RPM]);
    }
    ne = ee - eb;
    ne = ne < 0 ? 0 : ne;
  };
  auto chunk_e0 = [&](int which) {
    if constexpr (SCALAR_BOUNDS) {
      return which ? se0[1] : se0[0];
    } else {
      const int* buf = s_ptr + which * kWPtr;
      const uint32_t lo = (uint32_t)uni(buf[52]), hi = (uint32_t)uni(buf[53]);
      return (int64_t)(((uint64_t)hi << 32) | lo);
    }
  };

  // Start-up.  A launch over few rows is mostly this: 128 KB of codebook per CU and three dependent
  // round trips (row offsets -> source ids -> code bytes) before the first sum.  The wave's first
  // row offsets and the source ids of its first mini-block are requested and waited for on their
  // own; the eight codebook loads of a thread go out behind them and are still in flight while the
  // code bytes of the first and the source ids of the second mini-block are requested, so the tile
  // and the chain arrive together instead of one after the other.
  int eb0 = 0, ne0 = 0;      // mini-block g
  int eb1 = 0, ne1 = 0;      // g + 1
  int64_t Ireg = 0;
  CW Creg = {};
  int64_t g_first = -2;
  if (K_FITS_ONE_PASS && stage_codebook_vec_ok(a.codebooks, a.w, tile_cols)) {
    if (threadIdx.x == 0) *s_next = kWaves;   // chunks 0 .. 15 are the waves' first ones
    int64_t e0 = 0;
    if (has_rows) {
      issue_P(base_cur);
      park_P(0);
      bounds(0, 0, eb0, ne0);
      e0 = chunk_e0(0);
    }
    bool on = has_rows && ne0 <= kWEdges && lane < ne0;
    {
      const Idx* src = on ? indices + e0 + eb0 + lane : indptr;
      Ireg = (int64_t)*src;                                // I(0)
    }
    float4 cbv[8];
    stage_codebook_load<kThreads>(cbv, a.codebooks, a.K, a.w, tile, tile_cols);
    {
      const uint64_t raw = (uint64_t)Ireg;
      const uint32_t id = (raw >> 32) ? n_last : ((uint32_t)raw < n_last ? (uint32_t)raw : n_last);
      Creg = load_codes(on ? id : 0u);   // C(0)
    }
    {
      const bool v = has_rows && 1 < n_mini;
      if (v) bounds(0, 1, eb1, ne1);
      on = v && ne1 <= kWEdges && lane < ne1;
      const Idx* src = on ? indices + e0 + eb1 + lane : indptr;
      Ireg = (int64_t)*src;                                // I(1)
    }
    stage_codebook_store<kThreads, H == 2>(s_cb, cbv, a.K, own_lg);
    __syncthreads();
    if (!has_rows) return;
    g_first = 0;
  } else {
    stage_codebook_tile<kThreads, H == 2>(s_cb, a.codebooks, a.K, a.w, tile, tile_cols, own_lg);
    if (threadIdx.x == 0) *s_next = kWaves;
    __syncthreads();
    if (!has_rows) return;
    issue_P(base_cur);
    park_P(0);
  }
  // The two 16-byte stores of a lane and step are issued where the results are ready, at the end of
  // the step, back to back from one base register.  In the direct (not LDS-staged) form they are
  // the two halves of the lane's 32 bytes, and they have to reach the L1 together: issued a few
  // instructions apart (separate predicated blocks) the halves are written to memory separately
  // and the kernel falls into a regime twice as slow (24 x 32 codebooks: 497 -> 870-960 us, L2 ->
  // memory write-credit stalls up from 2e4 to 3.7e7 cycles per launch).
  //
  // Loads and stores complete in order on one counter.  A step issues its loads (code bytes of the
  // next mini-block, source ids of the one after) in front of its sums and its stores behind them,
  // and the next step waits for those loads only: it may leave the younger stores in flight if the
  // compiler can count them, i.e. if every path through a step issues the same number of stores.
  // Hence no store below sits under a condition: a lane group without a row of its own (the last
  // mini-block of a range) takes the mini-block's last row again and stores the same values to the
  // same place, as do the lane groups that shared a row's edges.  With conditional stores every
  // step began by waiting for the stores of the one before, a full trip to memory per step and wave.
  unsigned long long t_first = 0;
  if constexpr (TRACE) t_first = wall_clock64();
  int eb2 = 0, ne2 = 0;
  // the load stages of step g at position m of its chunk: park C(g), issue C(g+1), issue I(g+2)
  // Every lane always loads: a lane beyond the mini-block's edges reads its last edge again (and
  // with no mini-block to load for, the first row offset, which is a valid id once clamped), so the
  // id a lane holds is always one whose code row may be read, and neither load needs a per-lane
  // choice of address: the ids come from a uniform base plus a 32-bit lane offset, the code bytes of
  // every lane are parked whether the mini-block uses them or not.
  auto front = [&](int64_t g, int m) {
    if (g >= 0) *reinterpret_cast<CW*>(s_codes + lane * BT) = Creg;
    {  // C(g+1): the id fetched one step ago is clamped only now (ids outside [0, N) read row N - 1)
      const uint64_t raw = (uint64_t)Ireg;
      const uint32_t id = (raw >> 32) ? n_last : ((uint32_t)raw < n_last ? (uint32_t)raw : n_last);
      Creg = load_codes(id);
    }
    eb2 = 0; ne2 = 0;
    {  // I(g+2)
      const bool v = g + 2 < n_mini;
      int64_t e0 = 0;
      if (v) {
        const bool over = m + 2 >= kMini;   // in the next chunk
        const int which = over ? par ^ 1 : par;
        bounds(which, over ? m + 2 - kMini : m + 2, eb2, ne2);
        e0 = chunk_e0(which);
      }
      const bool ok = v && ne2 <= kWEdges && ne2 > 0;
      const char* base = reinterpret_cast<const char*>(ok ? indices + e0 + eb2 : indptr);
      const uint32_t last = ok ? (uint32_t)(ne2 - 1) : 0u;
      const uint32_t li = (uint32_t)lane < last ? (uint32_t)lane : last;
      Ireg = (int64_t)*reinterpret_cast<const Idx*>(base + li * (uint32_t)sizeof(Idx));
    }
  };
  // start-up without the early loads (large or unaligned codebooks): two steps that only load
  for (int64_t g = g_first; g < 0; ++g) {
    front(g, (int)g);
    eb0 = eb1; ne0 = ne1;
    eb1 = eb2; ne1 = ne2;
  }
  int m = 0;   // position of g inside its chunk
  // One step.  The first step runs ahead of the loop on its own copy of the code, so that the loop
  // is entered with the same memory operations in flight as after any of its own iterations (two
  // loads, then two stores): the compiler's counts for the waits are the minimum over every way
  // into the loop, and the start-up, which has no stores yet, would otherwise set them to "all".
  auto step = [&](int64_t g) __attribute__((always_inline)) {
    // chunk-level P stage, driven by the position of g inside its chunk
    if (m == 0) {
      // take the next free chunk of the workgroup and request its row offsets
      int id = 0;
      if (lane == 0) id = atomicAdd(s_next, 1);
      id = uni(id);
      have_next = id < wg_chunks;
      if (have_next) {
        base_next = wg_row0 + (int64_t)id * kWChunk;
        n_mini += minis_of(base_next);
        issue_P(base_next);
      }
    } else if (m == kMini / 2 && have_next) {   // `else`: never in the step that issued the load
      park_P(par ^ 1);
    }
    front(g, m);
    // compute mini-block g
    {
      const int* buf = s_ptr + par * kWPtr + m * RPM;
      const int64_t row0 = base_cur + m * RPM;
      const int64_t left = row_end - row0;
      const int nr = (int)(left < RPM ? left : RPM);          // >= 1: the mini-block exists
      const bool staged = ne0 <= kWEdges;
      // RPM < 4 (H == 2 only): the 4 / RPM lane groups ("slots") of a pass share a row, slot s of
      // them takes the row's edges s, s + SPR, ... and the partial sums are added across the slots
      constexpr int SPR = kRowsPerPass / (RPM < kRowsPerPass ? RPM : kRowsPerPass);
      constexpr int kPasses = RPM * SPR / kRowsPerPass;
      // sum of the codebook entries of this slot's share of row `row` (all of it when SPR == 1),
      // in edge order; returns the row's edge count
      auto row_sum = [&](int row, int sub, float (&acc)[H][4]) -> int {
        int rb = buf[row] - eb0, re = buf[row + 1] - eb0;
        int n;
        if (staged) {
          rb = min(max(rb, 0), ne0);
          re = min(max(re, 0), ne0);
          n = re - rb;
          const int ns = n > sub ? (n - sub + SPR - 1) / SPR : 0;   // edges of this slot
          const unsigned char* cp = s_codes + (rb + sub) * BT + byte_idx;
          int k = 0;
          if (ns >= kGroup) {
            // the first group starts the sums (0 + x is x: the same values as adding to zero)
            uint32_t code[kGroup];
            float4 x[kGroup][H];
#pragma unroll
            for (int u = 0; u < kGroup; ++u) code[u] = cp[u * SPR * BT];
            cp += kGroup * SPR * BT;
#pragma unroll
            for (int u = 0; u < kGroup; ++u)
#pragma unroll
              for (int h = 0; h < H; ++h) x[u][h] = *reinterpret_cast<const float4*>(cbp + code[u] * 128 + h * 64);
#pragma unroll
            for (int h = 0; h < H; ++h) {
              acc[h][0] = x[0][h].x; acc[h][1] = x[0][h].y; acc[h][2] = x[0][h].z; acc[h][3] = x[0][h].w;
            }
#pragma unroll
            for (int u = 1; u < kGroup; ++u)
#pragma unroll
              for (int h = 0; h < H; ++h) {
                acc[h][0] += x[u][h].x; acc[h][1] += x[u][h].y; acc[h][2] += x[u][h].z; acc[h][3] += x[u][h].w;
              }
            k = kGroup;
          } else {
#pragma unroll
            for (int h = 0; h < H; ++h) acc[h][0] = acc[h][1] = acc[h][2] = acc[h][3] = 0.f;
          }
          for (; k + kGroup <= ns; k += kGroup) {
            uint32_t code[kGroup];
            float4 x[kGroup][H];
#pragma unroll
            for (int u = 0; u < kGroup; ++u) code[u] = cp[u * SPR * BT];
            cp += kGroup * SPR * BT;
#pragma unroll
            for (int u = 0; u < kGroup; ++u)
#pragma unroll
              for (int h = 0; h < H; ++h) x[u][h] = *reinterpret_cast<const float4*>(cbp + code[u] * 128 + h * 64);
#pragma unroll
            for (int u = 0; u < kGroup; ++u)
#pragma unroll
              for (int h = 0; h < H; ++h) {
                acc[h][0] += x[u][h].x; acc[h][1] += x[u][h].y; acc[h][2] += x[u][h].z; acc[h][3] += x[u][h].w;
              }
          }
          for (; k < ns; ++k) {
            const uint32_t code = *cp;
            cp += SPR * BT;
#pragma unroll
            for (int h = 0; h < H; ++h) {
              const float4 x = *reinterpret_cast<const float4*>(cbp + code * 128 + h * 64);
              acc[h][0] += x.x; acc[h][1] += x.y; acc[h][2] += x.z; acc[h][3] += x.w;
            }
          }
        } else {
          // A mini-block with more edges than the staging holds (rows longer than the degree the launch was
          // sized for): its edges go through the same staging 64 at a time, ids and code bytes fetched by
          // all lanes at once for each slice (two round trips per 64 edges, not hidden, instead of two per
          // edge and lane group), and every slot adds the edges of its row that fall into the slice.
#pragma unroll
          for (int h = 0; h < H; ++h) acc[h][0] = acc[h][1] = acc[h][2] = acc[h][3] = 0.f;
          n = re - rb;
          const int64_t e0 = chunk_e0(par) + eb0;
          for (int base = 0; base < ne0; base += kWEdges) {
            const int cnt = (ne0 - base) < kWEdges ? (ne0 - base) : kWEdges;
            const int li = lane < cnt ? lane : cnt - 1;
            const int64_t id = clamp_idx(indices[e0 + base + li], a.N);
            const CW c = load_codes((uint32_t)id);
            __builtin_amdgcn_wave_barrier();   // the previous slice has been read
            *reinterpret_cast<CW*>(s_codes + lane * BT) = c;
            __builtin_amdgcn_wave_barrier();
            const int wb = rb > base ? rb : base;
            const int we = re < base + cnt ? re : base + cnt;
            // edge k of the row (counted from the row's first edge) belongs to slot k % SPR
            const int first = wb + (sub - (wb - rb) % SPR + SPR) % SPR;
            for (int k = first; k < we; k += SPR) {
              const uint32_t code = s_codes[(k - base) * BT + byte_idx];
#pragma unroll
              for (int h = 0; h < H; ++h) {
                const float4 x = *reinterpret_cast<const float4*>(cbp + code * 128 + h * 64);
                acc[h][0] += x.x; acc[h][1] += x.y; acc[h][2] += x.z; acc[h][3] += x.w;
              }
            }
          }
        }
        return n;
      };
      auto mean = [&](int n, float (&acc)[H][4]) {
        if (n > 1) {
          const float r = mean_scale(n);
#pragma unroll
          for (int h = 0; h < H; ++h)
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[h][t] *= r;
        }
      };
      if constexpr (DENSE) {
        static_assert(H == 2 && SPR == 1 && kPasses == 1, "the LDS-turned stores are for 4-row steps of 16-lane rows");
        // Four rows, sixteen lanes each.  A lane's result is 32 consecutive bytes, which as two
        // stores would be 16 of every 32 bytes per instruction (half-written sectors on the way to
        // memory).  The wave's 1 KB staging area, free once the edge loops are done, turns them
        // around: the lanes of columns [64 p, 64 p + 64) write their two float4, every lane reads
        // back the float4 of its own lane index, and each store instruction covers 256 contiguous
        // bytes of every row.  (Lanes beyond a partial tile's columns hold a copy of its last
        // column group and skip the write to the staging area; their stores repeat the last float4.)
        const int lane_c = lane & (kLanesPerRow - 1);
        const int row = half < nr ? half : nr - 1;
        float acc[H][4];
        const int n = row_sum(row, 0, acc);
        mean(n, acc);
        float4* stg = reinterpret_cast<float4*>(s_codes);
        char* obase = reinterpret_cast<char*>(out + row0 * (int64_t)a.feat_dim + tile * 128);   // uniform
        const uint32_t orow_b = (uint32_t)row * ((uint32_t)a.feat_dim * 4u);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          __builtin_amdgcn_wave_barrier();
          if ((lane_c >> 3) == p && lane_c < groups) {
#pragma unroll
            for (int h = 0; h < H; ++h)
              stg[half * 16 + (lane_c & 7) * 2 + h] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
          }
          __builtin_amdgcn_wave_barrier();
          // a lane beyond the tile's columns stores the tile's last float4 again; when that lies in
          // the other half (tile_cols <= 64 p) nobody wrote to the staging area in this pass and it
          // still holds that half
          int col = 64 * p + 4 * lane_c;
          const int last = tile_cols - 4;                  // first column of the tile's last float4
          col = col < last ? col : last;
          const float4 v = stg[half * 16 + ((col & 63) >> 2)];
          store_nt4(reinterpret_cast<float*>(obase + (orow_b + 4u * (uint32_t)col)), v.x, v.y, v.z, v.w);
        }
      } else {
        // uniform base + 32-bit byte offset of the lane: no 64-bit address arithmetic per lane
        char* obase = reinterpret_cast<char*>(out + row0 * (int64_t)a.feat_dim + tile * 128);
#pragma unroll
        for (int pass = 0; pass < kPasses; ++pass) {
          const int slot = pass * kRowsPerPass + half;
          int row = slot / SPR;
          const int sub = slot % SPR;
          row = row < nr ? row : nr - 1;
          float acc[H][4];
          const int n = row_sum(row, sub, acc);
          if (SPR > 1) {
#pragma unroll
            for (int h = 0; h < H; ++h)
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                acc[h][t] += __shfl_xor(acc[h][t], kLanesPerRow);
                if (SPR > 2) acc[h][t] += __shfl_xor(acc[h][t], 2 * kLanesPerRow);
              }
          }
          mean(n, acc);
#ifdef F2CGT_EXPERIMENTS
          if (a.dense_store == 2 && acc[0][0] != 12345.678f) continue;   // no stores: what the rest of the kernel costs
#endif
          // the lane's two 16-byte stores: one address, the second 16 bytes on as an immediate offset,
          // so that they are issued back to back (see above)
          const uint32_t off_b = (uint32_t)row * ((uint32_t)a.feat_dim * 4u) + 4u * (uint32_t)col0;
          float* dst = reinterpret_cast<float*>(obase + off_b);
          if constexpr (EVEN2) {
            if (tile_cols_out < 4) {          // a tile of two columns: nothing to pair them with
              store_nt2(dst, acc[0][0], acc[0][1]);
            } else if (tile_cols_out & 2) {   // the tile ends with a group of two columns
              const bool half_group = col0 + 2 >= tile_cols_out;
              const float p2 = __shfl(acc[0][2], prev_group_lane), p3 = __shfl(acc[0][3], prev_group_lane);
              store_nt4_align8(half_group ? dst - 2 : dst, half_group ? p2 : acc[0][0], half_group ? p3 : acc[0][1],
                               half_group ? acc[0][0] : acc[0][2], half_group ? acc[0][1] : acc[0][3]);
            } else {
              store_nt4_align8(dst, acc[0][0], acc[0][1], acc[0][2], acc[0][3]);
            }
          } else if constexpr (QUAD) {
            // A lane's eight columns are 32 contiguous bytes; stored as they are, each of the two store
            // instructions writes 16 of every 32 bytes.  Here the four lanes of a quad exchange their halves
            // (lane permutes inside the quad, no LDS), so that one instruction writes the first 64 contiguous
            // bytes of the quad's 128 and the other the last 64: lane k stores half (k & 1) of lane (k >> 1),
            // then of lane 2 + (k >> 1).
            const int lr = lane & (kLanesPerRow - 1), k = lr & 3;
            const bool odd = (k & 1) != 0;
            float va[4], vb[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int lo_a = __builtin_amdgcn_update_dpp(0, __float_as_int(acc[0][t]), 0x50, 0xf, 0xf, false);
              const int hi_a = __builtin_amdgcn_update_dpp(0, __float_as_int(acc[1][t]), 0x50, 0xf, 0xf, false);
              const int lo_b = __builtin_amdgcn_update_dpp(0, __float_as_int(acc[0][t]), 0xfa, 0xf, 0xf, false);
              const int hi_b = __builtin_amdgcn_update_dpp(0, __float_as_int(acc[1][t]), 0xfa, 0xf, 0xf, false);
              va[t] = __int_as_float(odd ? hi_a : lo_a);
              vb[t] = __int_as_float(odd ? hi_b : lo_b);
            }
            // Columns of this lane's two pieces inside the tile.  A first piece beyond the tile's columns belongs to
            // a lane beyond them as well, which holds a copy of the last column group: it stores that group's second
            // half, the tile's last 16 bytes.  A second piece beyond the columns repeats the lane's first store.
            const int col_a = (lr >> 2) * 32 + 4 * k, col_b = col_a + 16;
            const int last = tile_cols - 4;
            const bool in_a = col_a <= last, in_b = col_b <= last;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              va[t] = in_a ? va[t] : acc[1][t];
              vb[t] = in_b ? vb[t] : va[t];
            }
            const int pa = in_a ? col_a : last, pb = in_b ? col_b : pa;
            const uint32_t row_b = (uint32_t)row * ((uint32_t)a.feat_dim * 4u);
            store_nt4(reinterpret_cast<float*>(obase + (row_b + 4u * (uint32_t)pa)), va[0], va[1], va[2], va[3]);
            store_nt4(reinterpret_cast<float*>(obase + (row_b + 4u * (uint32_t)pb)), vb[0], vb[1], vb[2], vb[3]);
          } else {
            // H == 2: the second float4 lies 16 bytes on, or 64 with columns owned in groups of four lanes (pair_pos).
            // The distance is a literal so that it folds into the second store: with it in a register the two are no
            // longer issued back to back, the halves of a 32-byte piece reach the L2 apart and leave it as partial
            // writes (24 x 32 from a 5.8 GB table: 433 -> 958 us).
#pragma unroll
            for (int h = 0; h < H; ++h)
              store_nt4(dst + ((4 * h) << own_lg), acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
          }
        }
      }
    }
    eb0 = eb1; ne0 = ne1;
    eb1 = eb2; ne1 = ne2;
    if (++m == kMini) {   // on to the next chunk (the loop ends here when there is none)
      m = 0;
      par ^= 1;
      base_cur = base_next;
      have_next = false;
    }
  };
  if (n_mini > 0) {
    step(0);
    for (int64_t g = 1; g < n_mini; ++g) step(g);
  }
  if constexpr (TRACE) {
    if (lane == 0) {
      unsigned long long* t = a.trace + ((size_t)blockIdx.x * kWaves + wave) * 4;
      t[0] = t_start; t[1] = t_first; t[2] = wall_clock64(); t[3] = (unsigned long long)n_mini;
    }
  }
}

#ifdef F2CGT_EXPERIMENTS
// ---- strip variant: a lane owns 32 columns of a row --------------------------------------------
// The vector ALUs bound this operator before HBM or LDS do: the 128 adds of an edge and column tile
// are two wave instructions, and everything else a wave executes per edge comes on top of them.
// Here a quad of lanes owns a destination row of the 128-column tile and a wave works on 16 rows at
// a time: a lane reads its own code bytes straight from HBM (one load per edge; nothing is staged
// in LDS), turns them into LDS addresses once per code, and issues eight 16-byte reads per edge.
// The LDS serves 16 consecutive lanes together from 64 four-byte banks, so those lanes (four rows)
// must hit 16 different 16-byte groups of a 256-byte window whatever their codes are: lane l reads
// chunk j ^ x(l) of its 128 bytes in step j (x = 2 * (row & 3) + (quarter >> 1); the quarter's low
// bit picks the half of the window), i.e. the address of step 0 xor (j << 4).  The accumulators are
// therefore held in step order.  For the stores they go, four rows at a time, through 2 KB of
// wave-private staging laid out like the output tile and come back one float4 per lane in address
// order: every store instruction writes two whole 512-byte row pieces.
// Per wave the stages of consecutive 16-row groups are software pipelined through registers:
//     P  indptr[row], indptr[row + 1]                    issued three groups ahead
//     I  the row's first KE source ids, four per lane     two groups ahead
//     C  the lane's code bytes of those KE edges          one group ahead (ids handed round the quad)
//     X  codebook reads + adds in edge order, mean
//     S  staging round trips + stores of the group before, spread over the first eight edges of X
//        (two waves per SIMD cannot hide an LDS round trip that nothing else is issued behind)
// Rows with more than KE edges finish their tail straight from HBM (same order, unpipelined).
constexpr int kSRows = 16;     // rows per group (64 lanes / 4)

template <int W> struct strip_code;
template <> struct strip_code<8> { using type = uint32_t; };
template <> struct strip_code<16> { using type = uint16_t; };
template <> struct strip_code<32> { using type = uint8_t; };

template <int S>
__device__ __forceinline__ uint32_t quad_bcast(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, S * 0x55, 0xf, 0xf, true);
}

template <int W, int KE, bool IL, int kSThreads, int kStgRows, typename Idx>
__global__ __launch_bounds__(kSThreads) void vq_strip_kernel(VqArgs a, const Idx* __restrict__ indptr,
                                                             const Idx* __restrict__ indices,
                                                             float* __restrict__ out) {
  // IL (32-wide codes only): the lanes of a quad interleave instead of owning a quarter each: lane t
  // holds the chunks 4 i + t of the row's 32, so a quad's store i is 64 contiguous bytes and nothing
  // has to be turned round; a lane then needs all four codes of the tile (one dword), and the rows
  // of a 16-lane group stay conflict free by walking i in the order i ^ (row & 3).
  static_assert(!IL || W == 32, "interleaved quads need one code per 32 columns");
  using CT = typename strip_code<IL ? 8 : W>::type;
  typedef float f4v __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) f4v lds_float4;
  constexpr int kWaves = kSThreads / 64;
  constexpr int BT = 128 / W;           // code bytes per row and tile
  constexpr int NCODE = IL ? 4 : BT / 4;   // codes a lane reads per edge
  constexpr int CPC = 8 / NCODE;        // 16-byte chunks per code
  constexpr int XSH = IL ? 6 : 4;       // the steps of one code differ in this address bit (and up)
  static_assert(KE % 4 == 0 && KE >= 8 && KE <= 16, "edges per row held in registers");
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_cb = reinterpret_cast<float*>(smem);
  const int wave = uni((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;

  int tile, stripe;
  if (a.stripes_per_xcd > 0) {
    const int xcd = blockIdx.x % kXcds, k = blockIdx.x / kXcds;
    if (k >= a.stripes_per_xcd * a.n_tiles) return;
    tile = k % a.n_tiles;
    stripe = xcd * a.stripes_per_xcd + k / a.n_tiles;
  } else {
    tile = blockIdx.x % a.n_tiles;
    stripe = blockIdx.x / a.n_tiles;
  }
  const int tile_cols = (a.feat_dim - tile * 128) >= 128 ? 128 : (a.feat_dim - tile * 128);
  stage_codebook_tile<kSThreads, false>(s_cb, a.codebooks, a.K, a.w, tile, tile_cols);
  __syncthreads();

  const int64_t total_waves = (int64_t)a.n_stripes * kWaves;
  const int64_t rows_per_wave = ((a.R + total_waves - 1) / total_waves + kSRows - 1) / kSRows * kSRows;
  const int64_t row_begin = ((int64_t)stripe * kWaves + wave) * rows_per_wave;
  if (row_begin >= a.R) return;
  const int64_t row_end = row_begin + rows_per_wave < a.R ? row_begin + rows_per_wave : a.R;
  const int64_t n_groups = (row_end - row_begin + kSRows - 1) / kSRows;

  const int q = lane & 3, rr = lane >> 2, x = IL ? (rr & 3) : (((rr & 3) << 1) | (q >> 1));
  // LDS addresses (the tile starts the workgroup's LDS; staging follows it)
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
  // step 0 inside a code's 512 bytes: chunk x of the lane's quarter, or chunk 4 x + q of the row
  const uint32_t lane_base = lds0 + (IL ? (uint32_t)(x * 64 + q * 16) : (uint32_t)(q * 128 + x * 16));
  uint32_t lane_base_s[NCODE];   // ... of the first step of code s: steps j = s * CPC + r read at (this ^ (r << XSH))
#pragma unroll
  for (int s = 0; s < NCODE; ++s) lane_base_s[s] = lane_base ^ (uint32_t)((s * CPC) << XSH);
  const uint32_t stg0 = lds0 + (uint32_t)a.K * 512u + (uint32_t)(wave * kStgRows * 512);
  const uint32_t stg_wr = stg0 + (uint32_t)((rr & (kStgRows - 1)) * 512 + q * 128 + x * 16);  // chunk of step 0
  const uint32_t stg_rd = stg0 + (uint32_t)(lane * 16);
  // byte i of the permuted code word = code of the chunks (i * CPC ..) ^ x
  const uint32_t slot_x = (uint32_t)(x / CPC);   // (interleaved: steps 2 m, 2 m + 1 belong to quarter m ^ (x >> 1))
  const uint32_t sel = (0u ^ slot_x) | ((1u ^ slot_x) << 8) | ((2u ^ slot_x) << 16) | ((3u ^ slot_x) << 24);
  const uint8_t* code_base = a.codes + tile * BT + (IL ? 0 : q * NCODE);
  const uint32_t n_last = (uint32_t)(a.N - 1);
  const int64_t e_last = a.E - 1;
  // a lane's float4 of the staged rows: column (lane & 31) * 4 of staged row 2 i + (lane >> 5)
  const uint32_t out_lane = (uint32_t)((lane & 31) * 4) + (uint32_t)(lane >> 5) * (uint32_t)a.feat_dim;
  const bool col_ok = (lane & 31) * 4 < tile_cols;
  const bool nt = a.dense_store == 1 || a.dense_store == 3;

  // pipeline registers: two generations of everything that is in flight for two steps
  Idx praw0[2] = {0, 0}, praw1[2] = {0, 0};          // P -> I
  Idx iraw[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};     // I -> C
  int degq[5] = {0, 0, 0, 0, 0};                     // degq[d]: degree of this lane's row in group g + d
  CT cbuf[2][KE];                                     // C -> X (copied out at the top of the step that uses them)
#pragma unroll
  for (int k = 0; k < KE; ++k) cbuf[0][k] = cbuf[1][k] = 0;

  auto group_row = [&](int64_t g) {            // row of this lane in group g (groups past the end repeat the last)
    const int64_t gg = g < n_groups ? g : n_groups - 1;
    return row_begin + gg * kSRows + rr;
  };
  auto edge_reads = [&](uint32_t cw, f4v (&v)[8]) {
    uint32_t pw = cw;
    if (NCODE > 1) pw = __builtin_amdgcn_perm(cw, cw, sel);
    uint32_t addr[NCODE];
#pragma unroll
    for (int s = 0; s < NCODE; ++s) addr[s] = (((pw >> (8 * s)) & 0xffu) << 9) + lane_base_s[s];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      v[j] = *(const lds_float4*)(uintptr_t)(addr[j / CPC] ^ (uint32_t)((j % CPC) << XSH));
  };
  auto add_edge = [&](uint32_t cw, float (&acc)[8][4]) {
    f4v v[8];
    edge_reads(cw, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      acc[j][0] += v[j][0]; acc[j][1] += v[j][1]; acc[j][2] += v[j][2]; acc[j][3] += v[j][3];
    }
  };
  // The stores of group g in eight steps: ops 0, 2, 4, 6 put the rows [4 p, 4 p + 4) of the group
  // into the staging area (chunk j ^ x of a lane at its place in the row); ops 1, 3, 5, 7 fetch them
  // back in address order (stage_fetch) and, once the edge work issued behind that has covered the
  // round trip, store them (stage_store).
  auto stage_put = [&](int p, const float (&acc)[8][4]) {
    __builtin_amdgcn_wave_barrier();
    if ((rr / kStgRows) == p) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        *(lds_float4*)(uintptr_t)(stg_wr ^ (uint32_t)(j << 4)) = f4v{acc[j][0], acc[j][1], acc[j][2], acc[j][3]};
    }
    __builtin_amdgcn_wave_barrier();
  };
  auto stage_fetch = [&](f4v (&sv)[kStgRows / 2]) {
#pragma unroll
    for (int i = 0; i < kStgRows / 2; ++i) sv[i] = *(const lds_float4*)(uintptr_t)(stg_rd + (uint32_t)(i * 1024));
    __builtin_amdgcn_wave_barrier();
  };
  auto stage_store = [&](int p, const f4v (&sv)[kStgRows / 2], int64_t g) {
    const int64_t grow0 = row_begin + g * kSRows + p * kStgRows;    // uniform
    float* obase = out + grow0 * (int64_t)a.feat_dim + tile * 128;  // uniform
#pragma unroll
    for (int i = 0; i < kStgRows / 2; ++i) {
      const int64_t lrow = grow0 + 2 * i + (lane >> 5);
      if (lrow < row_end && col_ok) {
        float* o = obase + (int64_t)(2 * i) * a.feat_dim + out_lane;
        if (nt) store_nt4(o, sv[i][0], sv[i][1], sv[i][2], sv[i][3]);
        else *reinterpret_cast<float4*>(o) = make_float4(sv[i][0], sv[i][1], sv[i][2], sv[i][3]);
      }
    }
  };
  // interleaved quads: store i of a lane is the chunk 4 (i ^ x) + q of its row, straight from the registers
  auto direct_store = [&](int i, const float (&acc)[8][4], int64_t g) {
    const int64_t row = row_begin + g * kSRows + rr;
    const int col = ((i ^ x) << 4) + q * 4;
    if (row < row_end && col < tile_cols) {
      float* o = out + row * (int64_t)a.feat_dim + tile * 128 + col;
      if (nt) store_nt4(o, acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
      else *reinterpret_cast<float4*>(o) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
    }
  };
  auto store_op = [&](int op, const float (&acc)[8][4], int64_t g) {   // unpipelined form
    if (IL) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i == op) direct_store(i, acc, g);
      return;
    }
    if ((op & 1) == 0) {
      stage_put(op >> 1, acc);
    } else {
      f4v sv[kStgRows / 2];
      stage_fetch(sv);
      stage_store(op >> 1, sv, g);
    }
  };

  // One step = one 16-row group.  Loads are consumed two steps after they were issued and the
  // results are stored at the end of the step: the memory counter retires loads and stores in
  // issue order, so a wait for a load also waits for every older store, and a store takes several
  // microseconds to be acknowledged while the write path is busy.  With this order the youngest
  // store a wait can depend on is two steps old.
  auto step = [&](auto par, int64_t g) {
    constexpr int PAR = decltype(par)::value;
    // ---- codes of group g (issued two steps ago) leave their landing registers ----
    CT ccur[KE];
#pragma unroll
    for (int k = 0; k < KE; ++k) ccur[k] = cbuf[PAR][k];
    // ---- C(g + 2): code bytes of the edges whose ids were issued two steps ago ----
    {
      uint32_t nid[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint64_t raw = (uint64_t)(int64_t)iraw[PAR][i];
        uint32_t id = (raw >> 32) ? ((int64_t)raw < 0 ? 0u : n_last) : ((uint32_t)raw < n_last ? (uint32_t)raw : n_last);
        nid[i] = (q * 4 + i) < degq[2] ? id : 0u;     // edges past the row's end read row 0 (a cached line)
      }
#pragma unroll
      for (int k = 0; k < KE; ++k) {
        uint32_t id;
        switch (k >> 2) {
          case 0: id = quad_bcast<0>(nid[k & 3]); break;
          case 1: id = quad_bcast<1>(nid[k & 3]); break;
          case 2: id = quad_bcast<2>(nid[k & 3]); break;
          default: id = quad_bcast<3>(nid[k & 3]); break;
        }
        cbuf[PAR][k] = *reinterpret_cast<const CT*>(code_base + (uint64_t)id * (uint32_t)a.n_cb);
      }
    }
    // ---- I(g + 4): the row's first KE source ids, four per lane ----
    {
      const int64_t row = group_row(g + 4);
      int64_t b = (int64_t)praw0[PAR], e = (int64_t)praw1[PAR];
      b = b < 0 ? 0 : (b > a.E ? a.E : b);
      e = e < b ? b : (e > a.E ? a.E : e);
      const int64_t d = e - b;
      degq[4] = (g + 4 >= 0 && g + 4 < n_groups && row < row_end) ? (int)(d > 0x3fffffff ? 0x3fffffff : d) : 0;
      if (q * 4 < KE) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          int64_t at = b + q * 4 + i;
          at = at > e_last ? e_last : at;
          iraw[PAR][i] = indices[at];
        }
      }
    }
    // ---- P(g + 6) ----
    {
      int64_t row = group_row(g + 6);
      row = row < a.R ? row : a.R - 1;
      praw0[PAR] = indptr[row];
      praw1[PAR] = indptr[row + 1];
    }
    // ---- X(g) ----
    if (g >= 0) {
      float acc[8][4];
      const int64_t row = row_begin + g * kSRows + rr;
      const int deg = degq[0];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j][0] = acc[j][1] = acc[j][2] = acc[j][3] = 0.f;
#pragma unroll
      for (int k = 0; k < KE; ++k) {
        if (__ballot(k < deg) == 0) break;
        if (a.dense_store == 3 && k >= 1) break;   // experiment: stores only
        if (k == 0) {
          if (0 < deg) {   // the first edge lands in the accumulators as it is
            f4v v[8];
            edge_reads((uint32_t)ccur[0], v);
#pragma unroll
            for (int j = 0; j < 8; ++j) { acc[j][0] = v[j][0]; acc[j][1] = v[j][1]; acc[j][2] = v[j][2]; acc[j][3] = v[j][3]; }
          }
        } else if (k < deg) {
          add_edge((uint32_t)ccur[k], acc);
        }
      }
      if (__ballot(deg > KE) != 0) {
        // the tail of long rows, in edge order, straight from HBM
        int64_t b = 0;
        if (deg > KE) {
          b = (int64_t)indptr[row];
          b = b < 0 ? 0 : (b > a.E ? a.E : b);
        }
        for (int k = KE; __ballot(k < deg) != 0; ++k) {
          if (k < deg) {
            const int64_t id = clamp_idx(indices[b + k], a.N);
            const CT cw = *reinterpret_cast<const CT*>(code_base + (uint64_t)id * (uint32_t)a.n_cb);
            add_edge((uint32_t)cw, acc);
          }
        }
      }
      if (deg > 1) {
        const float d = (float)deg;
        float r = __builtin_amdgcn_rcpf(d);
        r = __fmaf_rn(__fmaf_rn(-d, r, 1.f), r, r);
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int t = 0; t < 4; ++t) acc[j][t] = div_by(acc[j][t], d, r);
      }
      if (a.dense_store != 2) {
        if (IL) {
#pragma unroll
          for (int i = 0; i < 8; ++i) direct_store(i, acc, g);
        } else {
#pragma unroll
          for (int op = 0; op < 2 * (kSRows / kStgRows); ++op) store_op(op, acc, g);
        }
      }
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) degq[d] = degq[d + 1];
  };

  for (int64_t g = -6; g < n_groups; g += 2) {
    step(std::integral_constant<int, 0>{}, g);
    if (g + 1 < n_groups) step(std::integral_constant<int, 1>{}, g + 1);
  }
}

template <int W, int KE, bool IL, int kSThreads, int kStgRows>
int launch_strip(const VqArgs& a, const void* indptr, const void* indices, int idx_dtype, float* out, hipStream_t st,
                 const char* what, unsigned grid) {
  const size_t lds = (size_t)a.K * 128 * 4 + (IL ? 0 : (size_t)(kSThreads / 64) * kStgRows * 512);
  if (plan_only()) {
    plan_record("vq_strip_kernel", grid, kSThreads, (int64_t)lds, kSRows, W, KE, IL ? 1 : 0, kStgRows);
    return 0;
  }
  const void* kern = idx_dtype == F2CGT_DT_I32 ? reinterpret_cast<const void*>(vq_strip_kernel<W, KE, IL, kSThreads, kStgRows, int32_t>)
                                               : reinterpret_cast<const void*>(vq_strip_kernel<W, KE, IL, kSThreads, kStgRows, int64_t>);
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail((int)e, "%s: cannot reserve %zu B of LDS", what, lds);
  if (idx_dtype == F2CGT_DT_I32)
    vq_strip_kernel<W, KE, IL, kSThreads, kStgRows, int32_t><<<grid, kSThreads, lds, st>>>(a, static_cast<const int32_t*>(indptr),
                                                                static_cast<const int32_t*>(indices), out);
  else
    vq_strip_kernel<W, KE, IL, kSThreads, kStgRows, int64_t><<<grid, kSThreads, lds, st>>>(a, static_cast<const int64_t*>(indptr),
                                                                static_cast<const int64_t*>(indices), out);
  return launch_status(what);
}

template <int W>
int launch_strip_w(const VqArgs& a, int ke, const void* indptr, const void* indices, int idx_dtype, float* out,
                   hipStream_t st, const char* what, unsigned grid) {
  constexpr bool IL = W == 32;
  const char* v = getenv("F2CGT_VQ_VAR");
  const int var = v ? atoi(v) : 0;
  if (IL) {
    if (ke <= 12 && var == 1) return launch_strip<W, 12, IL, 768, 4>(a, indptr, indices, idx_dtype, out, st, what, grid);
    if (ke <= 12) return launch_strip<W, 12, IL, 512, 4>(a, indptr, indices, idx_dtype, out, st, what, grid);
    return launch_strip<W, 16, IL, 512, 4>(a, indptr, indices, idx_dtype, out, st, what, grid);
  }
  if (var == 1) return launch_strip<W, 16, IL, 512, 8>(a, indptr, indices, idx_dtype, out, st, what, grid);
  return launch_strip<W, 16, IL, 512, 4>(a, indptr, indices, idx_dtype, out, st, what, grid);
}

#endif  // F2CGT_EXPERIMENTS

#ifdef F2CGT_EXPERIMENTS
unsigned long long* g_trace = nullptr;   // device buffer for the time stamps of F2CGT_VQ_DEFER=9

// the 4-row, int64 form of the wave kernel with time stamps per wave
template <int BT>
int launch_wave_trace(const VqArgs& a, const void* indptr, const void* indices, float* out, hipStream_t st,
                      const char* what, unsigned grid, size_t wlds) {
  const void* kern = reinterpret_cast<const void*>(vq_wave_kernel<BT, 2, 4, int64_t, false, true>);
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)wlds);
  if (e != hipSuccess) return fail((int)e, "%s: cannot reserve %zu B of LDS", what, wlds);
  vq_wave_kernel<BT, 2, 4, int64_t, false, true><<<grid, kThreads, wlds, st>>>(
      a, static_cast<const int64_t*>(indptr), static_cast<const int64_t*>(indices), out);
  return launch_status(what);
}
#endif

template <int BT, int H, int RPM>
int launch_wave(const VqArgs& a, const void* indptr, const void* indices, int idx_dtype, float* out, hipStream_t st,
                const char* what, unsigned grid, size_t wlds) {
  if (plan_only()) {
    plan_record("vq_wave_kernel", grid, kThreads, (int64_t)wlds, 0, H, RPM, a.dense_store,
                (H == 2 && RPM == 4 && BT == 4 && a.dense_store == 0) ? a.own_lg : 0);
    return 0;
  }
#ifdef F2CGT_EXPERIMENTS
  if (H == 2 && RPM == 4 && idx_dtype == F2CGT_DT_I64) {
    if (a.store_late == 9 && a.trace) return launch_wave_trace<BT>(a, indptr, indices, out, st, what, grid, wlds);
  }
#endif
  // the sparse-row form (results turned round in LDS before they are stored) is its own instantiation
  constexpr bool CAN_DENSE = H == 2 && RPM == 4;
  const bool tail = a.n_cb % BT != 0 || !aligned(a.codes, BT);
  const bool dense = CAN_DENSE && a.dense_store == 1;
  const void* kern;
  if constexpr (H == 1 && RPM == 4) {
    if (a.feat_dim % 4 != 0) {   // even widths that are no multiple of 4
      kern = tail ? (idx_dtype == F2CGT_DT_I32
                         ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false, false, true, true>)
                         : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false, false, true, true>))
                  : (idx_dtype == F2CGT_DT_I32
                         ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false, false, false, true>)
                         : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false, false, false, true>));
      const hipError_t e2 = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)wlds);
      if (e2 != hipSuccess) return fail((int)e2, "%s: cannot reserve %zu B of LDS", what, wlds);
      void* params2[] = {const_cast<VqArgs*>(&a), &indptr, &indices, &out};
      const hipError_t le2 = hipLaunchKernel(kern, dim3(grid), dim3(kThreads), params2, wlds, st);
      if (le2 != hipSuccess) return fail((int)le2, "%s: launch failed: %s", what, hipGetErrorString(le2));
      return launch_status(what);
    }
  }
  constexpr bool CAN_QUAD = H == 2 && RPM == 4;
  const bool quad = CAN_QUAD && a.dense_store == 4;
  if constexpr (H == 2 && RPM == 4 && BT == 4) {   // codebooks of 32 columns
    if (a.own_lg == 2 && a.dense_store == 0) {
      kern = tail ? (idx_dtype == F2CGT_DT_I32
                         ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false, false, true, false, false, 2>)
                         : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false, false, true, false, false, 2>))
                  : (idx_dtype == F2CGT_DT_I32
                         ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false, false, false, false, false, 2>)
                         : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false, false, false, false, false, 2>));
      const hipError_t e3 = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)wlds);
      if (e3 != hipSuccess) return fail((int)e3, "%s: cannot reserve %zu B of LDS", what, wlds);
      void* params3[] = {const_cast<VqArgs*>(&a), &indptr, &indices, &out};
      const hipError_t le3 = hipLaunchKernel(kern, dim3(grid), dim3(kThreads), params3, wlds, st);
      if (le3 != hipSuccess) return fail((int)le3, "%s: launch failed: %s", what, hipGetErrorString(le3));
      return launch_status(what);
    }
  }
  if (quad && tail)
    kern = idx_dtype == F2CGT_DT_I32
               ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false, false, true, false, CAN_QUAD>)
               : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false, false, true, false, CAN_QUAD>);
  else if (quad)
    kern = idx_dtype == F2CGT_DT_I32
               ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false, false, false, false, CAN_QUAD>)
               : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false, false, false, false, CAN_QUAD>);
  else if (tail && dense)
    kern = idx_dtype == F2CGT_DT_I32
               ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, CAN_DENSE, false, true>)
               : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, CAN_DENSE, false, true>);
  else if (tail)
    kern = idx_dtype == F2CGT_DT_I32
               ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false, false, true>)
               : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false, false, true>);
  else if (idx_dtype == F2CGT_DT_I32)
    kern = dense ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, CAN_DENSE>)
                 : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int32_t, false>);
  else
    kern = dense ? reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, CAN_DENSE>)
                 : reinterpret_cast<const void*>(vq_wave_kernel<BT, H, RPM, int64_t, false>);
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)wlds);
  if (e != hipSuccess) return fail((int)e, "%s: cannot reserve %zu B of LDS", what, wlds);
  void* params[] = {const_cast<VqArgs*>(&a), &indptr, &indices, &out};
  const hipError_t le = hipLaunchKernel(kern, dim3(grid), dim3(kThreads), params, wlds, st);
  if (le != hipSuccess) return fail((int)le, "%s: launch failed: %s", what, hipGetErrorString(le));
  return launch_status(what);
}

template <int BT>
int launch_vq(VqArgs a, const void* indptr, const void* indices, int idx_dtype, float* out, hipStream_t st,
              const char* what) {
  const size_t lds = (size_t)a.K * 128 * 4 + (size_t)kEdgeCap * BT + kRing * 8 + kRing * (kRows + 2) * 4;
  const int cus = num_cus();
  a.n_tiles = (int)ceil_div(a.feat_dim, 128);
  a.n_stripes = cus / a.n_tiles;
  if (a.n_stripes < 1) a.n_stripes = 1;
  const int64_t nblocks = ceil_div(a.R, kRows);
  if (a.n_stripes > nblocks) a.n_stripes = (int)(nblocks > 0 ? nblocks : 1);
  unsigned grid = (unsigned)(a.n_stripes * a.n_tiles);
  a.stripes_per_xcd = 0;
  if (a.n_tiles > 1 && cus % kXcds == 0 && (cus / kXcds) / a.n_tiles >= 1 &&
      (int64_t)kXcds * ((cus / kXcds) / a.n_tiles) <= nblocks) {
    a.stripes_per_xcd = (cus / kXcds) / a.n_tiles;
    a.n_stripes = kXcds * a.stripes_per_xcd;
    grid = (unsigned)cus;
  }
  const double avg_deg = a.R > 0 ? (double)a.E / (double)a.R : 0.0;
  // The wave-granular kernel: 4-row mini-blocks up to 16 edges per row, and, with whole 8-column
  // groups in every tile (one lane per group, two float4 per edge), 2-row mini-blocks up to 32 and
  // 1-row ones beyond (larger mini-blocks for sparse rows were tried and were slower than 4-row ones).
  const size_t wlds = (size_t)a.K * 128 * 4 + (size_t)(kThreads / 64) * (kWEdges * BT > 1024 ? kWEdges * BT : 1024) +
                      (size_t)(kThreads / 64) * 2 * kWPtr * 4;
  // with few edges per row the output dominates and its store pattern decides (fanout 2 at the C3
  // shape: 845 -> 405 us); from about 8 edges per row the detour through LDS costs more than it saves
  a.dense_store = avg_deg <= 8.0;
  // Above that (up to 16 edges per row, four-row mini-blocks) the form is chosen by what binds the launch:
  //  * the code table beyond the caches (over 192 MB) or rows of more than four column tiles: the gather binds, the
  //    results are stored as they are (24 x 32 from a 5.8 GB table: 423 us; 446 through LDS, 454 with the exchange);
  //  * an output of 200 MB and more from a table of 64 to 192 MB, which shares the last-level cache with it: through
  //    LDS as for sparse rows, the form whose store instructions write whole lines.  Warm it is level with the exchange
  //    (7.5e6 edges at 15 per row from a 160 MB table, 16 x 8: 79.1 against 79.4 us; plain 80.7), with graphs and
  //    outputs in rotation, where the output's lines are not in the last-level cache when they are written, well
  //    ahead (108.7 against 125.8 us, plain 120; 16 x 16 at 10 edges per row 73 / 99 against 79 / 102);
  //  * from a smaller table, such an output or up to 11 edges per row (an output of 340 MB from 32 MB of codes,
  //    32 x 16 at 12 edges per row: 130 / 131 us warm / in rotation against 135 / 136 through LDS): the halves of a
  //    lane's eight columns are exchanged inside lane
  //    quads so that every store instruction writes whole 64-byte pieces (dense_store 4; 1e6 source rows, 3e6 edges
  //    at 10 per row, plain -> exchange: 16 x 16 121 -> 87 us, 32 x 16 166 -> 90, 8 x 32 126 -> 90, 64 x 8 150 -> 93,
  //    16 x 8 49 -> 42; the plain form's time at these shapes varies by a factor of two between builds and boxes,
  //    the exchange's does not).  64-column tiles (half the lanes of a row idle) measured 6-13 % slower with it.
  // F2CGT_STORE_STREAM (the caller's outputs are written once and read later) takes the LDS form throughout: with
  // buffers in rotation the 5.8 GB case runs in 588 us against 681.
  const bool rpm4 = avg_deg <= 16.0 * ((a.R > 0 && a.E % a.R == 0) ? 1.0 : 0.9);
  if (!a.dense_store && a.feat_dim % 8 == 0 && rpm4) {
    const bool cached_table = a.N * (int64_t)a.n_cb <= (192ll << 20);
    if (store_mode() == F2CGT_STORE_STREAM) {
      a.dense_store = 1;
    } else if (cached_table && a.feat_dim >= 128 && a.n_tiles <= 4) {
      const bool big_out = a.R * (int64_t)a.feat_dim * 4 >= (200ll << 20);
      if (big_out && a.N * (int64_t)a.n_cb >= (64ll << 20)) a.dense_store = 1;
      else if (big_out || avg_deg <= 11.0) a.dense_store = 4;
    }
  }
#ifdef F2CGT_EXPERIMENTS
  {
    if (const char* d = getenv("F2CGT_VQ_DEFER")) a.store_late = atoi(d);
    a.trace = g_trace;
    if (const char* d = getenv("F2CGT_VQ_DENSE")) a.dense_store = atoi(d) != 0;   // results through LDS at any degree
    const char* v = getenv("F2CGT_VQ_STRIP");
    const int mode = v ? atoi(v) : 0;     // 0 off; tens: 0 plain, 1 non-temporal, 2 no stores; units: 2 = KE by degree, 6 = KE 16
    if (mode == 20) a.dense_store = 2;
    if (mode % 10 > 0 && avg_deg <= 24.0 && a.n_cb % BT == 0 && aligned(a.codes, BT) && a.feat_dim % 4 == 0) {
      VqArgs b = a;
      b.dense_store = (mode / 10) % 10;
      if (mode >= 100) b.N = 1;   // experiment: every source id reads row 0
      const int ke = (mode % 10) == 6 ? 16 : (avg_deg <= 6.0 ? 8 : (avg_deg <= 10.0 ? 12 : 16));
      switch (a.w) {
        case 8: return launch_strip_w<8>(b, ke, indptr, indices, idx_dtype, out, st, what, grid);
        case 16: return launch_strip_w<16>(b, ke, indptr, indices, idx_dtype, out, st, what, grid);
        default: return launch_strip_w<32>(b, ke, indptr, indices, idx_dtype, out, st, what, grid);
      }
    }
  }
#endif
  // Codebooks of 32 columns: the four lanes that share a code can own its columns as a group, so that a store
  // instruction writes 64 contiguous bytes per group at no cost in instructions (pair_pos; its own instantiation,
  // OWN = 2).  Taken where the exchange inside quads is not and the code table stays cached.
  a.own_lg = 0;
  if (a.dense_store == 0 && a.w == 32 && a.feat_dim % 32 == 0 && a.feat_dim >= 128 &&
      avg_deg <= 16.0 * ((a.R > 0 && a.E % a.R == 0) ? 1.0 : 0.9) && a.N * (int64_t)a.n_cb <= (192ll << 20))
    a.own_lg = 2;
#ifdef F2CGT_EXPERIMENTS
  if (const char* v = getenv("F2CGT_VQ_STORE")) {   // the store form whatever the shape: plain | lds | quad | own | h1
    const bool rpm4 = avg_deg <= 16.0 * ((a.R > 0 && a.E % a.R == 0) ? 1.0 : 0.9);
    if (a.feat_dim % 8 == 0 && rpm4) {
      if (!strcmp(v, "h1")) {
        a.dense_store = 0; a.own_lg = 0;
        return launch_wave<BT, 1, 4>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
      }
      a.own_lg = (!strcmp(v, "own") && a.w == 32 && a.feat_dim % 32 == 0) ? 2 : 0;
      a.dense_store = !strcmp(v, "lds") ? 1 : (!strcmp(v, "quad") ? 4 : 0);
      return launch_wave<BT, 2, 4>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
    }
  }
  if (const char* v = getenv("F2CGT_VQ_RPM")) {   // rows per mini-block whatever the degree (mini-blocks above 64 edges unstaged)
    if (a.feat_dim % 8 == 0) {
      if (atoi(v) == 4) return launch_wave<BT, 2, 4>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
      if (atoi(v) == 2) return launch_wave<BT, 2, 2>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
      if (atoi(v) == 1) return launch_wave<BT, 2, 1>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
    } else if (atoi(v) == 4) {
      return launch_wave<BT, 1, 4>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
    }
  }
#endif
  if (a.feat_dim % 8 == 0) {
    // Rows per mini-block by the average degree: uniform rows of 16 / 32 / 64 edges just fit four / two / one
    // (7.5e6 edges, 16 x 8: 16 edges per row 72 us in fours against 87 in twos, 32: 105 in twos against 167 one
    // by one).  Mini-blocks with more edges than the staging holds go through it in slices (row_sum), so a
    // graph whose rows are longer than its average suggests loses little (rows capped at 20 with 14.2 on
    // average: 89 us in fours, 88 in twos; capped at 40 with 28.2: 161 in twos, 162 one by one), and rows of any
    // length stay in this kernel: one-row mini-blocks at 64 / 200 / 2000 edges per row take 249 (2.56e7 edges) /
    // 91 / 265 us where the block-synchronous kernel below, whose 1024-edge staging 64 such rows overflow,
    // takes 1525 / 502 / 1624 us.
    // An edge count that is a multiple of the row count gives rows of one length away (a sampled block with a
    // fixed fanout): those get the exact limits, ragged rows 0.9 of them (capped at 32 with 15.2 on average: 112 us
    // in fours, 91 in twos; capped at 64 with 30.1: 198 in twos, 171 one by one).
    const double fit = (a.R > 0 && a.E % a.R == 0) ? 1.0 : 0.9;
    // Sparse rows that are no whole 128-byte lines (feat_dim no multiple of 32): one float4 per lane, 32 lanes per
    // row, is ahead of the eight-column form whose results are turned round in LDS (3e6 edges at 3 / 6 per row:
    // 25 x 8 326 / 165 -> 299 / 146 us, 21 x 8 299 / 150 -> 257 / 123, 15 x 8 186 / 102 -> 152 / 76, 19 x 32 at 600
    // columns 603 / 313 -> 551 / 279; rows of whole lines the other way round: 24 x 8 172 / 101 against 191 / 100,
    // 7 x 32 180 / 96 against 192 / 103).
    if (avg_deg <= 8.0 && a.feat_dim % 32 != 0) {
      a.dense_store = 0;
      a.own_lg = 0;
      return launch_wave<BT, 1, 4>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
    }
    if (avg_deg <= 16.0 * fit) return launch_wave<BT, 2, 4>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
    if (avg_deg <= 32.0 * fit) return launch_wave<BT, 2, 2>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
    return launch_wave<BT, 2, 1>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
  } else if (avg_deg <= 15.0 || a.n_cb % BT != 0 || !aligned(a.codes, BT) || a.feat_dim % 4 != 0) {
    // (the block-synchronous kernel below reads whole aligned code words; longer rows go through the staging in slices)
    return launch_wave<BT, 1, 4>(a, indptr, indices, idx_dtype, out, st, what, grid, wlds);
  }
  if (plan_only()) {
    plan_record("vq_pipe_kernel", grid, kThreads, (int64_t)lds, kRows);
    return 0;
  }
  const void* kern = idx_dtype == F2CGT_DT_I32 ? reinterpret_cast<const void*>(vq_pipe_kernel<BT, int32_t>)
                                               : reinterpret_cast<const void*>(vq_pipe_kernel<BT, int64_t>);
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail((int)e, "%s: cannot reserve %zu B of LDS", what, lds);
  if (idx_dtype == F2CGT_DT_I32)
    vq_pipe_kernel<BT, int32_t><<<grid, kThreads, lds, st>>>(a, static_cast<const int32_t*>(indptr),
                                                            static_cast<const int32_t*>(indices), out);
  else
    vq_pipe_kernel<BT, int64_t><<<grid, kThreads, lds, st>>>(a, static_cast<const int64_t*>(indptr),
                                                            static_cast<const int64_t*>(indices), out);
  return launch_status(what);
}

}  // namespace

#ifdef F2CGT_EXPERIMENTS
void set_trace(unsigned long long* p) { g_trace = p; }
#endif

bool vq_pipe_eligible(const void* codes, const float* codebooks, const float* out, int64_t R, int64_t E,
                      int64_t N, int feat_dim, int n_cb, int K, int w) {
  if (E < 1 || N < 1 || codes == nullptr) return false;  // idle lanes read row 0 / indptr[0]
  if (K < 1 || K > 256) return false;
  if (w != 8 && w != 16 && w != 32) return false;
  if (feat_dim < 16 || feat_dim % 2 != 0 || feat_dim > n_cb * w) return false;
  if (!aligned(out, 16) || !aligned(codebooks, 4)) return false;
  if (N >= (1ll << 32)) return false;
  if (R < 4 * kRows) return false;  // tiny problems: the per-row skeleton has less start-up cost
  return true;
}

int vq_pipe_run(const uint8_t* codes, const float* codebooks, const void* indptr, const void* indices,
                int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int feat_dim, int n_cb, int K, int w,
                hipStream_t st, const char* what) {
  VqArgs a{};
  a.codes = codes;
  a.codebooks = codebooks;
  a.R = R; a.E = E; a.N = N;
  a.n_cb = n_cb; a.K = K; a.w = w; a.feat_dim = feat_dim;
  switch (128 / w) {
    case 16: return launch_vq<16>(a, indptr, indices, idx_dtype, out, st, what);
    case 8: return launch_vq<8>(a, indptr, indices, idx_dtype, out, st, what);
    default: return launch_vq<4>(a, indptr, indices, idx_dtype, out, st, what);
  }
}

}  // namespace f2cgt

#ifdef F2CGT_EXPERIMENTS
// Experiments build only: device buffer of 4 x 64-bit words per wave (workgroups x 16 waves) that
// the time-stamped form of vq_wave_kernel (F2CGT_VQ_DEFER=9) fills; nullptr switches it off.
extern "C" void f2cgt_experiment_set_trace(unsigned long long* device_buffer) { f2cgt::set_trace(device_buffer); }
#endif
