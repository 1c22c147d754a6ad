// packbits / unpackbits: streaming byte kernels, 64-bit indexing.
//
// Two shapes each:
//   * flat: unpack_dim is a multiple of 8/bits, so the whole tensor is one stream and a
//     lane converts 16 code bytes <-> 16/(8/bits) packed bytes, one dense 16-byte access on the
//     code side and one dense 2/4/8-byte access on the packed side;
//   * rows: ragged tails (unpack_dim not a multiple of 8/bits), one lane per packed byte
//     (pack) or per code byte (unpack).
#include "common.hpp"

namespace f2cgt {
namespace {

constexpr int kBlock = 256;

template <int BITS>
__global__ __launch_bounds__(kBlock) void pack_rows_kernel(const uint8_t* __restrict__ unpack,
                                                           uint8_t* __restrict__ pack,
                                                           int64_t first, int64_t n_out,
                                                           int64_t U, int64_t P) {
  constexpr int PER = 8 / BITS;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = first + (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n_out; i += stride) {
    const int64_t r = i / P;
    const int64_t c = i - r * P;
    const int64_t col0 = c * PER;
    const int64_t src = r * U + col0;
    const int n = (int)((U - col0) < PER ? (U - col0) : PER);
    uint32_t v = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k)
      if (k < n) v |= ((uint32_t)unpack[src + k] & MASK) << (BITS * k);
    pack[i] = (uint8_t)v;
  }
}

// Flat stream in units of 16 code bytes: a lane turns one 16-byte load of codes into 16 / PER
// packed bytes (one dense store per lane), four units per lane with the loads issued first.
constexpr int kUnitsPerThread = 4;
template <int BYTES> struct uint_of;
template <> struct uint_of<2> { using type = uint16_t; };
template <> struct uint_of<4> { using type = uint32_t; };
template <> struct uint_of<8> { using type = uint64_t; };
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int BITS>
__global__ __launch_bounds__(kBlock) void pack_flat_kernel(const u32x4* __restrict__ unpack,
                                                           typename uint_of<2 * BITS>::type* __restrict__ pack,
                                                           int64_t n_units) {
  constexpr int PER = 8 / BITS;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  using OT = typename uint_of<2 * BITS>::type;       // 16 / PER bytes
  const int64_t base = (int64_t)blockIdx.x * (kBlock * kUnitsPerThread) + threadIdx.x;
  u32x4 in[kUnitsPerThread];
#pragma unroll
  for (int u = 0; u < kUnitsPerThread; ++u) {
    const int64_t q = base + u * kBlock;
    in[u] = __builtin_nontemporal_load(unpack + (q < n_units ? q : 0));
  }
#pragma unroll
  for (int u = 0; u < kUnitsPerThread; ++u) {
    const int64_t q = base + u * kBlock;
    if (q >= n_units) break;
    uint64_t out = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const uint64_t code = (in[u][e / 4] >> (8 * (e % 4))) & MASK;
      out |= code << (8 * (e / PER) + BITS * (e % PER));
    }
    __builtin_nontemporal_store((OT)out, pack + q);
  }
}

template <int BITS>
__global__ __launch_bounds__(kBlock) void unpack_rows_kernel(const uint8_t* __restrict__ pack,
                                                             uint8_t* __restrict__ unpack,
                                                             int64_t first, int64_t n_out,
                                                             int64_t U, int64_t P) {
  constexpr int PER = 8 / BITS;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = first + (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n_out; i += stride) {
    const int64_t r = i / U;
    const int64_t o = i - r * U;
    const uint32_t byte = pack[r * P + o / PER];
    unpack[i] = (uint8_t)((byte >> (BITS * (int)(o % PER))) & MASK);
  }
}

template <int BITS>
__global__ __launch_bounds__(kBlock) void unpack_flat_kernel(const typename uint_of<2 * BITS>::type* __restrict__ pack,
                                                             u32x4* __restrict__ unpack, int64_t n_units) {
  constexpr int PER = 8 / BITS;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  using IT = typename uint_of<2 * BITS>::type;
  const int64_t base = (int64_t)blockIdx.x * (kBlock * kUnitsPerThread) + threadIdx.x;
  IT in[kUnitsPerThread];
#pragma unroll
  for (int u = 0; u < kUnitsPerThread; ++u) {
    const int64_t q = base + u * kBlock;
    in[u] = __builtin_nontemporal_load(pack + (q < n_units ? q : 0));
  }
#pragma unroll
  for (int u = 0; u < kUnitsPerThread; ++u) {
    const int64_t q = base + u * kBlock;
    if (q >= n_units) break;
    const uint64_t v = (uint64_t)in[u];
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t w = 0;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int e = 4 * j + t;
        w |= (uint32_t)((v >> (8 * (e / PER) + BITS * (e % PER))) & MASK) << (8 * t);
      }
      out[j] = w;
    }
    __builtin_nontemporal_store(out, unpack + q);
  }
}

int grid_for(int64_t items) {
  int64_t blocks = ceil_div(items, kBlock);
  int64_t cap = (int64_t)num_cus() * 32;
  return (int)(blocks < cap ? (blocks < 1 ? 1 : blocks) : cap);
}

template <int BITS>
int pack_launch(const uint8_t* unpack, uint8_t* pack, int64_t rows, int64_t U, hipStream_t st) {
  constexpr int PER = 8 / BITS;
  const int64_t P = ceil_div(U, PER);
  const int64_t n_out = rows * P;
  if (n_out == 0) return 0;
  int64_t done = 0;
  if (U % PER == 0 && aligned(unpack, 16) && aligned(pack, 16 / PER)) {
    const int64_t n_units = (rows * U) / 16;
    const int64_t blocks = ceil_div(n_units, kBlock * kUnitsPerThread);
    if (n_units > 0 && blocks <= 0x7fffffffll) {
      pack_flat_kernel<BITS><<<(unsigned)blocks, kBlock, 0, st>>>(
          reinterpret_cast<const u32x4*>(unpack), reinterpret_cast<typename uint_of<2 * BITS>::type*>(pack), n_units);
      done = n_units * (16 / PER);
    }
  }
  if (done < n_out)
    pack_rows_kernel<BITS><<<grid_for(n_out - done), kBlock, 0, st>>>(unpack, pack, done, n_out, U, P);
  return launch_status("packbits");
}

template <int BITS>
int unpack_launch(const uint8_t* pack, uint8_t* unpack, int64_t rows, int64_t P, int64_t U,
                  hipStream_t st) {
  constexpr int PER = 8 / BITS;
  const int64_t n_out = rows * U;
  if (n_out == 0) return 0;
  int64_t done = 0;
  if (U == P * PER && aligned(unpack, 16) && aligned(pack, 16 / PER)) {
    const int64_t n_units = (rows * U) / 16;
    const int64_t blocks = ceil_div(n_units, kBlock * kUnitsPerThread);
    if (n_units > 0 && blocks <= 0x7fffffffll) {
      unpack_flat_kernel<BITS><<<(unsigned)blocks, kBlock, 0, st>>>(
          reinterpret_cast<const typename uint_of<2 * BITS>::type*>(pack), reinterpret_cast<u32x4*>(unpack), n_units);
      done = n_units * 16;
    }
  }
  if (done < n_out)
    unpack_rows_kernel<BITS><<<grid_for(n_out - done), kBlock, 0, st>>>(pack, unpack, done, n_out, U, P);
  return launch_status("unpackbits");
}

}  // namespace
}  // namespace f2cgt

using namespace f2cgt;

extern "C" int f2cgt_packbits(const uint8_t* unpack, uint8_t* pack, int64_t rows,
                              int64_t unpack_dim, int target_bits, void* stream) {
  F2CGT_REQUIRE(rows >= 0 && unpack_dim >= 0, F2CGT_E_INVALID, "packbits: negative size");
  F2CGT_REQUIRE(target_bits == 1 || target_bits == 2 || target_bits == 4, F2CGT_E_UNSUPPORTED,
                "packbits: target_bits must be 1, 2 or 4 (got %d)", target_bits);
  F2CGT_REQUIRE(rows == 0 || unpack_dim == 0 || (unpack && pack), F2CGT_E_INVALID,
                "packbits: null buffer");
  hipStream_t st = as_stream(stream);
  switch (target_bits) {
    case 1: return pack_launch<1>(unpack, pack, rows, unpack_dim, st);
    case 2: return pack_launch<2>(unpack, pack, rows, unpack_dim, st);
    default: return pack_launch<4>(unpack, pack, rows, unpack_dim, st);
  }
}

extern "C" int f2cgt_unpackbits(const uint8_t* pack, uint8_t* unpack, int64_t rows,
                                int64_t pack_dim, int64_t unpack_dim, int target_bits,
                                void* stream) {
  F2CGT_REQUIRE(rows >= 0 && unpack_dim >= 0 && pack_dim >= 0, F2CGT_E_INVALID,
                "unpackbits: negative size");
  F2CGT_REQUIRE(target_bits == 1 || target_bits == 2 || target_bits == 4, F2CGT_E_UNSUPPORTED,
                "unpackbits: target_bits must be 1, 2 or 4 (got %d)", target_bits);
  F2CGT_REQUIRE(unpack_dim <= pack_dim * (8 / target_bits), F2CGT_E_INVALID,
                "unpackbits: unpack_dim %lld exceeds %lld packed bytes per row", (long long)unpack_dim,
                (long long)pack_dim);
  F2CGT_REQUIRE(rows == 0 || unpack_dim == 0 || (unpack && pack), F2CGT_E_INVALID,
                "unpackbits: null buffer");
  hipStream_t st = as_stream(stream);
  switch (target_bits) {
    case 1: return unpack_launch<1>(pack, unpack, rows, pack_dim, unpack_dim, st);
    case 2: return unpack_launch<2>(pack, unpack, rows, pack_dim, unpack_dim, st);
    default: return unpack_launch<4>(pack, unpack, rows, pack_dim, unpack_dim, st);
  }
}
