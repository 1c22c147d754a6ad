// packbits / unpackbits: streaming byte kernels, 64-bit indexing.
//
// Two shapes each:
//   * flat: unpack_dim is a multiple of 8/bits, so the whole tensor is one stream and a
//     lane converts 4 packed bytes <-> 4*(8/bits) code bytes with dword accesses;
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

// Flat stream: lane g turns code bytes [4*PER*g, 4*PER*(g+1)) into packed dword g.
template <int BITS>
__global__ __launch_bounds__(kBlock) void pack_flat_kernel(const uint32_t* __restrict__ unpack,
                                                           uint32_t* __restrict__ pack,
                                                           int64_t n_words) {
  constexpr int PER = 8 / BITS;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x; g < n_words; g += stride) {
    uint32_t in[PER];
#pragma unroll
    for (int w = 0; w < PER; ++w) in[w] = unpack[g * PER + w];
    uint32_t out = 0;
#pragma unroll
    for (int e = 0; e < 4 * PER; ++e) {
      const uint32_t code = (in[e / 4] >> (8 * (e % 4))) & MASK;
      out |= code << (8 * (e / PER) + BITS * (e % PER));
    }
    pack[g] = out;
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
__global__ __launch_bounds__(kBlock) void unpack_flat_kernel(const uint32_t* __restrict__ pack,
                                                             uint32_t* __restrict__ unpack,
                                                             int64_t n_words) {
  constexpr int PER = 8 / BITS;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x; g < n_words; g += stride) {
    const uint32_t in = pack[g];
#pragma unroll
    for (int w = 0; w < PER; ++w) {
      uint32_t out = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = 4 * w + j;
        const uint32_t code = (in >> (8 * (e / PER) + BITS * (e % PER))) & MASK;
        out |= code << (8 * j);
      }
      unpack[g * PER + w] = out;
    }
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
  if (U % PER == 0 && aligned(unpack, 4) && aligned(pack, 4)) {
    const int64_t n_words = n_out / 4;
    if (n_words > 0) {
      pack_flat_kernel<BITS><<<grid_for(n_words), kBlock, 0, st>>>(
          reinterpret_cast<const uint32_t*>(unpack), reinterpret_cast<uint32_t*>(pack), n_words);
      done = n_words * 4;
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
  if (U == P * PER && aligned(unpack, 4) && aligned(pack, 4)) {
    const int64_t n_words = (rows * P) / 4;
    if (n_words > 0) {
      unpack_flat_kernel<BITS><<<grid_for(n_words), kBlock, 0, st>>>(
          reinterpret_cast<const uint32_t*>(pack), reinterpret_cast<uint32_t*>(unpack), n_words);
      done = n_words * 4 * PER;
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
