// Experiments build only: does the matrix core run in the shadow of vector / LDS work of the same SIMD?
//
// The question behind fusing the dense layer into the aggregation (one kernel that gathers and
// sums codebook rows and multiplies the result by the layer's weights with fp32 MFMA): the gather
// side is LDS reads plus vector adds, the GEMM side is v_mfma_f32_32x32x2_f32.  The probe runs
// both instruction mixes on registers and a 64 KB LDS table, with no global memory traffic in the
// timed loops, in four arrangements per CU:
//     mfma     4 waves (one per SIMD), MFMA only
//     gather   4 waves (one per SIMD), ds_read_b128 + adds only
//     split    8 waves: waves 0-3 MFMA, waves 4-7 gather (the two kinds share every SIMD)
//     mixed    4 waves, each issuing both kinds from one loop (independent registers)
// and, to tell the two halves of the gather side apart, with only its LDS reads or only its adds:
//     lds / adds            4 waves, that half alone
//     split-lds / split-adds   8 waves: 4 MFMA + 4 of that half
// If the two kinds overlap, `split` and `mixed` take about max(mfma, gather); if they do not, about
// the sum.
#include "common.hpp"

namespace f2cgt {
namespace {

typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kProbeThreads = 512;
constexpr int kProbeLdsFloats = 16384;   // 64 KB

template <bool MFMA, bool GATHER, bool READS = true, bool ADDS = true>
__device__ __forceinline__ void probe_loop(const float* lds, int iters, int lane, float seed, float& sink) {
  f16v acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = seed + (float)(t * 16 + v);
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  unsigned int at = (unsigned int)lane * 2654435761u;
  const float a = seed * 0.5f, b = seed * 0.25f;
  for (int it = 0; it < iters; ++it) {
    if (MFMA) {
#pragma unroll
      for (int t = 0; t < 8; ++t) acc[t & 3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[t & 3], 0, 0, 0);
    }
    if (GATHER) {
      float4 x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (READS) {
          at = at * 1664525u + 1013904223u;
          x[u] = *reinterpret_cast<const float4*>(lds + ((at >> 8) & (kProbeLdsFloats - 4) & ~3u));
          if (!ADDS) asm volatile("" ::"v"(x[u].x), "v"(x[u].y), "v"(x[u].z), "v"(x[u].w));   // the read stays
        } else {
          x[u] = make_float4(seed, a, b, seed);
        }
      }
      if (ADDS) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          s[(u & 1) * 4 + 0] += x[u].x; s[(u & 1) * 4 + 1] += x[u].y;
          s[(u & 1) * 4 + 2] += x[u].z; s[(u & 1) * 4 + 3] += x[u].w;
        }
        if (!READS) asm volatile("" : "+v"(s[0]), "+v"(s[1]), "+v"(s[2]), "+v"(s[3]), "+v"(s[4]), "+v"(s[5]), "+v"(s[6]), "+v"(s[7]));
      }
    }
  }
  float r = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) r += acc[t][v];
#pragma unroll
  for (int u = 0; u < 8; ++u) r += s[u];
  sink = r;
}

// arrangement: 0 mfma, 1 gather, 2 split, 3 mixed, 4 lds, 5 adds, 6 split-lds, 7 split-adds
__global__ __launch_bounds__(kProbeThreads) void overlap_probe_kernel(float* out, int iters, int arrangement, float seed) {
  extern __shared__ __align__(16) float lds[];
  for (int i = threadIdx.x; i < kProbeLdsFloats; i += kProbeThreads) lds[i] = seed + (float)(i & 255);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float sink = 0.f;
  if (arrangement == 0) {
    if (wave < 4) probe_loop<true, false>(lds, iters, lane, seed, sink);
  } else if (arrangement == 1) {
    if (wave < 4) probe_loop<false, true>(lds, iters, lane, seed, sink);
  } else if (arrangement == 2) {
    if (wave < 4) probe_loop<true, false>(lds, iters, lane, seed, sink);
    else probe_loop<false, true>(lds, iters, lane, seed, sink);
  } else if (arrangement == 3) {
    if (wave < 4) probe_loop<true, true>(lds, iters, lane, seed, sink);
  } else if (arrangement == 4) {
    if (wave < 4) probe_loop<false, true, true, false>(lds, iters, lane, seed, sink);
  } else if (arrangement == 5) {
    if (wave < 4) probe_loop<false, true, false, true>(lds, iters, lane, seed, sink);
  } else if (arrangement == 6) {
    if (wave < 4) probe_loop<true, false>(lds, iters, lane, seed, sink);
    else probe_loop<false, true, true, false>(lds, iters, lane, seed, sink);
  } else {
    if (wave < 4) probe_loop<true, false>(lds, iters, lane, seed, sink);
    else probe_loop<false, true, false, true>(lds, iters, lane, seed, sink);
  }
  if (sink == 12345.678f) out[blockIdx.x] = sink;   // keeps the loops alive, never true for the seeds used
}

}  // namespace
}  // namespace f2cgt

// One launch of the probe on every CU (`workgroups` of them): out needs `workgroups` floats.
extern "C" int f2cgt_experiment_overlap_probe(float* out, int workgroups, int iters, int arrangement, void* stream) {
  using namespace f2cgt;
  if (out == nullptr || workgroups < 1 || iters < 1 || arrangement < 0 || arrangement > 7)
    return fail(F2CGT_E_INVALID, "overlap_probe: bad arguments");
  overlap_probe_kernel<<<(unsigned)workgroups, kProbeThreads, kProbeLdsFloats * 4, as_stream(stream)>>>(out, iters,
                                                                                                      arrangement, 1.0f);
  return launch_status("overlap_probe");
}
