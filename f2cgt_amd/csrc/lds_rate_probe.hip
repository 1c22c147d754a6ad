// Experiments build only: how many bytes per clock the LDS of a CU returns to ds_read instructions.
//
// The fused VQ aggregation reads 512 bytes of codebook per edge and 128-column tile from LDS, so its
// sums cannot be faster than the LDS read rate.  The probe fills a 128 KB table, then every wave of
// a 1024-thread workgroup (16 waves per CU, as in the aggregation kernel) issues eight independent
// reads per trip in the aggregation kernel's own access shape: 16 consecutive lanes read 256
// contiguous bytes of a random 512-byte entry (conflict free whatever the entries are), as
// ds_read_b128 (one float4 per lane), ds_read_b64 (32 lanes per 256 bytes) or ds_read_b32 (64
// lanes per 256 bytes).  No global memory traffic in the timed loop.  Every workgroup reports the
// shader clocks its loop took, so the rate comes out per clock whatever the clock was.
#include "common.hpp"

namespace f2cgt {
namespace {

constexpr int kRateThreads = 1024;
constexpr int kRateLdsWords = 32768;   // 128 KB

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// width: bytes per lane and read (16, 8 or 4)
template <int WIDTH>
__global__ __launch_bounds__(kRateThreads) void lds_rate_probe_kernel(unsigned int* out, int iters) {
  extern __shared__ __align__(16) unsigned int lds[];
  for (int i = threadIdx.x; i < kRateLdsWords; i += kRateThreads) lds[i] = (unsigned int)i;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const unsigned int entry = ((threadIdx.x >> 4) * 2654435761u >> 10) & 127u;   // one entry per 16 lanes, fixed over the loop
  unsigned int acc = 0;
  const long long t0 = clock64();   // shader clock
  if constexpr (WIDTH == 16) {
    const u32x4* p = reinterpret_cast<const u32x4*>(lds + entry * 128 + (lane & 15) * 4);
    for (int it = 0; it < iters; ++it) {
      const u32x4 a = p[0], b = p[16], c = p[512], d = p[528], e = p[1024], f = p[1040], g = p[1536], h = p[1552];
      acc ^= a.x ^ b.y ^ c.z ^ d.w ^ e.x ^ f.y ^ g.z ^ h.w;
      asm volatile("" ::: "memory");
    }
  } else if constexpr (WIDTH == 8) {
    const u32x2* p = reinterpret_cast<const u32x2*>(lds + entry * 128 + (lane & 31) * 2);
    for (int it = 0; it < iters; ++it) {
      const u32x2 a = p[0], b = p[32], c = p[1024], d = p[1056], e = p[2048], f = p[2080], g = p[3072], h = p[3104];
      acc ^= a.x ^ b.y ^ c.x ^ d.y ^ e.x ^ f.y ^ g.x ^ h.y;
      asm volatile("" ::: "memory");
    }
  } else {
    const unsigned int* p = lds + entry * 128 + lane;
    for (int it = 0; it < iters; ++it) {
      const unsigned int a = p[0], b = p[64], c = p[1024], d = p[1088], e = p[2048], f = p[2112], g = p[3072], h = p[3136];
      acc ^= a ^ b ^ c ^ d ^ e ^ f ^ g ^ h;
      asm volatile("" ::: "memory");
    }
  }
  __syncthreads();
  const long long t1 = clock64();
  // shader clocks from the first wave's first read to the last wave's last; the xor keeps the loop alive (it is 0 or 1 here)
  if (threadIdx.x == 0) out[blockIdx.x] = (unsigned int)(t1 - t0) + (acc == 0x12345u ? 1u : 0u);
}

}  // namespace
}  // namespace f2cgt

// One launch on `workgroups` CUs: every wave issues 8 * iters reads of `width` bytes per lane.
// out needs `workgroups` words and receives the shader clocks each workgroup's loop took.
extern "C" int f2cgt_experiment_lds_rate_probe(unsigned int* out, int workgroups, int iters, int width, void* stream) {
  using namespace f2cgt;
  if (out == nullptr || workgroups < 1 || iters < 1 || (width != 16 && width != 8 && width != 4))
    return fail(F2CGT_E_INVALID, "lds_rate_probe: bad arguments");
  const void* kern = width == 16 ? reinterpret_cast<const void*>(lds_rate_probe_kernel<16>)
                   : width == 8  ? reinterpret_cast<const void*>(lds_rate_probe_kernel<8>)
                                 : reinterpret_cast<const void*>(lds_rate_probe_kernel<4>);
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, kRateLdsWords * 4);
  if (e != hipSuccess) return fail((int)e, "lds_rate_probe: cannot reserve %d B of LDS", kRateLdsWords * 4);
  void* params[] = {&out, &iters};
  const hipError_t le = hipLaunchKernel(kern, dim3((unsigned)workgroups), dim3(kRateThreads), params,
                                        (size_t)kRateLdsWords * 4, as_stream(stream));
  if (le != hipSuccess) return fail((int)le, "lds_rate_probe: launch failed: %s", hipGetErrorString(le));
  return launch_status("lds_rate_probe");
}
