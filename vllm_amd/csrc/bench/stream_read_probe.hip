// Measurement aid, not part of the quantized-linear library (built into libvaq_bench_probe.so, which only the
// benchmark loads): a kernel that does nothing but read a buffer, every load of
// a wavefront in flight at once.  Launched inside the same kind of HIP graph as the decode GEMMs, on buffers of a
// layer's size that have left the caches, its launch-to-launch time is the ceiling any kernel that has to read those
// bytes can reach on this machine (launch gap + first-byte latency + streaming): the "practical peak" the benchmark
// reports beside the nominal 8 TB/s.
#include "../vaq_common.h"

namespace vaq {

// Each wavefront reads `per` consecutive 1 KiB pieces (one 16-byte load per lane and piece), U of them per trip.
template <int U>
__global__ __launch_bounds__(256) void stream_read_kernel(const v4u* __restrict__ src, uint32_t* sink, int per) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const v4u* p = src + wave * (int64_t)per * 64 + lane;
  v4u acc = {0u, 0u, 0u, 0u};
  for (int i = 0; i + U <= per; i += U) {
    v4u v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + (int64_t)(i + u) * 64);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  for (int i = per - per % U; i < per; ++i) acc ^= __builtin_nontemporal_load(p + (int64_t)i * 64);
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;      // keeps the loads alive; practically never true
}

}  // namespace vaq

// Reads `bytes` (rounded down to whole KiB per wavefront) from `src` with `waves` wavefronts (a multiple of 4) and
// `depth` (2, 4 or 8) 16-byte loads per lane in flight.  `sink` is a device word that is practically never written.
// Returns 0, or -1 for arguments it does not take and -3 for a refused launch.
extern "C" __attribute__((visibility("default"))) int vaq_stream_read_probe(const void* src, int64_t bytes, int waves, int depth, void* sink, void* stream) {
  using namespace vaq;
  if (!(src && sink && ((uintptr_t)src % 16) == 0)) return -1;
  if (!(waves > 0 && waves % 4 == 0 && waves <= (1 << 20))) return -1;
  if (!(depth == 2 || depth == 4 || depth == 8)) return -1;
  const int64_t per = bytes / 1024 / waves;
  if (!(per >= 1 && per < (1 << 30))) return -1;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(waves / 4), block(256);
  if (depth == 2) hipLaunchKernelGGL(stream_read_kernel<2>, grid, block, 0, s, (const v4u*)src, (uint32_t*)sink, (int)per);
  else if (depth == 4) hipLaunchKernelGGL(stream_read_kernel<4>, grid, block, 0, s, (const v4u*)src, (uint32_t*)sink, (int)per);
  else hipLaunchKernelGGL(stream_read_kernel<8>, grid, block, 0, s, (const v4u*)src, (uint32_t*)sink, (int)per);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
