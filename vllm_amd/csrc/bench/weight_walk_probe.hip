// Measurement aid, not part of the quantized-linear library (built into libvaq_bench_probe.so, which only the
// benchmark loads): reads a row-major weight matrix the way a GEMM tile kernel does, and nothing else.  A workgroup owns
// ROWS consecutive weight rows and walks along them, taking C bytes of every row per step with DEPTH steps in flight.
// On weights that have left the caches this tells whether that access pattern -- short pieces of many rows instead of
// long runs of one -- is what holds a GEMM of few activation rows below the memory system's rate.
#include "../vaq_common.h"

namespace vaq {

template <int C, int DEPTH, int ROWS>
__global__ __launch_bounds__(256) void weight_walk_kernel(const uint8_t* __restrict__ base, int rowbytes, uint32_t* sink) {
  constexpr int PPR = C / 16;            // 16-byte pieces per row and step
  constexpr int RPP = 256 / PPR;         // rows covered by one load instruction of the workgroup
  constexpr int PASSES = ROWS / RPP;     // load instructions per step
  static_assert(PASSES >= 1 && ROWS % RPP == 0, "rows per workgroup");
  const int t = threadIdx.x;
  const int piece = t % PPR, r0 = t / PPR;
  const uint8_t* wg = base + (size_t)blockIdx.x * ROWS * rowbytes;
  v4u acc = {0u, 0u, 0u, 0u};
  const int steps = rowbytes / C;
  for (int it = 0; it + DEPTH <= steps; it += DEPTH) {
    v4u v[DEPTH][PASSES];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
#pragma unroll
      for (int p = 0; p < PASSES; ++p)
        v[d][p] = *reinterpret_cast<const v4u*>(wg + (size_t)(p * RPP + r0) * rowbytes + (size_t)(it + d) * C + piece * 16);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
#pragma unroll
      for (int p = 0; p < PASSES; ++p) acc ^= v[d][p];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;      // keeps the loads alive; practically never true
}

struct WalkConfig {
  const char* name;
  int rows;
  void (*launch)(const uint8_t*, int, int, uint32_t*, hipStream_t);
};

template <int C, int DEPTH, int ROWS>
static void launch_walk(const uint8_t* base, int rows_total, int rowbytes, uint32_t* sink, hipStream_t s) {
  hipLaunchKernelGGL((weight_walk_kernel<C, DEPTH, ROWS>), dim3(rows_total / ROWS), dim3(256), 0, s, base, rowbytes, sink);
}

static const WalkConfig WALKS[] = {
    {"128 rows per workgroup,   64 bytes per row and step, 4 steps in flight", 128, launch_walk<64, 4, 128>},
    {"128 rows per workgroup,  128 bytes per row and step, 2 steps in flight", 128, launch_walk<128, 2, 128>},
    {"128 rows per workgroup,  256 bytes per row and step, 2 steps in flight", 128, launch_walk<256, 2, 128>},
    {"128 rows per workgroup,  512 bytes per row and step, 1 step  in flight", 128, launch_walk<512, 1, 128>},
    {"256 rows per workgroup,   64 bytes per row and step, 4 steps in flight", 256, launch_walk<64, 4, 256>},
    {"256 rows per workgroup,  256 bytes per row and step, 1 step  in flight", 256, launch_walk<256, 1, 256>},
    {" 64 rows per workgroup,   64 bytes per row and step, 8 steps in flight", 64, launch_walk<64, 8, 64>},
    {" 16 rows per workgroup, 4096 bytes per row and step, 1 step  in flight", 16, launch_walk<4096, 1, 16>},
};

}  // namespace vaq

extern "C" __attribute__((visibility("default"))) int vaq_weight_walk_probe_count() {
  return (int)(sizeof(vaq::WALKS) / sizeof(vaq::WALKS[0]));
}
extern "C" __attribute__((visibility("default"))) const char* vaq_weight_walk_probe_name(int i) {
  return i >= 0 && i < vaq_weight_walk_probe_count() ? vaq::WALKS[i].name : "";
}
// Walks configuration `i` over `rows` rows of `rowbytes` bytes at `src` (16-byte aligned; rows a multiple of 256, rowbytes
// of 4096).  Returns 0, or -1 for arguments it does not take and -3 for a refused launch.
extern "C" __attribute__((visibility("default"))) int vaq_weight_walk_probe(int i, const void* src, int rows, int rowbytes,
                                                                            void* sink, void* stream) {
  using namespace vaq;
  if (!(i >= 0 && i < vaq_weight_walk_probe_count() && src && sink && ((uintptr_t)src % 16) == 0)) return -1;
  if (!(rows > 0 && rows % 256 == 0 && rowbytes > 0 && rowbytes % 4096 == 0)) return -1;
  WALKS[i].launch((const uint8_t*)src, rows, rowbytes, (uint32_t*)sink, (hipStream_t)stream);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
