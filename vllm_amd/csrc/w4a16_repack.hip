// GPTQ / AWQ int4 weight repack for gfx950.
//
// Input : GPTQ checkpoint tensor int32 [K/8, N]; word (r, n) holds codes of rows 8r..8r+7 of column n, row 8r+e in
//         bits [4e, 4e+4);
//         or AWQ (AutoAWQ) checkpoint tensor int32 [K, N/8]; word (k, c) holds the codes of row k, columns 8c..8c+7,
//         column 8c + {0,2,4,6,1,3,5,7}[p] in nibble position p.
// Output: int32 [K/16, 2N] (same byte count) in one of two orders.
//
//  NATIVE (what the GEMM kernels stream)
//    The matrix is cut into tiles of 128 rows (k) x 16 columns (n); tile (kt, nt) is the 1 KiB block number
//    nt * (K/128) + kt: the tiles of one 16-column strip are contiguous along K, so a wavefront that walks K for its
//    strip reads one sequential stream (measured: strided 1 KiB reads cost ~1.6x against sequential ones).
//    Inside a tile, lane L = 16*o + r (o = 0..3, r = 0..15) of a 64-wide wavefront owns the
//    16 bytes at offset 16*L: four words j = 0..3, word j holding the 8 codes of rows
//        k = 128*kt + 32*j + 8*o + e  (e = 0..7),  column n = 16*nt + r,
//    with code e stored in nibble position p where {0,2,4,6,1,3,5,7}[p] == e.  One 16-byte load per lane therefore
//    yields the A operands (row = n, 8 consecutive k per lane) of four v_mfma_f32_16x16x32 instructions that together
//    cover one quantisation group of 128 rows, and `(w >> 4i) & 0x000f000f | EX` produces operand register i directly.
//
//  MARLIN (bit-exact with the reference's gptq_marlin_repack, kept for the parity contract)
//    16 x 64 tiles; output word (kt*(N/64) + nt)*128 + th*4 + warp, th = 0..31, warp = 0..3, holds codes of rows
//    16*kt + 2*(th%4) + {0,1,8,9} for column 64*nt + 16*warp + th/4 (first four) and that column + 8 (last four),
//    nibble order {0,2,4,6,1,3,5,7}.
//
// 8-bit codes (GPTQ int32 [K/4, N], row 4r+e in bits [8e, 8e+8)) go to int32 [K/16, 4N]:
//  NATIVE  two 4-bit planes per tile: block 2*(nt*(K/128)+kt) holds the high nibbles (code >> 4) of the tile in the
//          order above, the next block the low nibbles, so the 4-bit kernels' dequantisation applies to each plane.
//  MARLIN  16 x 64 tiles of 256 words; words th*8 + warp*2 + {0, 1} hold, one byte each, rows 16*kt + 2*(th%4) +
//          {0, 8, 1, 9} of column 64*nt + 16*warp + th/4 (word 0) and that column + 8 (word 1).
//  NATIVE_BYTES (FP8 e4m3 weights, whose codes are not linear in their bits, so the nibble planes are of no use): per
//          tile two 1 KiB blocks; block h (0 / 1) gives lane L = 16*o + r the 16 bytes of rows 128*kt + 32*j + 8*o + e,
//          j = 2h (bytes 0..7, e = byte index) and j = 2h + 1 (bytes 8..15), column 16*nt + r: every 8 bytes are the A
//          operand of one v_mfma_f32_16x16x32 after four packed FP8 -> 16-bit conversions.
//
// With `perm` (act_order sort indices) output row k takes input row perm[k].
#include "vaq_common.h"

namespace vaq {

__device__ inline uint32_t fetch_code(const uint32_t* __restrict__ qw, const int32_t* __restrict__ perm, int64_t k,
                                      int64_t n, int64_t size_n) {
  int64_t src = perm ? (int64_t)perm[k] : k;
  uint32_t word = qw[(src >> 3) * size_n + n];
  return (word >> ((src & 7) * 4)) & 0xFu;
}

// AWQ source: nibble position of column n inside its word is {0,4,1,5,2,6,3,7}[n % 8] (the inverse of the AutoAWQ
// interleave {0,2,4,6,1,3,5,7}); reference: awq_marlin_repack.cu:95-103.
__device__ inline uint32_t fetch_code_awq(const uint32_t* __restrict__ qw, int64_t k, int64_t n, int64_t size_n) {
  const uint32_t word = qw[k * (size_n >> 3) + (n >> 3)];
  const int pos = (int)(((n & 1) << 2) | ((n & 7) >> 1));
  return (word >> (pos * 4)) & 0xFu;
}

__device__ inline uint32_t fetch_code8(const uint32_t* __restrict__ qw, const int32_t* __restrict__ perm, int64_t k,
                                       int64_t n, int64_t size_n) {
  int64_t src = perm ? (int64_t)perm[k] : k;
  uint32_t word = qw[(src >> 2) * size_n + n];
  return (word >> ((src & 3) * 8)) & 0xFFu;
}

__device__ inline uint32_t interleave_pack(const uint32_t v[8]) {
  // nibble position p <- element {0,2,4,6,1,3,5,7}[p]
  return v[0] | (v[2] << 4) | (v[4] << 8) | (v[6] << 12) | (v[1] << 16) | (v[3] << 20) | (v[5] << 24) | (v[7] << 28);
}

// One thread per output word; native layout.
template <bool HAS_PERM, bool AWQ>
__global__ __launch_bounds__(256) void repack_native_kernel(const uint32_t* __restrict__ qw,
                                                             const int32_t* __restrict__ perm,
                                                             uint32_t* __restrict__ out, int64_t size_k,
                                                             int64_t size_n) {
  const int64_t total = size_k * size_n / 8;
  const int64_t k_tiles = size_k / 128;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int j = idx & 3;
    const int lane = (idx >> 2) & 63;
    const int64_t tile = idx >> 8;
    const int64_t nt = tile / k_tiles, kt = tile - nt * k_tiles;
    const int o = lane >> 4, r = lane & 15;
    const int64_t k0 = kt * 128 + j * 32 + o * 8;
    const int64_t n = nt * 16 + r;
    uint32_t res;
    if constexpr (AWQ) {
      uint32_t v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = fetch_code_awq(qw, k0 + e, n, size_n);
      res = interleave_pack(v);
    } else if constexpr (HAS_PERM) {
      uint32_t v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = fetch_code(qw, perm, k0 + e, n, size_n);
      res = interleave_pack(v);
    } else {
      // the 8 codes are exactly one input word; only the nibble order changes
      const uint32_t w = qw[(k0 >> 3) * size_n + n];
      uint32_t v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (w >> (4 * e)) & 0xFu;
      res = interleave_pack(v);
    }
    out[idx] = res;
  }
}

// One thread per output word; reference (Marlin) order.
template <bool AWQ>
__global__ __launch_bounds__(256) void repack_marlin_kernel(const uint32_t* __restrict__ qw,
                                                             const int32_t* __restrict__ perm,
                                                             uint32_t* __restrict__ out, int64_t size_k,
                                                             int64_t size_n) {
  const int64_t total = size_k * size_n / 8;
  const int64_t n_tiles = size_n / 64;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int warp = idx & 3;
    const int th = (idx >> 2) & 31;
    const int64_t tile = idx >> 7;
    const int64_t kt = tile / n_tiles, nt = tile - kt * n_tiles;
    const int64_t n = nt * 64 + warp * 16 + (th >> 2);
    const int64_t kbase = kt * 16 + (th & 3) * 2;
    const int off[4] = {0, 1, 8, 9};
    uint32_t v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (AWQ) {
        v[i] = fetch_code_awq(qw, kbase + off[i], n, size_n);
        v[4 + i] = fetch_code_awq(qw, kbase + off[i], n + 8, size_n);
      } else {
        v[i] = fetch_code(qw, perm, kbase + off[i], n, size_n);
        v[4 + i] = fetch_code(qw, perm, kbase + off[i], n + 8, size_n);
      }
    }
    out[idx] = interleave_pack(v);
  }
}

// 8-bit codes, native layout: one thread per output word of one nibble plane.
__global__ __launch_bounds__(256) void repack_native8_kernel(const uint32_t* __restrict__ qw,
                                                              const int32_t* __restrict__ perm,
                                                              uint32_t* __restrict__ out, int64_t size_k,
                                                              int64_t size_n) {
  const int64_t total = size_k * size_n / 4;
  const int64_t k_tiles = size_k / 128;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int j = idx & 3;
    const int lane = (idx >> 2) & 63;
    const int plane = (idx >> 8) & 1;
    const int64_t tile = idx >> 9;
    const int64_t nt = tile / k_tiles, kt = tile - nt * k_tiles;
    const int o = lane >> 4, r = lane & 15;
    const int64_t k0 = kt * 128 + j * 32 + o * 8;
    const int64_t n = nt * 16 + r;
    uint32_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t c = fetch_code8(qw, perm, k0 + e, n, size_n);
      v[e] = plane ? (c & 0xFu) : (c >> 4);
    }
    out[idx] = interleave_pack(v);
  }
}

// 8-bit codes kept as bytes (NATIVE_BYTES): one thread per output word (four consecutive rows of one column).
__global__ __launch_bounds__(256) void repack_native8_bytes_kernel(const uint32_t* __restrict__ qw,
                                                                    const int32_t* __restrict__ perm,
                                                                    uint32_t* __restrict__ out, int64_t size_k,
                                                                    int64_t size_n) {
  const int64_t total = size_k * size_n / 4;
  const int64_t k_tiles = size_k / 128;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int q = idx & 3;
    const int lane = (idx >> 2) & 63;
    const int h = (idx >> 8) & 1;
    const int64_t tile = idx >> 9;
    const int64_t nt = tile / k_tiles, kt = tile - nt * k_tiles;
    const int o = lane >> 4, r = lane & 15;
    const int j = 2 * h + (q >> 1);
    const int64_t k0 = kt * 128 + j * 32 + o * 8 + (q & 1) * 4;
    const int64_t n = nt * 16 + r;
    uint32_t res = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) res |= fetch_code8(qw, perm, k0 + e, n, size_n) << (8 * e);
    out[idx] = res;
  }
}

// 8-bit codes, reference (Marlin) order: one thread per output word.
__global__ __launch_bounds__(256) void repack_marlin8_kernel(const uint32_t* __restrict__ qw,
                                                              const int32_t* __restrict__ perm,
                                                              uint32_t* __restrict__ out, int64_t size_k,
                                                              int64_t size_n) {
  const int64_t total = size_k * size_n / 4;
  const int64_t n_tiles = size_n / 64;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int which = idx & 1;
    const int warp = (idx >> 1) & 3;
    const int th = (idx >> 3) & 31;
    const int64_t tile = idx >> 8;
    const int64_t kt = tile / n_tiles, nt = tile - kt * n_tiles;
    const int64_t n = nt * 64 + warp * 16 + (th >> 2) + which * 8;
    const int64_t kbase = kt * 16 + (th & 3) * 2;
    const int off[4] = {0, 8, 1, 9};     // byte i <- row offset {0, 1, 8, 9}[{0, 2, 1, 3}[i]]
    uint32_t res = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) res |= fetch_code8(qw, perm, kbase + off[i], n, size_n) << (8 * i);
    out[idx] = res;
  }
}

}  // namespace vaq

static int repack_common(const int32_t* qweight, const int32_t* perm, int32_t* out, int64_t size_k, int64_t size_n,
                         int num_bits, int layout, bool awq, void* stream) {
  using namespace vaq;
  VAQ_CHECK_ARG(num_bits == 4 || num_bits == 8, "w4a16_repack: num_bits must be 4 or 8. Got = %d", num_bits);
  VAQ_CHECK_SUPPORTED(num_bits == 4 || !awq, "w4a16_repack: 8-bit AWQ weights are not built");
  VAQ_CHECK_ARG(size_k > 0 && size_k % 16 == 0, "w4a16_repack: size_k = %lld is not divisible by tile_k_size = 16",
                (long long)size_k);
  VAQ_CHECK_ARG(size_n > 0 && size_n % 64 == 0, "w4a16_repack: size_n = %lld is not divisible by tile_n_size = 64",
                (long long)size_n);
  VAQ_CHECK_ARG(layout == VAQ_LAYOUT_MARLIN || layout == VAQ_LAYOUT_NATIVE || layout == VAQ_LAYOUT_NATIVE_BYTES,
                "w4a16_repack: unknown layout %d", layout);
  VAQ_CHECK_ARG(layout != VAQ_LAYOUT_NATIVE_BYTES || (num_bits == 8 && !awq),
                "w4a16_repack: the byte layout is for 8-bit GPTQ-packed weights");
  VAQ_CHECK_ARG(layout == VAQ_LAYOUT_MARLIN || size_k % 128 == 0,
                "w4a16_repack: native layout needs size_k %% 128 == 0, got size_k = %lld", (long long)size_k);
  VAQ_CHECK_ARG(qweight && out, "w4a16_repack: null pointer");
  const int64_t total = size_k * size_n / (32 / num_bits);
  const int threads = 256;
  int64_t blocks = (total + threads - 1) / threads;
  const int64_t cap = (int64_t)num_cus_current_device() * 16;
  if (blocks > cap) blocks = cap;
  hipStream_t s = (hipStream_t)stream;
  const uint32_t* qw = (const uint32_t*)qweight;
  uint32_t* o = (uint32_t*)out;
  const dim3 grid((unsigned)blocks), block(threads);
  if (num_bits == 8) {
    if (layout == VAQ_LAYOUT_NATIVE) hipLaunchKernelGGL(repack_native8_kernel, grid, block, 0, s, qw, perm, o, size_k, size_n);
    else if (layout == VAQ_LAYOUT_NATIVE_BYTES) hipLaunchKernelGGL(repack_native8_bytes_kernel, grid, block, 0, s, qw, perm, o, size_k, size_n);
    else hipLaunchKernelGGL(repack_marlin8_kernel, grid, block, 0, s, qw, perm, o, size_k, size_n);
  } else if (layout == VAQ_LAYOUT_NATIVE) {
    if (awq)
      hipLaunchKernelGGL((repack_native_kernel<false, true>), grid, block, 0, s, qw, perm, o, size_k, size_n);
    else if (perm)
      hipLaunchKernelGGL((repack_native_kernel<true, false>), grid, block, 0, s, qw, perm, o, size_k, size_n);
    else
      hipLaunchKernelGGL((repack_native_kernel<false, false>), grid, block, 0, s, qw, perm, o, size_k, size_n);
  } else {
    if (awq)
      hipLaunchKernelGGL(repack_marlin_kernel<true>, grid, block, 0, s, qw, perm, o, size_k, size_n);
    else
      hipLaunchKernelGGL(repack_marlin_kernel<false>, grid, block, 0, s, qw, perm, o, size_k, size_n);
  }
  VAQ_CHECK_LAUNCH("w4a16_repack");
  return VAQ_OK;
}

extern "C" int vaq_w4a16_repack(const int32_t* qweight, const int32_t* perm, int32_t* out, int64_t size_k,
                                int64_t size_n, int num_bits, int layout, void* stream) {
  return repack_common(qweight, perm, out, size_k, size_n, num_bits, layout, false, stream);
}

extern "C" int vaq_w4a16_repack_awq(const int32_t* qweight, int32_t* out, int64_t size_k, int64_t size_n, int num_bits,
                                    int layout, void* stream) {
  return repack_common(qweight, nullptr, out, size_k, size_n, num_bits, layout, true, stream);
}
