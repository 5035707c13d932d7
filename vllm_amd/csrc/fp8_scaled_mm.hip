// FP8 (e4m3fn x e4m3fn) scaled GEMM for gfx950:
//     out[m,n] = round( sa[m] * ( sb[n] * sum_k a[m,k] b[k,n] ) + bias[n] ),   fp32 accumulation and epilogue.
// a is [M,K] row-major, b is [K,N] column-major (= weight [N,K] row-major with row pitch ldb), so both operands are
// k-contiguous and go to the matrix cores without any data re-arrangement.
//
// Two kernels:
//  * tile kernel (any M): one workgroup of 4 wavefronts (2 x 2) per BM x BN output tile, K walked in steps of 128
//    bytes through double-buffered, padded LDS (pitch 144 B), v_mfma_f32_32x32x64_f8f6f4 (the full-rate gfx950 FP8
//    instruction, 32 bytes per lane per operand);
//  * stream kernel (M <= 32; M <= 64 on narrow layers with K <= 4096): weight-streaming GEMV-like kernel, weights are the A operand of
//    v_mfma_f32_16x16x128_f8f6f4 straight from global memory, activations stay in registers, the wavefronts of a
//    workgroup split K and reduce through LDS.
//
// The per-lane byte -> k assignment inside an MFMA operand is the same function for A and B, so any consistent choice
// of which 32 bytes a lane supplies yields the exact dot product; both kernels give lane (row, q) the bytes
// k0 + 32*q .. k0 + 32*q + 31 of its row.
#include "vaq_common.h"
#include "tile_handover.h"

#include <type_traits>

namespace vaq {

struct Fp8MMParams {
  const uint8_t* a;
  int64_t lda;
  const uint8_t* b;
  int64_t ldb;
  const float* sa;
  int sa_per_row;   // 1: sa[m], 0: sa[0]
  const float* sb;
  int sb_per_col;
  const uint16_t* bias;
  uint16_t* out;
  int64_t ldc;
  int M, N, K;
  float* c_tmp = nullptr;        // fp32 partial tiles when K is split over workgroups (SK > 1)
  int32_t* counters = nullptr;   // arrival counters, zero on entry, left zero
  int SK = 1;
  int tail_first = 0;            // 0: every tile in SK parts; > 0: only the tiles from this position on (see tile_slot)
  int rotate_k = 0;              // multi-stage tile kernel: 1 tile rows, 2 tile columns start their K loop at different places (see the kernel)
  int m_tiles_extra = 0;         // multi-stage tile kernel: tile rows past M (see dispatch_tile: they read the weights with the real ones and store nothing)
  uint32_t a_extent = 0, b_extent = 0;   // stream kernel: bytes up to the end of the last row of a / b (below 2 GiB)
  int nt_base = 0, nt_rem = 0;   // stream kernel: n-tiles per workgroup = nt_base, one more for the first nt_rem (N/16 split on the host)
};

__device__ inline v16f mfma_fp8_32(v8i a, v8i b, v16f c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
__device__ inline v4f mfma_fp8_16(v8i a, v8i b, v4f c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

constexpr int F8_BK = 128;       // bytes of K per step
constexpr int F8_PITCH = 144;    // LDS row pitch in bytes

// Epilogue of the tile kernels.  The MFMAs are issued with the weight fragment as the A operand, so a 32x32
// accumulator block holds D[n_local][m_local]: lane -> column m_local = lane & 31, registers e -> rows
// n_local = 8*(e/4) + 4*(lane/32) + e%4.  Four consecutive registers are four consecutive n of one output row: one
// 8-byte store, one scale load per row, one 16-byte load of the channel scales.
template <bool BF16_OUT, int WMB, int WNB>
__device__ inline void tile_epilogue(const Fp8MMParams& p, v16f (&acc)[WMB][WNB], int m0, int n0, int wm, int wn, int lane) {
#pragma clang fp contract(off)      // sa * (sb * acc), then + bias: two fp32 roundings, like the oracle's separate operations
  using T = F16Traits<BF16_OUT>;
  // Every scale and bias value this lane needs is requested before the first store: a load that follows a store to
  // memory it might alias cannot be moved above it, and the epilogue would pay one memory latency per 8-byte store.
  float sam[WMB];
#pragma unroll
  for (int i = 0; i < WMB; ++i) {
    const int m = m0 + wm * 32 * WMB + i * 32 + (lane & 31);
    sam[i] = m < p.M ? p.sa[p.sa_per_row ? m : 0] : 0.f;
  }
  v4f sbv[WNB][4];
  v2u bv[WNB][4];
#pragma unroll
  for (int j = 0; j < WNB; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + wn * 32 * WNB + j * 32 + 8 * q + 4 * (lane >> 5);
      sbv[j][q] = v4f{0.f, 0.f, 0.f, 0.f};
      bv[j][q] = v2u{0u, 0u};
      if (n < p.N) {
        if (p.sb_per_col) sbv[j][q] = *reinterpret_cast<const v4f*>(p.sb + n);
        else sbv[j][q] = v4f{p.sb[0], p.sb[0], p.sb[0], p.sb[0]};
        if (p.bias) bv[j][q] = *reinterpret_cast<const v2u*>(p.bias + n);
      }
    }
#pragma unroll
  for (int i = 0; i < WMB; ++i) {
    const int m = m0 + wm * 32 * WMB + i * 32 + (lane & 31);
    if (m >= p.M) continue;
    uint16_t* orow = p.out + (int64_t)m * p.ldc;
#pragma unroll
    for (int j = 0; j < WNB; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * 32 * WNB + j * 32 + 8 * q + 4 * (lane >> 5);
        if (n >= p.N) continue;
        float o[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = sam[i] * (sbv[j][q][r] * acc[i][j][4 * q + r]);
        if (p.bias) {
          o[0] += T::to_float((uint16_t)(bv[j][q].x & 0xffffu));
          o[1] += T::to_float((uint16_t)(bv[j][q].x >> 16));
          o[2] += T::to_float((uint16_t)(bv[j][q].y & 0xffffu));
          o[3] += T::to_float((uint16_t)(bv[j][q].y >> 16));
        }
        v2u ov;
        ov.x = (uint32_t)T::from_float(o[0]) | ((uint32_t)T::from_float(o[1]) << 16);
        ov.y = (uint32_t)T::from_float(o[2]) | ((uint32_t)T::from_float(o[3]) << 16);
        *reinterpret_cast<v2u*>(orow + n) = ov;
      }
    }
  }
}

// Epilogue of the multi-stage kernel: same arithmetic as tile_epilogue, but the 16-bit results cross a wavefront-private
// piece of LDS (32 rows of WNB * 64 + 16 bytes) so that they leave as 16-byte stores, 8 or 16 lanes to a row.  With the
// direct 8-byte stores every instruction touches 32 rows with 16 bytes each, and the write requests of a whole device
// finishing its tiles at the same time (one 16-byte piece each) took 10-17 us per tile.
// Requires: every wavefront of the workgroup has finished reading the operand ring, out 16-byte aligned.
template <bool BF16_OUT, int WMB, int WNB>
__device__ inline void tile_epilogue_lds(const Fp8MMParams& p, v16f (&acc)[WMB][WNB], int m0, int n0, int wm, int wn, int lane,
                                         uint8_t* wave_lds) {
#pragma clang fp contract(off)      // sa * (sb * acc), then + bias: two fp32 roundings, like the oracle's separate operations
  using T = F16Traits<BF16_OUT>;
  constexpr int PITCH = WNB * 64 + 16;
  constexpr int CPR = WNB * 4;                 // 16-byte chunks per row
  float sam[WMB];
#pragma unroll
  for (int i = 0; i < WMB; ++i) {
    const int m = m0 + wm * 32 * WMB + i * 32 + (lane & 31);
    sam[i] = m < p.M ? p.sa[p.sa_per_row ? m : 0] : 0.f;
  }
  v4f sbv[WNB][4];
  v2u bv[WNB][4];
#pragma unroll
  for (int j = 0; j < WNB; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + wn * 32 * WNB + j * 32 + 8 * q + 4 * (lane >> 5);
      sbv[j][q] = v4f{0.f, 0.f, 0.f, 0.f};
      bv[j][q] = v2u{0u, 0u};
      if (n < p.N) {
        if (p.sb_per_col) sbv[j][q] = *reinterpret_cast<const v4f*>(p.sb + n);
        else sbv[j][q] = v4f{p.sb[0], p.sb[0], p.sb[0], p.sb[0]};
        if (p.bias) bv[j][q] = *reinterpret_cast<const v2u*>(p.bias + n);
      }
    }
#pragma unroll
  for (int i = 0; i < WMB; ++i) {
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float o[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = sam[i] * (sbv[j][q][r] * acc[i][j][4 * q + r]);
        if (p.bias) {
          o[0] += T::to_float((uint16_t)(bv[j][q].x & 0xffffu));
          o[1] += T::to_float((uint16_t)(bv[j][q].x >> 16));
          o[2] += T::to_float((uint16_t)(bv[j][q].y & 0xffffu));
          o[3] += T::to_float((uint16_t)(bv[j][q].y >> 16));
        }
        v2u ov;
        ov.x = (uint32_t)T::from_float(o[0]) | ((uint32_t)T::from_float(o[1]) << 16);
        ov.y = (uint32_t)T::from_float(o[2]) | ((uint32_t)T::from_float(o[3]) << 16);
        *reinterpret_cast<v2u*>(wave_lds + (lane & 31) * PITCH + (j * 32 + 8 * q + 4 * (lane >> 5)) * 2) = ov;
      }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();           // lanes exchange data through LDS; its operations run in program order
#pragma unroll
    for (int it = 0; it < 32 * CPR / 64; ++it) {
      const int idx = it * 64 + lane;
      const int row = idx / CPR, ch = idx % CPR;
      const v4u v = *reinterpret_cast<const v4u*>(wave_lds + row * PITCH + ch * 16);
      const int m = m0 + wm * 32 * WMB + i * 32 + row;
      const int n = n0 + wn * 32 * WNB + ch * 8;
      if (m < p.M && n < p.N) *reinterpret_cast<v4u*>(p.out + (int64_t)m * p.ldc + n) = v;
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
  }
}

// The tail of the multi-stage tile kernels: (split K) hand the partial tile over and let one wavefront sum
// (tile_handover.h), then the scaled epilogue.  `sl` = the workgroup's (tile, K part); `lds8` = at least
// NW * 32 * (WNB * 64 + 16) bytes of LDS that every wavefront of the workgroup is done with.
template <bool BF16_OUT, int WMB, int WNB, int NW>
__device__ inline void fp8_tile_tail(const Fp8MMParams& p, v16f (&acc)[WMB][WNB], uint8_t* lds8, const TileSlot& sl,
                                     int wave, int lane, int m0, int n0, int wm, int wn) {
  if (sl.nsplit > 1 && !handover_finish<WMB, WNB, NW>(p.c_tmp, p.counters, acc, sl, wave, lane)) return;

  if (((uintptr_t)p.out & 15) == 0)
    tile_epilogue_lds<BF16_OUT, WMB, WNB>(p, acc, m0, n0, wm, wn, lane, lds8 + wave * (32 * (WNB * 64 + 16)));
  else
    tile_epilogue<BF16_OUT, WMB, WNB>(p, acc, m0, n0, wm, wn, lane);
}

// ----------------------------------------------------------------------------- tile kernel
template <bool BF16_OUT, int WMB, int WNB>
__global__ __launch_bounds__(256) void fp8_mm_tile_kernel(const Fp8MMParams p) {
  constexpr int BM = 64 * WMB, BN = 64 * WNB;
  constexpr int A_CH = BM / 32, B_CH = BN / 32;   // 16-byte chunks per thread per step
  extern __shared__ __attribute__((aligned(16))) uint8_t lds8[];
  uint8_t* As = lds8;                         // [2][BM][PITCH]
  uint8_t* Bs = lds8 + 2 * BM * F8_PITCH;     // [2][BN][PITCH]

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  int bid = blockIdx.x;
  if (total % 8 == 0) bid = (bid & 7) * (total / 8) + (bid >> 3);   // one contiguous band of tiles per XCD
  const int tm = bid % tiles_m, tn = bid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  v4u areg[A_CH], breg[B_CH];
  auto load_g = [&](int step) {
    const int kb = step * F8_BK;
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, ch = c & 7;
      const int m = m0 + row, k = kb + ch * 16;
      v4u v = {0u, 0u, 0u, 0u};
      if (m < p.M && k < p.K) v = *reinterpret_cast<const v4u*>(p.a + (int64_t)m * p.lda + k);
      areg[i] = v;
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, ch = c & 7;
      const int n = n0 + row, k = kb + ch * 16;
      v4u v = {0u, 0u, 0u, 0u};
      if (n < p.N && k < p.K) v = *reinterpret_cast<const v4u*>(p.b + (int64_t)n * p.ldb + k);
      breg[i] = v;
    }
  };
  auto store_l = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + 256 * i;
      *reinterpret_cast<v4u*>(As + ((size_t)buf * BM + (c >> 3)) * F8_PITCH + (c & 7) * 16) = areg[i];
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const int c = tid + 256 * i;
      *reinterpret_cast<v4u*>(Bs + ((size_t)buf * BN + (c >> 3)) * F8_PITCH + (c & 7) * 16) = breg[i];
    }
  };

  v16f acc[WMB][WNB];
#pragma unroll
  for (int i = 0; i < WMB; ++i)
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int steps = (p.K + F8_BK - 1) / F8_BK;
  load_g(0);
  store_l(0);
  if (steps > 1) load_g(1);
  __syncthreads();

  for (int step = 0; step < steps; ++step) {
    const int cur = step & 1;
    if (step + 1 < steps) {
      store_l(cur ^ 1);
      if (step + 2 < steps) load_g(step + 2);
    }
    const uint8_t* Ab = As + ((size_t)cur * BM + wm * 32 * WMB + (lane & 31)) * F8_PITCH + (lane >> 5) * 32;
    const uint8_t* Bb = Bs + ((size_t)cur * BN + wn * 32 * WNB + (lane & 31)) * F8_PITCH + (lane >> 5) * 32;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      v8i af[WMB], bf[WNB];
#pragma unroll
      for (int i = 0; i < WMB; ++i) {
        const v4i lo = *reinterpret_cast<const v4i*>(Ab + (size_t)i * 32 * F8_PITCH + kk * 64);
        const v4i hi = *reinterpret_cast<const v4i*>(Ab + (size_t)i * 32 * F8_PITCH + kk * 64 + 16);
        af[i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
#pragma unroll
      for (int j = 0; j < WNB; ++j) {
        const v4i lo = *reinterpret_cast<const v4i*>(Bb + (size_t)j * 32 * F8_PITCH + kk * 64);
        const v4i hi = *reinterpret_cast<const v4i*>(Bb + (size_t)j * 32 * F8_PITCH + kk * 64 + 16);
        bf[j] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
#pragma unroll
      for (int i = 0; i < WMB; ++i)
#pragma unroll
        for (int j = 0; j < WNB; ++j) acc[i][j] = mfma_fp8_32(bf[j], af[i], acc[i][j]);   // rows = n, columns = m
    }
    __syncthreads();
  }

  tile_epilogue<BF16_OUT, WMB, WNB>(p, acc, m0, n0, wm, wn, lane);
}

// ----------------------------------------------------------------------------- tile kernel, direct-to-LDS variant
// Same tiling as fp8_mm_tile_kernel, but both operand tiles go global -> LDS with `buffer_load_dwordx4 ... lds`
// (no registers, no VALU, no ds_write): each wavefront instruction moves 8 rows x 128 bytes.  The LDS tile is
// unpadded [row][8 chunks of 16 B] with the chunk index XOR-ed by (row & 7), applied on the *global* side (the LDS
// side of such a load is fixed: lane L writes bytes 16L..16L+15), which keeps the 16-byte operand reads of 8
// consecutive rows on 8 different bank groups.  Rows beyond M / N fall outside the buffer descriptor and read as zero.
// Requires K % 128 == 0 (a partial last step would read the neighbouring row instead of zeros).
template <bool BF16_OUT, int WMB, int WNB>
__global__ __launch_bounds__(256) void fp8_mm_tile2_kernel(const Fp8MMParams p) {
  constexpr int BM = 64 * WMB, BN = 64 * WNB;
  constexpr int STAGE = (BM + BN) * 128;          // bytes per stage
  extern __shared__ __attribute__((aligned(16))) uint8_t lds8[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  int bid = blockIdx.x;
  if (total % 8 == 0) bid = (bid & 7) * (total / 8) + (bid >> 3);   // one contiguous band of tiles per XCD
  const int tm = bid % tiles_m, tn = bid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.a), 0, (int)((uint32_t)p.M * (uint32_t)p.lda), 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b), 0, (int)((uint32_t)p.N * (uint32_t)p.ldb), 0x00020000);
  const int lrow = lane >> 3, lchunk = (lane & 7) ^ lrow;
  const uint32_t voff_a = (uint32_t)lrow * (uint32_t)p.lda + (uint32_t)lchunk * 16u;
  const uint32_t voff_b = (uint32_t)lrow * (uint32_t)p.ldb + (uint32_t)lchunk * 16u;

  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto issue_loads = [&](int step, int buf) {
    uint8_t* Ab = lds8 + (size_t)buf * STAGE;
    uint8_t* Bb = Ab + BM * 128;
#pragma unroll
    for (int i = 0; i < BM / 32; ++i) {
      const int r0 = wave * (BM / 4) + i * 8;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(Ab + r0 * 128), 16, (int)voff_a,
                                               (int)((uint32_t)(m0 + r0) * (uint32_t)p.lda + (uint32_t)step * 128u), 0, 0);
    }
#pragma unroll
    for (int i = 0; i < BN / 32; ++i) {
      const int r0 = wave * (BN / 4) + i * 8;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(Bb + r0 * 128), 16, (int)voff_b,
                                               (int)((uint32_t)(n0 + r0) * (uint32_t)p.ldb + (uint32_t)step * 128u), 0, 0);
    }
  };

  v16f acc[WMB][WNB];
#pragma unroll
  for (int i = 0; i < WMB; ++i)
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // operand read offsets: row r = lane&31 of a 32-row block, 32 bytes = chunks (kk*4 + kh*2, +1), swizzled by (r & 7)
  const int r7 = lane & 7, kh = lane >> 5;
  uint32_t coff[2][2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int h = 0; h < 2; ++h) coff[kk][h] = (uint32_t)(((kk * 4 + kh * 2 + h) ^ r7) * 16);
  const uint32_t arow = (uint32_t)((wm * 32 * WMB + (lane & 31)) * 128);
  const uint32_t brow = (uint32_t)(BM * 128 + (wn * 32 * WNB + (lane & 31)) * 128);

  const int steps = p.K / F8_BK;
  issue_loads(0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int step = 0; step < steps; ++step) {
    const int cur = step & 1;
    if (step + 1 < steps) issue_loads(step + 1, cur ^ 1);
    const uint8_t* base = lds8 + (size_t)cur * STAGE;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      v8i af[WMB], bf[WNB];
#pragma unroll
      for (int i = 0; i < WMB; ++i) {
        const v4i lo = *reinterpret_cast<const v4i*>(base + arow + i * 4096 + coff[kk][0]);
        const v4i hi = *reinterpret_cast<const v4i*>(base + arow + i * 4096 + coff[kk][1]);
        af[i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
#pragma unroll
      for (int j = 0; j < WNB; ++j) {
        const v4i lo = *reinterpret_cast<const v4i*>(base + brow + j * 4096 + coff[kk][0]);
        const v4i hi = *reinterpret_cast<const v4i*>(base + brow + j * 4096 + coff[kk][1]);
        bf[j] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
#pragma unroll
      for (int i = 0; i < WMB; ++i)
#pragma unroll
        for (int j = 0; j < WNB; ++j) acc[i][j] = mfma_fp8_32(bf[j], af[i], acc[i][j]);   // rows = n, columns = m
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // next stage has landed in LDS
    __syncthreads();
  }

  tile_epilogue<BF16_OUT, WMB, WNB>(p, acc, m0, n0, wm, wn, lane);
}

// ----------------------------------------------------------------------------- tile kernel, multi-stage direct-to-LDS
// The kernel the M > 32 path normally uses.  Differences from fp8_mm_tile2_kernel:
//  * one MFMA k-slice (64 bytes of K) per stage, NST stages in a ring: the requests for step s+NST-1 go out at the
//    start of step s, so a tile has NST-2 full steps to arrive before anybody waits for it (with two stages of 128
//    bytes the wait at the end of every step saw most of the L2 latency);
//  * vector-memory operations retire in issue order, so "the tile of step s+1 has landed" is `vmcnt <= requests issued
//    after it`, a compile-time constant; the workgroup barrier is the bare instruction (a __syncthreads() carries a fence
//    that drains every outstanding load);
//  * LDS rows are 64 bytes; four rows form one 256-byte line of 16 chunks (chunk index (row & 3) * 4 + c) and the chunk
//    index is XOR-ed with (row >> 2) & 3.  The LDS has 64 banks (256 bytes per cycle): 16 lanes reading 16 consecutive
//    rows at the same k chunk touch 16 different 16-byte bank groups;
//  * WAVES_M x WAVES_N wavefronts; tiles are handed out in bands of 4 tile rows inside each XCD's contiguous range so
//    that the tiles resident on one XCD share activation rows and weight columns in its L2.
// Requires K % 64 == 0 (a partial last step would read the neighbouring row instead of zeros) and M*lda, N*ldb < 2^32.
template <bool BF16_OUT, int BM, int BN, int WAVES_M, int WAVES_N, int NST, int KS = 1, int PP = 0>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void fp8_mm_tile3_kernel(const Fp8MMParams p) {
  // A step is KS k-slices of 64 bytes (KS = 2 for the small tiles, whose steps are otherwise shorter than the barrier
  // and the LDS round trip that every step pays); a stage holds the KS slices of one step, each as [A tile | B tile].
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;
  constexpr int WMB = TM / 32, WNB = TN / 32;
  constexpr int A_ST = BM * 64, B_ST = BN * 64, SLICE = A_ST + B_ST, STAGE = KS * SLICE;
  constexpr int A_LD = BM / (16 * NW), B_LD = BN / (16 * NW);     // DMA instructions per wavefront and slice (16 rows each)
  constexpr int LPW = KS * (A_LD + B_LD);
  static_assert(A_LD >= 1 && B_LD >= 1, "tile too small for this many wavefronts");
  static_assert((NST - 2) * LPW <= 63, "wait counter range");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds8[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  const int tiles_m = (p.M + BM - 1) / BM + p.m_tiles_extra, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  const TileSlot sl = tile_slot(total, p.SK, p.tail_first);          // one contiguous range of tile positions per XCD
  const int t = sl.pos;
  constexpr int GM = 4;                                              // band height in tiles (2 .. 16 measured: 4 is 1-2 % ahead of 8)
  const int band = t / (GM * tiles_n);
  const int first_m = band * GM;
  const int gsz = min(tiles_m - first_m, GM);
  const int tin = t - band * GM * tiles_n;
  const int tm = first_m + tin % gsz, tn = tin / gsz;
  const int m0 = tm * BM, n0 = tn * BN;

  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.a), 0, (int)((uint32_t)p.M * (uint32_t)p.lda), 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b), 0, (int)((uint32_t)p.N * (uint32_t)p.ldb), 0x00020000);
  // DMA instruction: 16 rows x 64 bytes = four 256-byte lines; lane l lands in slot l: line j = r0/4 + (l >> 4), swizzled
  // chunk l & 15 -> c16 = (l & 15) ^ (j & 3), row = 4j + (c16 >> 2), chunk = c16 & 3.  r0 is a multiple of 16, so j & 3 = l >> 4.
  const int c16 = (lane & 15) ^ (lane >> 4);
  const int lrow = 4 * (lane >> 4) + (c16 >> 2);
  const uint32_t voff_a = (uint32_t)lrow * (uint32_t)p.lda + (uint32_t)(c16 & 3) * 16u;
  const uint32_t voff_b = (uint32_t)lrow * (uint32_t)p.ldb + (uint32_t)(c16 & 3) * 16u;

  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  // K may be split over workgroups: this one covers the steps [s_lo, s_hi)
  const int all_steps = p.K / (64 * KS);
  const int s_lo = (int)(((int64_t)all_steps * sl.split) / sl.nsplit), s_hi = (int)(((int64_t)all_steps * (sl.split + 1)) / sl.nsplit);
  const int steps = s_hi - s_lo;
  // Few tile rows (M at most 4 tiles high) on a device that the tiles do not fill: the tiles of one column would read
  // the same weight rows at the same time, which leaves only (ring depth x 64 KS) bytes per weight row in flight --
  // with cold weights the kernel then runs at a fraction of the memory bandwidth.  Tile row tm starts its K loop
  // tm / tiles_m of the way into its range and wraps around: the rows are read at tiles_m places at once, and the later
  // readers find them in the L2 (4096 x 4096 at M = 256, cold: 24.4 -> 18.3 us).
  // rotate_k = 2, one or two tile rows on a wide layer: every workgroup reads the same activation rows, and with K a power
  // of two all of them ask the same few L2 channels for the same lines at the same time.  Tile column tn starts tn / tiles_n
  // of the way into K instead (4096 x 28672 at M = 72 .. 256, cold: 33.9 .. 45.4 -> 31.1 .. 43.6 us; no change on K = 3584 or
  // 5120; with 16 tile rows it costs 3-9 %: the tiles of one column then no longer read their weights together).
  const int rot = p.rotate_k == 1 ? (tm * steps) / tiles_m : (p.rotate_k == 2 ? (tn * steps) / tiles_n : 0);
  auto issue_loads = [&](int step_in, int stage) {
    int step = step_in - s_lo + rot;
    if (step >= steps) step -= steps;
    step += s_lo;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint8_t* Ab = lds8 + (size_t)stage * STAGE + ks * SLICE;
      uint8_t* Bb = Ab + A_ST;
      const uint32_t koff = (uint32_t)(step * KS + ks) * 64u;
#pragma unroll
      for (int i = 0; i < A_LD; ++i) {
        const int r0 = (wave * A_LD + i) * 16;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(Ab + r0 * 64), 16, (int)voff_a,
                                                 (int)((uint32_t)(m0 + r0) * (uint32_t)p.lda + koff), 0, 0);
      }
#pragma unroll
      for (int i = 0; i < B_LD; ++i) {
        const int r0 = (wave * B_LD + i) * 16;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(Bb + r0 * 64), 16, (int)voff_b,
                                                 (int)((uint32_t)(n0 + r0) * (uint32_t)p.ldb + koff), 0, 0);
      }
    }
  };

  v16f acc[WMB][WNB];
#pragma unroll
  for (int i = 0; i < WMB; ++i)
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // operand reads: row = lane & 31 of a 32-row block (blocks start at multiples of 32 rows), the lane's 32 bytes are
  // chunks 2*kh and 2*kh+1 (kh = lane >> 5)
  const int kh = lane >> 5;
  uint32_t coff[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    coff[h] = (uint32_t)(((lane & 31) >> 2) * 256 + ((((lane & 3) * 4 + kh * 2 + h) ^ ((lane >> 2) & 3)) * 16));
  const uint32_t arow = (uint32_t)(wm * TM * 64);
  const uint32_t brow = (uint32_t)(A_ST + wn * TN * 64);

  // (Reading the fragments of step s+1 during the MFMAs of step s -- one more stage of slack, double-buffered weight
  // fragments -- was measured 5% slower than reading them at the start of their own step, and is not done.)
  auto compute = [&](int stage) {
#pragma unroll
   for (int ks = 0; ks < KS; ++ks) {
    const uint8_t* base = lds8 + (size_t)stage * STAGE + ks * SLICE;
    v8i af[WMB], bf[WNB];
#pragma unroll
    for (int j = 0; j < WNB; ++j) {
      const v4i lo = *reinterpret_cast<const v4i*>(base + brow + j * 2048 + coff[0]);
      const v4i hi = *reinterpret_cast<const v4i*>(base + brow + j * 2048 + coff[1]);
      bf[j] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
#pragma unroll
    for (int i = 0; i < WMB; ++i) {
      const v4i lo = *reinterpret_cast<const v4i*>(base + arow + i * 2048 + coff[0]);
      const v4i hi = *reinterpret_cast<const v4i*>(base + arow + i * 2048 + coff[1]);
      af[i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
#pragma unroll
    for (int i = 0; i < WMB; ++i)
#pragma unroll
      for (int j = 0; j < WNB; ++j) acc[i][j] = mfma_fp8_32(bf[j], af[i], acc[i][j]);   // rows = n, columns = m
   }
  };
  // end of a step: LDS reads of this wavefront done, requests older than the newest `n` landed, then the bare barrier
  auto sync_step = [&](auto n_c) {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(decltype(n_c)::value) : "memory");
  };
  using WAIT_STEADY = std::integral_constant<int, (NST - 2) * LPW>;
  using WAIT_NONE = std::integral_constant<int, 0>;

  // Invariant at the start of step s: the tile of step s complete in LDS, the tiles of steps s+1 .. s+NST-2 requested,
  // stage (s-1) % NST free.  The requests of step s+NST-1 go out first thing in step s.
  if (PP != 0 && steps >= NST) {
    // Alternating phases: the two wavefronts that share a SIMD run half a step apart, so that one reads its fragments
    // (and requests tiles) while the other one issues its MFMAs.  A step is [requests, fragment reads, wait] barrier
    // [MFMAs] barrier; the late half of the workgroup passes one extra barrier first and skips its last one, so every
    // wavefront passes the same number.  The tile of step s+1 must have landed at the END OF THE READ PHASE of step s
    // (the early half reads it two barriers later, the late half three).
    auto read_frags = [&](int stage, v8i (&af)[KS][WMB], v8i (&bf)[KS][WNB]) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const uint8_t* base = lds8 + (size_t)stage * STAGE + ks * SLICE;
#pragma unroll
        for (int j = 0; j < WNB; ++j) {
          const v4i lo = *reinterpret_cast<const v4i*>(base + brow + j * 2048 + coff[0]);
          const v4i hi = *reinterpret_cast<const v4i*>(base + brow + j * 2048 + coff[1]);
          bf[ks][j] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
#pragma unroll
        for (int i = 0; i < WMB; ++i) {
          const v4i lo = *reinterpret_cast<const v4i*>(base + arow + i * 2048 + coff[0]);
          const v4i hi = *reinterpret_cast<const v4i*>(base + arow + i * 2048 + coff[1]);
          af[ks][i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
      }
    };
    auto mfmas = [&](v8i (&af)[KS][WMB], v8i (&bf)[KS][WNB]) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int i = 0; i < WMB; ++i)
#pragma unroll
          for (int j = 0; j < WNB; ++j) acc[i][j] = mfma_fp8_32(bf[ks][j], af[ks][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    };
    auto bare_barrier = [&]() { asm volatile("s_barrier" ::: "memory"); };
    const bool late = wave >= NW / 2;     // wavefronts w and w + 4 share a SIMD (the other pairing measured 10-25 % slower)
    v8i af[KS][WMB], bf[KS][WNB];
#pragma unroll
    for (int s0 = 0; s0 < NST - 1; ++s0) issue_loads(s_lo + s0, s0);
    sync_step(WAIT_STEADY{});           // tile 0 landed
    if (late) bare_barrier();
    int cur = 0, dst = NST - 1;
    int step = 0;
    for (; step + NST - 1 < steps; ++step) {
      issue_loads(s_lo + step + NST - 1, dst);
      read_frags(cur, af, bf);
      sync_step(WAIT_STEADY{});
      mfmas(af, bf);
      bare_barrier();
      cur = cur + 1 == NST ? 0 : cur + 1;
      dst = dst + 1 == NST ? 0 : dst + 1;
    }
    for (; step < steps; ++step) {      // nothing left to request: drain
      read_frags(cur, af, bf);
      sync_step(WAIT_NONE{});
      mfmas(af, bf);
      if (!(late && step == steps - 1)) bare_barrier();
      cur = cur + 1 == NST ? 0 : cur + 1;
    }
  } else if (steps >= NST) {
#pragma unroll
    for (int s0 = 0; s0 < NST - 1; ++s0) issue_loads(s_lo + s0, s0);
    sync_step(WAIT_STEADY{});           // tile 0 landed
    int cur = 0, dst = NST - 1;
    int step = 0;
    for (; step + NST - 1 < steps; ++step) {
      issue_loads(s_lo + step + NST - 1, dst);
      compute(cur);
      sync_step(WAIT_STEADY{});
      cur = cur + 1 == NST ? 0 : cur + 1;
      dst = dst + 1 == NST ? 0 : dst + 1;
    }
    for (; step < steps; ++step) {      // nothing left to request: drain
      compute(cur);
      sync_step(WAIT_NONE{});
      cur = cur + 1 == NST ? 0 : cur + 1;
    }
  } else {
    // short K: no ring, one tile at a time
    for (int step = 0; step < steps; ++step) {
      issue_loads(s_lo + step, 0);
      sync_step(WAIT_NONE{});
      compute(0);
      sync_step(WAIT_NONE{});
    }
  }

  static_assert(NST * STAGE >= NW * 32 * (WNB * 64 + 16), "operand ring too small for the epilogue staging");
  if (m0 >= p.M) return;      // a tile row past M (m_tiles_extra): nothing to hand over or store
  fp8_tile_tail<BF16_OUT, WMB, WNB, NW>(p, acc, lds8, sl, wave, lane, m0, n0, wm, wn);
}

// ----------------------------------------------------------------------------- stream kernel (M <= 32, narrow layers M <= 64)
// blockDim = (64, WK).  Wavefront w owns K steps [w*KS, (w+1)*KS) of 128 bytes; activations of that slab live in
// registers for the whole kernel; the workgroup walks a contiguous range of 16-row weight tiles.
template <bool BF16_OUT, int KS, int MB, bool HALVES = false, bool PF = true>
__global__ __launch_bounds__(512) void fp8_mm_stream_kernel(const Fp8MMParams p, int WK) {
  using T = F16Traits<BF16_OUT>;
  extern __shared__ v4f red[];   // [2][WK][MB][64]
  const int lane = threadIdx.x, w = threadIdx.y;
  const int q = lane >> 4, r16 = lane & 15;
  // HALVES (gridDim.y = 2): the K range is split over two workgroups (the second starts where the slabs of the first
  // end); their partial tiles are summed by whichever arrives last (see the hand-over below).  A template parameter,
  // because the extra live values cost the other instances registers they do not have (14 steps: 12 -> 260 bytes spilled).
  const int kbase = ((HALVES ? (int)blockIdx.y * WK : 0) + w) * KS * 128 + q * 32;

  // Operand loads go through buffer descriptors (the host checks that both operands end below 2 GiB): a 16-byte piece
  // past K or past the last row gets an offset beyond the descriptor's extent and arrives as zeros -- one compare and
  // one select per load instead of a branch and eight zeroed registers.
  constexpr uint32_t OOB = 0x80000000u;
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.a), 0, (int)p.a_extent, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b), 0, (int)p.b_extent, 0x00020000);
  v8i breg[KS][MB];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = mb * 16 + r16;
      const int k = kbase + s * 128;
      const uint32_t base = (uint32_t)m * (uint32_t)p.lda + (uint32_t)k;
      const uint32_t o_lo = (m < p.M && k < p.K) ? base : OOB, o_hi = (m < p.M && k + 16 < p.K) ? base + 16u : OOB;
      const v4i lo = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, (int)o_lo, 0, 0));
      const v4i hi = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, (int)o_hi, 0, 0));
      breg[s][mb] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  }

  const int NT = p.N / 16;
  const int bx = blockIdx.x;
  const int nt0 = bx * p.nt_base + (bx < p.nt_rem ? bx : p.nt_rem);
  const int nt1 = nt0 + p.nt_base + (bx < p.nt_rem ? 1 : 0);

  v4i wlo[KS], whi[KS];
  // `live` = false requests nothing (offsets beyond the extent): the request for the tile after the last one stays in
  // the instruction stream, so that the count of loads in flight -- which the waits are derived from -- is the same on
  // every path (behind a branch the compiler assumes the shorter path and waits for the next tile's loads as well).
  auto issue = [&](int nt, int s, bool live) {
    const int k = kbase + s * 128;
    const uint32_t base = (uint32_t)(nt * 16 + r16) * (uint32_t)p.ldb + (uint32_t)k;
    const uint32_t o_lo = (live && k < p.K) ? base : OOB, o_hi = (live && k + 16 < p.K) ? base + 16u : OOB;
    wlo[s] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rb, (int)o_lo, 0, 2));     // 2: streamed once
    whi[s] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rb, (int)o_hi, 0, 2));
  };
#pragma unroll
  for (int s = 0; s < KS; ++s) issue(nt0, s, nt0 < nt1);

  // Epilogue operands are requested ahead of their use (a load issued after the reduction would stall the reducing
  // wavefront, and through the next barrier the whole workgroup, for a memory round trip per n-tile): the activation
  // scales once per kernel, the weight scales and the bias of an n-tile before its MFMAs.  With 14 steps per wavefront
  // there are no registers to spare for that: there they are requested after the tile's last MFMA (14336 x 4096 at
  // M = 1 / 16: 16.5 / 20.8 -> 15.7 / 19.6 us).  Requesting the first tile's weights before the activations was slower
  // on every shape (3-5 %, and 40 % with 14 steps, where it changes what the compiler spills).
  constexpr bool AHEAD = KS < 14;
  const bool reducer_wave = WK > 1 ? w < MB : true;
  float sam_mb[MB];
  if constexpr (AHEAD) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = mb * 16 + r16;
      sam_mb[mb] = (reducer_wave && m < p.M) ? p.sa[p.sa_per_row ? m : 0] : 0.f;
    }
  }

  int parity = 0;
  // One n-tile.  PF: request the next tile's weights behind each step's MFMAs.  Launches in which every workgroup has a
  // single tile use the instance without those requests (they would be 2 KS loads that fetch nothing but still pass
  // through the load path: 14336 x 4096 at M = 1 / 16 15.4 / 19.2 -> 16.0 / 20.2 us); as a run-time condition the compiler
  // would derive the waits of the multi-tile case from the shorter path and wait for the next tile's loads too, and
  // both variants in one kernel cost registers (spills with 8 steps and two m-blocks).
  auto do_tile = [&](int nt) {
    v4f acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = v4f{0.f, 0.f, 0.f, 0.f};
    float sb_r[4] = {0.f, 0.f, 0.f, 0.f};
    uint16_t bias_r[4] = {0, 0, 0, 0};
    if constexpr (AHEAD) {
      if (reducer_wave) {
        const int n = nt * 16 + q * 4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          sb_r[r] = p.sb[p.sb_per_col ? n + r : 0];
          if (p.bias) bias_r[r] = p.bias[n + r];
        }
      }
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const v8i aop = v8i{wlo[s].x, wlo[s].y, wlo[s].z, wlo[s].w, whi[s].x, whi[s].y, whi[s].z, whi[s].w};
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb] = mfma_fp8_16(aop, breg[s][mb], acc[mb]);
      // the step's registers are free once its MFMAs have issued: request the next tile's step into them right away
      // (the fence keeps the compiler from collecting these requests behind the tile's last MFMA)
      if constexpr (PF) {
        issue(nt + 1, s, nt + 1 < nt1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    if constexpr (!AHEAD) {
      // registers are full until the last MFMA of the tile: request the epilogue operands now, across the reduction
      static_assert(AHEAD || MB == 1, "14 steps per wavefront only with one m-block");
      if (reducer_wave) {
        const int n = nt * 16 + q * 4;
        sam_mb[0] = r16 < p.M ? p.sa[p.sa_per_row ? r16 : 0] : 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          sb_r[r] = p.sb[p.sb_per_col ? n + r : 0];
          if (p.bias) bias_r[r] = p.bias[n + r];
        }
      }
    }

    v4f tot = v4f{0.f, 0.f, 0.f, 0.f};
    bool reducer = w < MB;
    if (WK > 1) {
      v4f* buf = red + (size_t)parity * WK * MB * 64;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) buf[(w * MB + mb) * 64 + lane] = acc[mb];
      __syncthreads();
      if (reducer)
        for (int ww = 0; ww < WK; ++ww) tot += buf[(ww * MB + w) * 64 + lane];
      parity ^= 1;
    } else {
      reducer = true;
    }
    if (HALVES && reducer) {
      // Hand-over as in the tile kernel: the partial tile goes out in device-scope 16-byte stores, one arrival counter
      // per (n-tile, m-block); the workgroup that arrives last adds the parts in the order of the K halves and returns the
      // counter to zero.  (WK > 1 always here: the host splits only a long K.)
      constexpr int SC1 = 16;
      const uint32_t units = (uint32_t)NT * (uint32_t)MB;
      const uint32_t unit = (uint32_t)nt * (uint32_t)MB + (uint32_t)w;
      const __amdgpu_buffer_rsrc_t rt =
          __builtin_amdgcn_make_buffer_rsrc(p.c_tmp, 0, (int)(units * gridDim.y * 1024u), 0x00020000);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, tot), rt, lane * 16,
                                             (int)((blockIdx.y * units + unit) * 1024u), SC1);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // partial tile acknowledged before the counter moves
      int32_t* ctr = p.counters + unit;
      int old = 0;
      if (lane == 0) old = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      old = __builtin_amdgcn_readfirstlane(old);      // lane 0 holds it; a scalar keeps what depends on it scalar
      if (old != (int)gridDim.y - 1) {
        reducer = false;
      } else {
        v4f sum = {0.f, 0.f, 0.f, 0.f};
        for (uint32_t h = 0; h < gridDim.y; ++h) {
          const v4u r = __builtin_amdgcn_raw_buffer_load_b128(rt, lane * 16, (int)((h * units + unit) * 1024u), SC1);
          sum += __builtin_bit_cast(v4f, r);
        }
        tot = sum;
        if (lane == 0) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (reducer) {
      const int mb_lo = (WK > 1) ? w : 0, mb_hi = (WK > 1) ? w + 1 : MB;
      auto emit = [&](int mb, float sam, const float* sbv, const uint16_t* bsv) {
        const v4f val = (WK > 1) ? tot : acc[mb];
        const int m = mb * 16 + r16;
        if (m < p.M) {
#pragma clang fp contract(off)      // sa * (sb * acc), then + bias: two fp32 roundings, like the tile kernels
          const int n = nt * 16 + q * 4;
          float o[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            o[r] = sam * (sbv[r] * val[r]);
            if (p.bias) o[r] += T::to_float(bsv[r]);
          }
          v2u ov;
          ov.x = (uint32_t)T::from_float(o[0]) | ((uint32_t)T::from_float(o[1]) << 16);
          ov.y = (uint32_t)T::from_float(o[2]) | ((uint32_t)T::from_float(o[3]) << 16);
          *reinterpret_cast<v2u*>(p.out + (int64_t)m * p.ldc + n) = ov;
        }
      };
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)       // unrolled: sam_mb stays in registers
        if (mb >= mb_lo && mb < mb_hi) emit(mb, sam_mb[mb], sb_r, bias_r);
    }
  };
  if constexpr (PF) {
    for (int nt = nt0; nt < nt1; ++nt) do_tile(nt);
  } else {
    if (nt0 < nt1) do_tile(nt0);       // the launcher picks this instance only for one tile per workgroup
  }
}

// ----------------------------------------------------------------------------- stream kernel, weights through LDS
// The stream kernel above fetches the weights in the MFMA operand layout: every load instruction takes 64-byte pieces
// of 16 rows, half a cache line each.  Measured on bare reads of a 4096 x 28672 byte matrix with cold lines, that
// pattern reaches 4.2-5.3 TB/s where instructions that read whole lines reach 5.3-5.9 TB/s.  Here every load
// instruction is a direct-to-LDS load of 4 rows x 256 contiguous bytes into a ring that belongs to the wavefront alone
// (no barrier: the wavefront waits on its own load counter), and the operands are read back from LDS, 16-byte chunks
// XOR-swizzled by the row so that the 16 rows of an operand read hit 16 different bank groups.
//  * blockDim = (64, WK).  Wavefront w owns K steps [w*KS, (w+1)*KS) of 128 bytes; its activations live in registers;
//    the workgroup walks a contiguous range of 16-row n-tiles; per n-tile the wavefronts reduce through LDS as above.
//  * A stage is two steps (16 rows x 256 bytes = 4 KiB, four load instructions); the ring holds NSR stages, and the
//    stage NSR ahead -- of this n-tile or the next -- is requested as soon as a stage's operands have been read.
template <bool BF16_OUT, int KS, int MB, int NSR>
__global__ __launch_bounds__(512) void fp8_mm_stream2_kernel(const Fp8MMParams p, int WK) {
  using T = F16Traits<BF16_OUT>;
  constexpr int NS = KS / 2;                       // stages per n-tile
  static_assert(KS % 2 == 0 && NS % NSR == 0, "whole stages, ring slots fixed at compile time");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds8[];
  const int lane = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.y);
  const int q = lane >> 4, r16 = lane & 15;
  const int kw = w * KS * 128;                     // first byte of K of this wavefront
  const int kbase = kw + q * 32;
  uint8_t* const ring = lds8 + (size_t)w * NSR * 4096;
  v4f* const red = reinterpret_cast<v4f*>(lds8 + (size_t)WK * NSR * 4096);      // [2][WK][MB][64]

  constexpr uint32_t OOB = 0x80000000u;
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.a), 0, (int)p.a_extent, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b), 0, (int)p.b_extent, 0x00020000);
  v8i breg[KS][MB];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = mb * 16 + r16;
      const int k = kbase + s * 128;
      const uint32_t base = (uint32_t)m * (uint32_t)p.lda + (uint32_t)k;
      const uint32_t o_lo = (m < p.M && k < p.K) ? base : OOB, o_hi = (m < p.M && k + 16 < p.K) ? base + 16u : OOB;
      const v4i lo = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, (int)o_lo, 0, 0));
      const v4i hi = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, (int)o_hi, 0, 0));
      breg[s][mb] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  }

  const int NT = p.N / 16;
  const int bx = blockIdx.x;
  const int nt0 = bx * p.nt_base + (bx < p.nt_rem ? bx : p.nt_rem);
  const int nt1 = nt0 + p.nt_base + (bx < p.nt_rem ? 1 : 0);

  // Load instruction i of a stage fills LDS bytes [1024 i, 1024 i + 1024) = rows 4i .. 4i+3; lane l lands at row
  // 4i + l/16, position l & 15, which holds chunk (l & 15) ^ row of the row's 256 bytes.
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  uint32_t voffb[4], kchunk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 4 * i + (lane >> 4);
    kchunk[i] = (uint32_t)(((lane & 15) ^ row) * 16);
    voffb[i] = (uint32_t)row * (uint32_t)p.ldb + kchunk[i];
  }
  // `live` = false requests nothing (offsets beyond the extent) but keeps the count of loads in flight the same
  auto issue_stage = [&](int nt, int st, int slot, bool live) {
    const int k0 = kw + st * 256;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t vo = (live && k0 + (int)kchunk[i] < p.K) ? voffb[i] : OOB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(ring + slot * 4096 + i * 1024), 16, (int)vo,
                                               (int)((uint32_t)(nt * 16) * (uint32_t)p.ldb + (uint32_t)k0), 0, 2);
    }
  };
#pragma unroll
  for (int st = 0; st < NSR; ++st) issue_stage(nt0, st, st, nt0 < nt1);

  const bool reducer_wave = WK > 1 ? w < MB : true;
  float sam_mb[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + r16;
    sam_mb[mb] = (reducer_wave && m < p.M) ? p.sa[p.sa_per_row ? m : 0] : 0.f;
  }

  int parity = 0;
  for (int nt = nt0; nt < nt1; ++nt) {
    v4f acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = v4f{0.f, 0.f, 0.f, 0.f};
    float sb_r[4] = {0.f, 0.f, 0.f, 0.f};
    uint16_t bias_r[4] = {0, 0, 0, 0};
    if (reducer_wave) {
      const int n = nt * 16 + q * 4;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sb_r[r] = p.sb[p.sb_per_col ? n + r : 0];
        if (p.bias) bias_r[r] = p.bias[n + r];
      }
    }
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      constexpr int W_AFTER = (NSR - 1) * 4;      // load instructions requested after this stage's (any others in flight only make the wait stricter)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(W_AFTER) : "memory");
      const int slot = st % NSR;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const int c0 = 8 * s2 + 2 * q;
        const v4i lo = *reinterpret_cast<const v4i*>(ring + slot * 4096 + r16 * 256 + ((c0 ^ r16) << 4));
        const v4i hi = *reinterpret_cast<const v4i*>(ring + slot * 4096 + r16 * 256 + (((c0 + 1) ^ r16) << 4));
        const v8i aop = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb] = mfma_fp8_16(aop, breg[2 * st + s2][mb], acc[mb]);
      }
      // the slot is free once its operands are in registers: request the stage NSR ahead into it
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (st + NSR < NS) issue_stage(nt, st + NSR, slot, true);
      else issue_stage(nt + 1, st + NSR - NS, slot, nt + 1 < nt1);
    }

    v4f tot = v4f{0.f, 0.f, 0.f, 0.f};
    bool reducer = w < MB;
    if (WK > 1) {
      v4f* buf = red + (size_t)parity * WK * MB * 64;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) buf[(w * MB + mb) * 64 + lane] = acc[mb];
      // the partial tiles are written; the bare barrier leaves the next tile's weight requests in flight (a
      // __syncthreads() would wait for every direct-to-LDS load)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (reducer)
        for (int ww = 0; ww < WK; ++ww) tot += buf[(ww * MB + w) * 64 + lane];
      parity ^= 1;
    } else {
      reducer = true;
    }
    if (reducer) {
      const int mb_lo = (WK > 1) ? w : 0, mb_hi = (WK > 1) ? w + 1 : MB;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        if (mb < mb_lo || mb >= mb_hi) continue;
        const v4f val = (WK > 1) ? tot : acc[mb];
        const int m = mb * 16 + r16;
        if (m < p.M) {
#pragma clang fp contract(off)      // sa * (sb * acc), then + bias: two fp32 roundings, like the tile kernels
          const int n = nt * 16 + q * 4;
          float o[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            o[r] = sam_mb[mb] * (sb_r[r] * val[r]);
            if (p.bias) o[r] += T::to_float(bias_r[r]);
          }
          v2u ov;
          ov.x = (uint32_t)T::from_float(o[0]) | ((uint32_t)T::from_float(o[1]) << 16);
          ov.y = (uint32_t)T::from_float(o[2]) | ((uint32_t)T::from_float(o[3]) << 16);
          *reinterpret_cast<v2u*>(p.out + (int64_t)m * p.ldc + n) = ov;
        }
      }
    }
  }
}

// ----------------------------------------------------------------------------- host side

// Overrides for tests and benchmarks come through tuning() (all zero = automatic): fp8_path 1 stream / 2 tile,
// fp8_tile_impl 1 = register-staged tile kernel, fp8_tile_cfg = fixed multi-stage tile shape (-1: two-stage kernel),
// fp8_split = K split of the tile kernel, fp8_gx = stream-kernel grid, fp8_stream_split -1 = no two-halves stream route.

template <bool BF16_OUT, int WMB, int WNB>
static int launch_tile(const Fp8MMParams& p, hipStream_t s) {
  constexpr int BM = 64 * WMB, BN = 64 * WNB;
  const size_t lds = (size_t)2 * (BM + BN) * F8_PITCH;
  auto kern = fp8_mm_tile_kernel<BF16_OUT, WMB, WNB>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (const int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "fp8_scaled_mm"); rc != VAQ_OK) return rc;
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(256), lds, s, p);
  return VAQ_OK;
}

template <bool BF16_OUT, int WMB, int WNB>
static int launch_tile2(const Fp8MMParams& p, hipStream_t s) {
  constexpr int BM = 64 * WMB, BN = 64 * WNB;
  const size_t lds = (size_t)2 * (BM + BN) * 128;
  auto kern = fp8_mm_tile2_kernel<BF16_OUT, WMB, WNB>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (const int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "fp8_scaled_mm"); rc != VAQ_OK) return rc;
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(256), lds, s, p);
  return VAQ_OK;
}

template <bool BF16_OUT, int BM, int BN, int WAVES_M, int WAVES_N, int NST, int KS = 1, int PP = 0>
static int launch_tile3(const Fp8MMParams& p, hipStream_t s) {
  const size_t lds = (size_t)NST * KS * (BM + BN) * 64;
  auto kern = fp8_mm_tile3_kernel<BF16_OUT, BM, BN, WAVES_M, WAVES_N, NST, KS, PP>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (const int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "fp8_scaled_mm"); rc != VAQ_OK) return rc;
  const int tiles = ((p.M + BM - 1) / BM + p.m_tiles_extra) * ((p.N + BN - 1) / BN);
  const dim3 grid = p.tail_first > 0 ? dim3(p.tail_first + (tiles - p.tail_first) * p.SK) : dim3(tiles, p.SK);
  hipLaunchKernelGGL(kern, grid, dim3(WAVES_M * WAVES_N * 64), lds, s, p);
  return VAQ_OK;
}

struct Fp8TilePlan {
  int cfg, sk, bm, bn, nw;
  int64_t tiles;
  int64_t tail_first = 0;      // > 0: only the tiles from this position on are split (tile_handover.h)
  int64_t extra_tiles = 0;     // split K: the tiles of a tile row past M that runs beside the real ones (see m_tiles_extra in dispatch_tile)
  // scratch of the K split: partial tiles and arrival counters of the tiles that are split
  int64_t split_tiles() const { return sk > 1 ? tiles + extra_tiles - tail_first : 0; }
  int64_t tmp_bytes() const { return (int64_t)sk * split_tiles() * bm * bn * 4; }
  int64_t counter_ints() const { return split_tiles() * nw; }
};

// Tile shape and K split of the multi-stage kernel.  K is split when the output tiles alone leave compute units idle,
// at most 8 ways; the rules for large and small tiles are below, each measured with cold weights.
static Fp8TilePlan plan_tile3(int M, int N, int K) {
  const int cus = num_cus_current_device();
  auto tiles = [&](int bm, int bn) { return (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  Fp8TilePlan pl;
  pl.cfg = tuning().fp8_tile_cfg;
  // the largest tile shape that fills 70 % of the compute units (measured on the Llama shapes, M = 256 .. 4096: a
  // partly filled device of large tiles beats a full one of small tiles by 25-40 %); for 128 x 128 also when two
  // parts of a long K get it there (14336 x 4096 at M = 512, cold, 73 -> 62 us)
  // ... and for 256 x 256 when two parts of a very long K do (14336 x 4096 at M = 1536 / 2048, cold: 139 / 145 -> 116 / 130 us;
  // 4096 x 4096 at M = 2048 in two parts: 45 -> 66 us)
  // (256 x 256 from 55 % of the compute units on, 50 % in two parts of a long K: 4096 x 6144 at M = 1408 .. 1792 70 ->
  // 49 .. 55 us, 4096 x 4096 at M = 2304 / 2560 70 -> 54 us, 14336 x 4096 at M = 1024 / 1280 89 / 132 -> 79 / 105 us;
  // at 47-50 % on a short K the smaller tiles win, 4096 x 4096 at M = 2048 45 against 53 us)
  const int parts128 = K / 64 >= 128 ? 2 : 1;
  const int parts256 = K / 64 >= 160 ? 2 : 1;      // (11008 x 4096 at M = 2048 in two parts: 115 -> 98 us)
  // 128 x 128 also from half a device's worth of tiles on a long K (14336 x 4096 at M = 160 / 224: 42 -> 35 us), and
  // wherever the 64 x 128 tiles (one workgroup per compute unit) would need a second round and these do not
  // (4096 x 6144 at M = 384: 39 -> 27 us; 4096 x 4096 at M = 640: 38.5 -> 28 us)
  const bool take128 = tiles(128, 128) * parts128 * 10 >= cus * (parts128 == 2 ? 5 : 7) ||
                       (tiles(64, 128) > cus && tiles(128, 128) <= cus);
  // ... and when the K parts that 256 x 256 tiles get, counted only down to 40 steps, bring them to 60 % of the compute units
  // and M fills 80 % of their rows (cold: 18944 x 3584 at M = 640 .. 1024, 42 / 56 tiles in 4 parts, 94 .. 101 -> 76 .. 84 us;
  // 8192 x 8192 at M = 640 / 768, 96 tiles in 2 parts, 84 / 81 -> 62 / 70 us; 14336 x 4096 at M = 640 / 768 79 -> 64 / 71 us;
  // parts of 32 steps lose 5 %, 8192 x 8192 at M = 512; rows filled to 75 % lose 15 %, 13824 x 5120 at M = 384)
  auto long_k_256 = [&]() {
    const int64_t t = tiles(256, 256);
    if (t >= cus || t < 1) return false;
    // the parts these tiles would get below, of those only parts of at least 40 steps
    const int min_steps = t * 4 <= cus ? 32 : 64;
    int sk = (int)((int64_t)cus / t);
    if (sk > 8) sk = 8;
    if (sk > K / 64 / min_steps) sk = K / 64 / min_steps;
    if (sk < 1) sk = 1;
    while (sk & (sk - 1)) --sk;
    while (sk > 1 && K / 64 / sk < 40) sk /= 2;
    // (rows filled to 80 %; to 70 % from three tile rows on, where the poorly filled row is a third of the tiles or less:
    // 14336 x 4096 at M = 544 .. 608, cold, 74 .. 76 -> 61 .. 62 us)
    const int64_t rows256 = (M + 255) / 256;
    const bool filled = (int64_t)M * 5 >= rows256 * 256 * 4 || (rows256 >= 3 && (int64_t)M * 10 >= rows256 * 256 * 7);
    return t * sk * 10 >= (int64_t)cus * 6 && filled;
  };
  const bool take256 = tiles(256, 256) * parts256 * 20 >= cus * (parts256 == 2 ? 10 : 11) || long_k_256();
  // (not when M fills less than 70 % of the 256-row tiles and the 128 x 256 tiles fit the device in one round: 3584 x 18944
  // at M = 288 / 320, 222 tiles, 47.4 -> 41.3 us; on 4096 x 28672, 336 tiles, the 256 x 256 tiles stay ahead, 53 against 75 us)
  const bool rows_poorly_filled = (int64_t)M * 10 < (int64_t)((M + 255) / 256) * 256 * 7 && tiles(128, 256) <= cus &&
                                  tiles(128, 256) * 10 >= cus * 7 && tuning().exp[9] != 1;
  // (128 x 256 from 70 % of the compute units on.  Between 55 and 70 % they win on weights that are already cached -- 4096 x
  // 6144 at M = 768, 144 tiles, 40.5 -> 36.1 us -- and lose on cold ones, 36.1 against 42.5 us for the 128 x 128 tiles: a
  // layer's weights are cold when its turn comes, so the cold figure decides.)
  if (pl.cfg <= 0)
    pl.cfg = take256 && !rows_poorly_filled ? 1 : (tiles(128, 256) * 10 >= cus * 7 ? 7 : (take128 ? 3 : 4));
  // One tile row of 129 .. 256 rows on a wide layer: 256 x 128 tiles (8 wavefronts of 64 x 64) from 55 % of the compute units
  // up to one round -- as many tiles as 128 x 256 ones, but every weight row is read by one workgroup only (cold:
  // 4096 x 28672 at M = 224 / 256 49.7 / 51.9 -> 45.0 / 47.0 us, 3584 x 18944 at M = 136 .. 256 37.5 .. 46.3 -> 31.2 .. 39.1 us,
  // 8192 x 28672 at M = 256 97.9 -> 85.7 us; at 42-44 % of the units, 5120 x 13824 and 4096 x 14336, the 128 x 128 tiles
  // stay ahead by 6-10 %)
  if (tuning().fp8_tile_cfg <= 0 && M > 128 && M <= 256 && tiles(256, 128) <= cus && tiles(256, 128) * 20 >= (int64_t)cus * 11)
    pl.cfg = 9;
  // 256 x 384 tiles (wavefronts of 128 x 96) where the 256 x 256 tiles leave the last round of workgroups badly filled and
  // these do not: 4096 x 6144 at M = 4096 is 384 tiles = 1.5 rounds, or 256 = one round (101.4 -> 92.3 us).  Per tile they
  // are slower (4096 x 4096 at M = 4096: 62.8 against 72.7 us), so only for a gain of a fifth in the fill of the rounds.
  if (tuning().fp8_tile_cfg <= 0 && pl.cfg == 1 && N % 384 == 0 && K / 64 < 160) {
    auto fill = [&](int64_t t) { return (double)t / (double)(((t + cus - 1) / cus) * cus); };
    if (tiles(256, 256) > cus && fill(tiles(256, 384)) >= 1.2 * fill(tiles(256, 256))) pl.cfg = 10;
  }
  // the smallest tile with two k-slices per step: 5-8 % faster on a short K (half the barriers), no gain on a long one
  if (tuning().fp8_tile_cfg <= 0 && pl.cfg == 4 && K % 128 == 0 && K <= 8192) pl.cfg = 14;
  // 64 x 64 tiles while they fit the device in one round, on a short K: twice the workgroups with loads in flight
  // (cold weights: 4096 x 6144 at M = 128 21.8 -> 15.0 us, 4096 x 4096 at M = 192 19.8 -> 13.8 us; 14336 x 4096 at
  // M = 128 30.0 -> 34.0 us, and slower as soon as the tiles need a second round)
  if (tuning().fp8_tile_cfg <= 0 && pl.cfg == 14 && tiles(64, 64) <= cus) pl.cfg = 15;
  // 128 x 64 tiles where the 64 x 64 ones need a second round: up to three tile rows, each weight row read by one workgroup
  // per tile row as with the 64 x 64 tiles, when they leave compute units for one more row of workgroups past M (see
  // m_tiles_extra in dispatch_tile), or are more workgroups than the 64 x 128 tiles while the last tile row holds at most
  // 32 rows of M.  Cold: 4096 x 4096 at M = 264 .. 384 18.0 .. 18.6 -> 15.2 .. 15.5 us, 5120 x 5120 at M = 200 .. 288 22.5 .. 24.2
  // -> 19.6 .. 20.3 us, 3584 x 4608 at M = 200 / 256 16.7 / 16.9 -> 13.9 / 14.0 us, 6656 x 6656 at M = 136 31.0 -> 24.4 us,
  // 4096 x 6144 at M = 136 / 160 19.0 -> 15.4 / 16.3 us and at M = 176 / 192, 48 / 64 rows in the last tile row, 19.1 -> 20.0 us;
  // with as many workgroups as the 64 x 128 tiles and no room for the row past M they lose 6 % (4096 x 6144 at M = 256).
  if (tuning().fp8_tile_cfg <= 0 && pl.cfg == 14 && K <= 6656 && M <= 384 && tiles(128, 64) <= cus && tuning().exp[14] != 1) {
    const int64_t t = tiles(128, 64), cols = (N + 63) / 64;
    const int last_rows = M - (M - 1) / 128 * 128;
    if (t + cols <= (int64_t)cus || (t > tiles(64, 128) && last_rows <= 32)) pl.cfg = 16;
  }
  if (pl.cfg >= 10 && K % 128 != 0) pl.cfg %= 10;      // two k-slices per step need K % 128 == 0
  int sk = 1;
  const int steps = K / 64;
  Fp8TilePlan saved = pl;
  for (int pass = 0; pass < 2; ++pass) {
  sk = 1;
  switch (pl.cfg) {
    case 3: case 13: case 23: pl.bm = 128; pl.bn = 128; pl.nw = 4; break;
    case 4: case 14: case 24: pl.bm = 64; pl.bn = 128; pl.nw = 4; break;
    case 5: case 15: pl.bm = 64; pl.bn = 64; pl.nw = 4; break;
    case 16: pl.bm = 128; pl.bn = 64; pl.nw = 4; break;
    case 7: case 17: pl.bm = 128; pl.bn = 256; pl.nw = 8; break;
    case 9: pl.bm = 256; pl.bn = 128; pl.nw = 8; break;
    case 2: pl.bm = 256; pl.bn = 256; pl.nw = 4; break;
    case 10: case 11: pl.bm = 256; pl.bn = 384; pl.nw = 8; break;
    default: pl.bm = 256; pl.bn = 256; pl.nw = 8; break;
  }
  pl.tiles = tiles(pl.bm, pl.bn);
  if (pl.tiles < cus && pl.bm * pl.bn >= 128 * 256) {
    // large tiles, one workgroup per compute unit
    const int min_steps = pl.tiles * 4 <= cus ? 32 : 64;        // shorter parts only when the tiles leave 3/4 of the device idle
    sk = (int)((int64_t)cus / pl.tiles);
    if (sk > 8) sk = 8;
    if (sk > steps / min_steps) sk = steps / min_steps;
    if (sk < 1) sk = 1;
    while (sk & (sk - 1)) --sk;       // a power of two (3 splits measured slower than 2)
  } else if (pl.tiles < cus) {
    // Small tiles (two workgroups share a compute unit), measured with cold weights on the Llama shapes, M = 48 .. 512:
    // tiles that leave 2/3 of the device idle are split until there is about one workgroup per compute unit (parts of
    // at least 16 steps: 4096 x 4096 at M = 128, 4 parts of 16 steps 15.7 us, 2 of 32 18.4 us, 8 of 8 22.7 us); fuller
    // devices stay unsplit (the rotated K loop of the unsplit kernel is worth more there: 4096 x 6144 at M = 192,
    // 20.8 against 31.0 us in 2 parts; 96 tiles in 2 parts: -3 % on 4096 x 6144, +6 % on 4096 x 4096) unless K is very
    // long, where a part is halved while the halves stay 50 steps long and the workgroups fit the device at once
    // (14336 x 4096 at M = 256: 62.6 / 45.8 / 44.3 us in 1 / 2 / 4 parts).
    if (pl.tiles * 3 <= (int64_t)cus) {
      sk = (int)((int64_t)cus / pl.tiles);
      if (sk > 8) sk = 8;
      // (parts of at least 16 steps; 32 between 1/4 and 1/3 of the device: 5120 x 5120 at M = 64, 80 tiles in two parts
      // of 40 steps, 22.8 -> 18.2 us; 2560 x 2560 at M = 128 in two parts of 20, 11.5 -> 12.3 us)
      const int min_part = pl.tiles * 4 <= (int64_t)cus ? 16 : 32;
      if (sk > steps / min_part) sk = steps / min_part;
      if (sk < 1) sk = 1;
      while (sk & (sk - 1)) --sk;
      // (two tile rows and more of a short K stay whole: their tile rows start at different K steps, which parts of 16
      // steps and a hand-over do not beat -- 2048 x 2048 at M = 72 .. 128, 64 tiles: 9.7 .. 10.6 us in two parts, 7.5 .. 8.6 us
      // whole, 3072 x 1024 at M = 128 11.8 against 11.0 us; from 56 steps on the parts are ahead, 3584 x 2048 at M = 128: 11.9
      // against 12.8 us, 4096 x 2048: 12.4 against 13.1 us)
      if (M > pl.bm && steps < 56) sk = 1;
    }
    while (sk < 8 && steps / sk >= 100 && pl.tiles * sk * 2 <= 2 * (int64_t)cus) sk *= 2;
    // between one and 1.75 workgroups per compute unit some units run two of them and set the pace: the parts that give
    // one per unit instead, unless they get longer than 128 steps (13824 x 5120 at M = 65 .. 256, 80 tiles: 320 workgroups
    // 41 .. 57 us, 240 workgroups 33 .. 42 us; 6656 x 6656 at M = 65, 208 tiles of 64 x 64: 20.8 -> 17.7 us unsplit;
    // 17920 x 6656 at M = 512, 208 tiles: 97 us in two parts of 140 steps, 105 us unsplit)
    const int64_t wgs = pl.tiles * sk;
    if (sk > 1 && wgs > cus && wgs * 4 < (int64_t)cus * 7) {
      const int fit = (int)((int64_t)cus / pl.tiles);
      // (an unsplit K, which also saves the hand-over, from 60 % of the units on -- 6656 x 6656 at M = 136 / 192, 156 tiles:
      // 41 / 45 -> 33 us, 7680 x 7680 47 / 51 -> 40 us; fewer parts from 90 % on -- 14336 x 4096
      // at M = 384, 96 tiles: 4 parts 52.0 us, 2 parts 54.8 us)
      const int64_t filled = (int64_t)fit * pl.tiles;
      if (fit >= 1 && steps / fit <= 128 && (fit == 1 ? filled * 5 >= (int64_t)cus * 3 : filled * 10 >= (int64_t)cus * 9)) sk = fit;
    }
    // Up to three tile rows of K <= 6656 with compute units left for one more row of workgroups stay whole: that row
    // then runs past M beside them (see m_tiles_extra in dispatch_tile), which parts and their hand-over do not beat:
    // 5120 x 5120 at M = 40 .. 128 14.2 .. 18.4 -> 13.2 us, 6656 x 6656 at M = 40 / 64 17.7 / 20.7 -> 16.0 / 16.7 us, 4096 x 2048 at
    // M = 192 12.6 -> 10.6 us; on K = 7168 and 8192 the parts stay ahead, 8192 x 3584 at M = 64 15.7 against 17.8 us.
    {
      const int64_t rows = (M + pl.bm - 1) / pl.bm;
      if (K <= 6656 && rows <= 3 && pl.tiles + pl.tiles / rows <= (int64_t)cus && tuning().exp[13] != 1) sk = 1;
    }
  }
  // 64 x 128 tiles of a long K whose parts still run 64 steps and more: 128 x 128 tiles instead -- half the tiles, so twice
  // the parts of half the length on the same number of workgroups (cold, M = 80 .. 128: 18944 x 3584 33.8 -> 31.7 us,
  // 9216 x 4608 30.7 -> 25.9 us, 17920 x 6656 52.6 -> 42.2 us, 24576 x 6144 71.7 -> 61.1 us; M = 136 .. 256: 12288 x 3072
  // 41 -> 32 us; with parts of 56 steps and less they lose 1-9 %: 14336 x 4096, 11008 x 4096, 10240 x 2560)
  // -- where those are fewer tiles (M beyond one 64-row block) and come to at least 80 % of the workgroups, or of the compute
  // units if the 64 x 128 tiles exceed them (13824 x 5120, 20480 x 5120: 240 against 160 workgroups, +3 .. +9 %)
  if (pass == 0 && tuning().fp8_tile_cfg <= 0 && tuning().fp8_split <= 0 && pl.cfg == 4 && steps / sk >= 64 &&
      tiles(128, 128) < pl.tiles) {
    saved = pl;
    saved.sk = sk;
    pl.cfg = 3;
    continue;
  }
  if (pass == 1) {
    const int64_t w4 = saved.tiles * saved.sk < cus ? saved.tiles * saved.sk : cus;
    if (pl.tiles * sk * 10 < w4 * 8) {      // too few workgroups: back to the 64 x 128 plan
      pl = saved;
      sk = saved.sk;
    }
  }
  break;
  }
  // 256 x 256 tiles (one workgroup per compute unit) whose count ends in a round of workgroups that is at most half full:
  // the tiles of that round are split over K so that their parts fill it, the others stay whole.  Parts of at least 16
  // steps.  (The gain is less than the rounds saved: a half-empty round runs faster per workgroup than a full one -- the
  // device is power-limited -- and the parts' hand-over costs 10-15 us.)
  pl.tail_first = 0;
  if (sk == 1 && pl.bm == 256 && pl.bn == 256 && pl.nw == 8 && pl.tiles > cus && tuning().exp[10] != 1 && tuning().fp8_split <= 0) {
    const int64_t rest = pl.tiles % cus;
    if (rest > 0 && rest * 2 <= cus && steps >= 32 && (steps >= 128 || rest * 8 <= cus || tuning().exp[10] == 2)) {
      int parts = (int)(cus / rest);
      if (parts > 4) parts = 4;
      if (parts > steps / 16) parts = steps / 16;
      if (parts >= 2) {
        sk = parts;
        pl.tail_first = pl.tiles - rest;
      }
    }
  }
  if (tuning().fp8_split > 0) sk = tuning().fp8_split <= steps ? tuning().fp8_split : steps;
  while (sk > 1 && (uint64_t)sk * (uint64_t)(pl.tiles - pl.tail_first) * pl.bm * pl.bn * 4 >= (1ull << 32)) --sk;   // 32-bit buffer offsets
  pl.sk = sk;
  if (sk == 1) pl.tail_first = 0;
  // A split K with compute units left for the parts of one more tile row: that row runs past M beside the real ones, as
  // with an unsplit K (see m_tiles_extra in dispatch_tile); its workgroups take no part in the hand-over, but tile
  // positions -- and with them the places in the scratch -- count it.  Cold: 7168 x 2048 at M = 40 / 64 / 192 12.1 / 13.6 /
  // 18.0 -> 10.3 / 10.4 / 12.8 us, 8192 x 1024 at M = 40 .. 192 12.4 .. 13.2 -> 10.7 .. 11.0 us.
  if (sk > 1 && pl.tail_first == 0 && tuning().exp[13] != 1) {
    const int64_t rows = (M + pl.bm - 1) / pl.bm, cols = pl.tiles / rows;
    if (rows <= 3 && (pl.tiles + cols) * sk <= (int64_t)cus) pl.extra_tiles = cols;
  }
  return pl;
}

template <bool BF16_OUT>
static int dispatch_tile(const Fp8MMParams& p_in, int64_t c_tmp_bytes, int64_t counter_ints, hipStream_t s) {
  Fp8MMParams p = p_in;
  const bool direct_ok = tuning().fp8_tile_impl == 0 && p.K % 64 == 0 && (uint64_t)p.M * (uint64_t)p.lda < (1ull << 32) &&
                         (uint64_t)p.N * (uint64_t)p.ldb < (1ull << 32);
  if (direct_ok && tuning().fp8_tile_impl == 0 && tuning().fp8_tile_cfg >= 0) {
    Fp8TilePlan pl = plan_tile3(p.M, p.N, p.K);
    // without (enough) scratch from the caller the unsplit kernel still gives the result
    if (pl.sk > 1 && (p.c_tmp == nullptr || p.counters == nullptr || counter_ints < pl.counter_ints() ||
                      c_tmp_bytes < pl.tmp_bytes()))
      pl.sk = 1;
    if (pl.sk == 1) pl.tail_first = 0;
    p.SK = pl.sk;
    p.tail_first = (int)pl.tail_first;
    {
      const int64_t tiles_m = (p.M + pl.bm - 1) / pl.bm;
      const int64_t cus = num_cus_current_device();
      // (with K split over workgroups the rotation gains nothing on cold weights and costs 20-30 % on cached ones.)
      // Up to 4 tile rows on a device that the tiles leave a fifth empty; any number of tile rows in one round of workgroups
      // when the weights are small enough (32 MiB: 4 MiB per L2) that the part another tile row has just read is still in
      // the L2 -- cold, 4096 x 4096 at M = 256 .. 512: 16.2 / 23.5 -> 12.7 / 18.8 us, 4096 x 6144 at M = 1024 41.4 -> 36.4 us,
      // 2048 x 2048 at M = 1024 13.9 -> 11.2 us; larger weights lose (6656 x 6656 at M = 72: 17.3 -> 24.1 us; 4096 x 28672
      // at M = 192 .. 384: +7 %), and so do tiles that need a second round (4096 x 6144 at M = 768: 35.9 -> 41.6 us).
      p.rotate_k = pl.sk == 1 && tiles_m > 1 &&
                   ((tiles_m <= 4 && pl.tiles * 5 < cus * 4) || (pl.tiles <= cus && (int64_t)p.K * p.N <= ((int64_t)32 << 20)));
      // A last tile row filled to a third at most.  Two tile rows: nobody rotates (the nearly empty row finishes early
      // whatever it reads, and rotated it reads for nothing what the full row does not read with it; cold: 4096 x 4096 at
      // M = 66 .. 84 13.3 -> 11.1 .. 11.8 us, 4096 x 6144 13.7 -> 11.6 .. 12.5 us).  64 x 64 tiles: the same with three and
      // four rows (4096 x 4096 at M = 132 .. 144 13.2 -> 11.2 .. 11.9 us, at M = 196 .. 208 13.1 -> 11.5 .. 12.1 us; from a fill
      // of 24 rows on the rotation is level or ahead).  Larger tiles with three rows and more keep the rotation (64 x 128:
      // 4096 x 6144 at M = 132 19.5 against 21.2 us, 4096 x 4096 at M = 264 18.2 against 21.1 us).
      if (p.rotate_k == 1 && ((int64_t)p.M - (tiles_m - 1) * pl.bm) * 3 <= pl.bm && (tiles_m == 2 || pl.bn == 64)) p.rotate_k = 0;
      // one or two tile rows on a wide layer: by tile column instead (see the kernel)
      if (p.rotate_k == 0 && pl.sk == 1 && tiles_m <= 2 && pl.tiles * 5 >= cus * 2) p.rotate_k = 2;
      if (tuning().exp[12] == 1) p.rotate_k = 0;      // (development switch: every tile starts at the first K step)
      // A tile row past M.  With at most three tile rows and compute units to spare, one more row of workgroups runs
      // beside the real ones: its activation rows lie past M (the loads return zeros, nothing is stored), its weight
      // loads are the real tiles' own.  Every weight line is then asked for by two workgroups on two compute units,
      // whichever gets there first, and arrives earlier for the other: what one compute unit has in flight is what bounds
      // a tile's operand stream at these sizes (deeper rings do not help, a second requester does).  Cold, 64 x 64 tiles:
      // 4096 x 4096 at M = 64 .. 192 13.2 .. 16.4 -> 10.8 .. 11.1 us, 5120 x 5120 at M = 64 / 128 17.0 / 17.4 -> 13.2 / 13.3 us,
      // 2048 x 2048 at M = 128 8.6 -> 7.3 us; 128 x 128 tiles: 4096 x 6144 at M = 384 25.8 -> 23.5 us, 8192 x 8192 at M = 384
      // 46.7 -> 41.7 us.  The real rows then start together (rotated they lose the gain); from four tile rows on the
      // rotation alone is level or ahead (3072 x 3072 at M = 384 14.8 against 16.0 us) and stays.
      p.m_tiles_extra = pl.extra_tiles > 0 && pl.sk > 1 ? 1 : 0;
      if (pl.sk == 1 && pl.tail_first == 0 && tiles_m <= 3 && pl.tiles + pl.tiles / tiles_m <= cus && tuning().exp[13] != 1) {
        p.m_tiles_extra = 1;
        p.rotate_k = 0;
      }
    }
    switch (pl.cfg) {
      case 1: return launch_tile3<BF16_OUT, 256, 256, 2, 4, 5, 1, 1>(p, s);   // alternating phases (see the kernel)
      case 8: return launch_tile3<BF16_OUT, 256, 256, 2, 4, 5>(p, s);
      case 2: return launch_tile3<BF16_OUT, 256, 256, 2, 2, 5>(p, s);
      case 10: return launch_tile3<BF16_OUT, 256, 384, 2, 4, 4, 1, 1>(p, s);   // 8 wavefronts of 128 x 96, alternating phases
      case 11: return launch_tile3<BF16_OUT, 256, 384, 2, 4, 4>(p, s);
      case 3: return launch_tile3<BF16_OUT, 128, 128, 2, 2, 5>(p, s);
      case 4: return launch_tile3<BF16_OUT, 64, 128, 2, 2, 5>(p, s);
      case 6: return launch_tile3<BF16_OUT, 256, 256, 2, 4, 3>(p, s);
      case 7: return launch_tile3<BF16_OUT, 128, 256, 2, 4, 5>(p, s);
      // two k-slices per step (K % 128 == 0)
      case 13: return launch_tile3<BF16_OUT, 128, 128, 2, 2, 4, 2>(p, s);
      case 23: return launch_tile3<BF16_OUT, 128, 128, 2, 2, 2, 2>(p, s);
      case 14: return launch_tile3<BF16_OUT, 64, 128, 2, 2, 5, 2>(p, s);
      case 24: return launch_tile3<BF16_OUT, 64, 128, 2, 2, 3, 2>(p, s);
      case 15: return launch_tile3<BF16_OUT, 64, 64, 2, 2, 5, 2>(p, s);
      case 5: return launch_tile3<BF16_OUT, 64, 64, 2, 2, 5>(p, s);
      case 16: return launch_tile3<BF16_OUT, 128, 64, 2, 2, 5, 2>(p, s);
      case 17: return launch_tile3<BF16_OUT, 128, 256, 2, 4, 3, 2>(p, s);
      case 9: return launch_tile3<BF16_OUT, 256, 128, 4, 2, 5>(p, s);
      default: break;
    }
  }
  p.SK = 1;
  if (direct_ok && p.K % F8_BK == 0) {
    const int cus2 = num_cus_current_device();
    auto tiles2 = [&](int bm, int bn) { return (int64_t)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn); };
    if (tiles2(256, 256) >= cus2) return launch_tile2<BF16_OUT, 4, 4>(p, s);
    if (tiles2(128, 128) >= cus2) return launch_tile2<BF16_OUT, 2, 2>(p, s);
    return launch_tile2<BF16_OUT, 1, 2>(p, s);
  }
  const int cus = num_cus_current_device();
  auto tiles = [&](int bm, int bn) { return (int64_t)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn); };
  if (tiles(256, 256) >= cus) return launch_tile<BF16_OUT, 4, 4>(p, s);
  if (tiles(128, 128) >= cus) return launch_tile<BF16_OUT, 2, 2>(p, s);
  return launch_tile<BF16_OUT, 1, 2>(p, s);
}

template <bool BF16_OUT, int KS, int MB, bool HALVES = false>
static void launch_stream(const Fp8MMParams& p_in, int wk, int gx, hipStream_t s) {
  Fp8MMParams p = p_in;
  p.nt_base = (p.N / 16) / gx;
  p.nt_rem = (p.N / 16) % gx;
  p.a_extent = (uint32_t)((int64_t)(p.M - 1) * p.lda + p.K);
  p.b_extent = (uint32_t)((int64_t)(p.N - 1) * p.ldb + p.K);
  const size_t lds = wk > 1 ? (size_t)2 * wk * MB * 64 * sizeof(v4f) : 0;
  if (p.nt_base == 1 && p.nt_rem == 0)
    hipLaunchKernelGGL((fp8_mm_stream_kernel<BF16_OUT, KS, MB, HALVES, false>), dim3(gx, HALVES ? 2 : 1), dim3(64, wk), lds, s, p, wk);
  else
    hipLaunchKernelGGL((fp8_mm_stream_kernel<BF16_OUT, KS, MB, HALVES, true>), dim3(gx, HALVES ? 2 : 1), dim3(64, wk), lds, s, p, wk);
}

// The stream kernel addresses its operands with 32-bit offsets from buffer descriptors: both must end below 2 GiB
// (otherwise the tile kernels take the problem).
static bool stream_offsets_fit(const Fp8MMParams& p) {
  return (int64_t)(p.M - 1) * p.lda + p.K < (1ll << 31) && (int64_t)(p.N - 1) * p.ldb + p.K < (1ll << 31);
}

// K steps (of 128) per wavefront of the stream kernel for a problem, 0 if the kernel does not take it (the activations of
// a wavefront's K slab live in registers: at most 8 wavefronts along K, 14 steps each for one m-block, 8 for two).
static int stream_steps_per_wave(int64_t M, int64_t N, int64_t K) {
  const int64_t steps = (K + 127) / 128;
  // three and four m-blocks: K = 1664 .. 4096 (4 steps per wavefront keep the registers, and the workgroup must have a
  // wavefront per m-block for the reduction).  Measured against the tile kernel with K split, cold weights, M = 48 / 64:
  // 4096 x 4096 21.0 / 21.4 -> 11.6 / 13.4 us, 4096 x 6144 22.7 / 22.9 -> 14.6 / 16.5 us, 4096 x 28672 36.3 / 37.3 ->
  // 35.9 / 38.7 us: four m-blocks only up to two rounds of workgroups.
  if (M > 32) {
    const bool fits = steps <= 8 * 4 && steps >= 13;
    // ... unless the 64 x 64 tiles with one more tile row past M fit the device (see m_tiles_extra in dispatch_tile) and the
    // weights are large enough: that plan takes the same time for 33 as for 64 rows, this kernel's time grows with the
    // m-blocks.  Cold, M = 40 / 64: 4096 x 6144 12.1 / 15.0 -> 11.3 / 11.4 us, 4096 x 8192 13.2 / 16.1 -> 12.0 / 12.2 us, 4096 x 4096
    // 9.8 / 12.7 against 10.8 / 10.8 us (the tiles from 49 rows on), 3072 x 3072 7.6 / 9.6 against 9.1 / 9.1 us, 2048 x 2048
    // 5.5 / 7.0 against 7.4 / 7.4 us (this kernel).
    const int64_t cols = (N + 63) / 64;
    if (tuning().exp[13] != 1 && tuning().fp8_tile_cfg <= 0 && K % 128 == 0 && 2 * cols <= (int64_t)num_cus_current_device() &&
        (K * N >= ((int64_t)20 << 20) || (M > 48 && K * N >= ((int64_t)8 << 20))))
      return 0;
    return (fits && (M <= 48 || (M <= 64 && N / 16 <= 2 * num_cus_current_device()))) ? 4 : 0;
  }
  if (steps <= 8 * 4) return 4;
  if (steps <= 8 * 8) return 8;
  if (steps <= 8 * 14 && M <= 16) return 14;
  return 0;
}

// The stream kernel over two halves of K (two workgroups per n-tile range, partial tiles handed over through the caller's
// scratch): K steps per wavefront, 0 if this route does not take the problem.  It covers what the registers of one
// workgroup cannot at two m-blocks: 16 < M <= 32 up to K = 16384 (cold weights, against the tile kernel with K split:
// 14336 x 4096 at M = 24 / 32 34.7 / 35.1 -> 21.6 / 22.5 us, 16384 x 4096 at M = 32 37.1 -> 27.4 us).  For M <= 16 beyond
// K = 14336 (14 steps per wavefront and half) the tile kernel stays ahead: 28672 x 8192 72 against 85 us.
static int stream_split_steps_per_wave(int64_t M, int64_t N, int64_t K) {
  if (tuning().fp8_stream_split < 0 || M <= 16 || M > 32 || stream_steps_per_wave(M, N, K) != 0) return 0;
  const int64_t half = ((K + 127) / 128 + 1) / 2;
  return half <= 8 * 8 ? 8 : 0;
}

template <bool BF16_OUT>
static bool dispatch_stream_split(const Fp8MMParams& p, int64_t c_tmp_bytes, int64_t counter_ints, hipStream_t s) {
  const int ks = stream_split_steps_per_wave(p.M, p.N, p.K);
  if (ks == 0 || !stream_offsets_fit(p)) return false;
  const int MB = (p.M + 15) / 16, NT = p.N / 16;
  if (p.c_tmp == nullptr || p.counters == nullptr || counter_ints < (int64_t)NT * MB ||
      c_tmp_bytes < (int64_t)2 * NT * MB * 1024 || (int64_t)2 * NT * MB * 1024 >= (1ll << 31))
    return false;                                   // without the scratch the tile kernel still gives the result
  const int half = ((p.K + 127) / 128 + 1) / 2;
  const int wk = (half + ks - 1) / ks;              // >= 5: the K range of this route starts above one workgroup's
  const int cus = num_cus_current_device();
  const int rounds = (2 * NT + cus - 1) / cus;
  int gx = tuning().fp8_gx > 0 ? tuning().fp8_gx : (NT + rounds - 1) / rounds;
  if (gx > NT) gx = NT;
  launch_stream<BF16_OUT, 8, 2, true>(p, wk, gx, s);
  return true;
}

template <bool BF16_OUT, int KS, int MB, int NSR>
static bool launch_stream2(const Fp8MMParams& p_in, int wk, int gx, hipStream_t s) {
  Fp8MMParams p = p_in;
  p.nt_base = (p.N / 16) / gx;
  p.nt_rem = (p.N / 16) % gx;
  p.a_extent = (uint32_t)((int64_t)(p.M - 1) * p.lda + p.K);
  p.b_extent = (uint32_t)((int64_t)(p.N - 1) * p.ldb + p.K);
  const size_t lds = (size_t)wk * NSR * 4096 + (wk > 1 ? (size_t)2 * wk * MB * 64 * sizeof(v4f) : 0);
  auto kern = fp8_mm_stream2_kernel<BF16_OUT, KS, MB, NSR>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "fp8_scaled_mm") != VAQ_OK) return false;      // (the kernel above then takes the problem)
  hipLaunchKernelGGL(kern, dim3(gx), dim3(64, wk), lds, s, p, wk);
  return true;
}

// Steps per wavefront of the stream kernel with the weights through LDS, 0 where the kernel above stays.  Measured with
// cold weights against the kernel above (us, M = 1 / 4 / 16): 4096 x 6144 8.6 / 9.0 / 10.3 -> 7.7 / 7.8 / 8.6, 4096 x 4096
// 6.0 / 6.2 / 7.1 -> 5.7 / 5.9 / 6.6, 4096 x 28672 25.8 / 26.1 / 27.8 -> 21.9 / 22.0 / 23.3, 14336 x 4096 13.8 / 14.8 / 18.0 ->
// 12.0 / 12.4 / 15.3; two m-blocks (M = 32): 4096 x 6144 11.4 -> 10.5, 4096 x 28672 30.6 -> 26.5, 4096 x 4096 8.7 -> 8.9
// with 4 steps per wavefront and 8.3 with 8 (M = 17 / 24: 7.5 / 8.2 -> 7.1 / 7.7), which layers of at most one n-tile per
// compute unit therefore take.
// (development switch exp[4]: 1 / 2 / 3 force 8 / 4 / 16 steps, 9 switches the kernel off)
static int stream2_steps_per_wave(const Fp8MMParams& p) {
  const int sw = tuning().exp[4];
  if (sw == 9 || p.M > 32 || p.K % 16 != 0 || !stream_offsets_fit(p)) return 0;
  const int steps = (p.K + 127) / 128, MB = (p.M + 15) / 16;
  int ks = 0;
  if (sw >= 1 && sw <= 3) ks = sw == 1 ? 8 : (sw == 2 ? 4 : 16);
  else if (MB == 1) ks = steps < 64 ? 8 : (steps <= 128 ? 16 : 0);      // (K = 8192: 8192 x 8192 at M = 1 16.9 us with 8 steps, 14.6 with 16)
  // (two m-blocks of K = 4224 .. 8192 with 8 steps per wavefront, M = 24 / 32 against the kernel above: 5120 x 5120 13.9 / 14.7 ->
  // 10.9 / 11.8 us, 6656 x 6656 16.8 / 18.0 -> 13.6 / 14.7 us, 5120 x 27648 38.2 / 39.2 -> 29.4 / 30.4 us, 8192 x 8192 20.9 / 22.3 -> 19.4 / 20.7 us)
  else ks = steps > 64 ? 0 : (steps > 32 ? 8 : (p.N / 16 > num_cus_current_device() ? 4 : 8));
  if (ks == 0 || (steps + ks - 1) / ks > 8 || (MB == 2 && ks == 16)) return 0;
  return ks;
}

template <bool BF16_OUT>
static bool dispatch_stream2(const Fp8MMParams& p, hipStream_t s) {
  const int ks = stream2_steps_per_wave(p);
  if (ks == 0) return false;
  const int steps = (p.K + 127) / 128;
  const int wk = (steps + ks - 1) / ks;
  const int MB = (p.M + 15) / 16, NT = p.N / 16;
  const int cus = num_cus_current_device();
  const int rounds = (NT + cus - 1) / cus;
  int gx = (NT + rounds - 1) / rounds;
  // one m-block on a layer of many rounds: two workgroups per compute unit (4096 x 28672 at M = 1: 23.8 -> 21.9 us; three
  // or more per unit 25.8 us and up)
  if (MB == 1 && NT >= 4 * cus) gx = 2 * cus;
  if (tuning().fp8_gx > 0) gx = tuning().fp8_gx;
  if (gx > NT) gx = NT;
  if (MB == 1) {
    if (ks == 4) return launch_stream2<BF16_OUT, 4, 1, 2>(p, wk, gx, s);
    if (ks == 8) return launch_stream2<BF16_OUT, 8, 1, 4>(p, wk, gx, s);
    return launch_stream2<BF16_OUT, 16, 1, 4>(p, wk, gx, s);
  }
  if (ks == 4) return launch_stream2<BF16_OUT, 4, 2, 2>(p, wk, gx, s);
  return launch_stream2<BF16_OUT, 8, 2, 4>(p, wk, gx, s);
}

template <bool BF16_OUT>
static bool dispatch_stream(const Fp8MMParams& p, hipStream_t s) {
  const int steps = (p.K + 127) / 128;
  const int MB = (p.M + 15) / 16;
  const int ks = stream_steps_per_wave(p.M, p.N, p.K);
  if (ks == 0 || !stream_offsets_fit(p)) return false;
  const int wk = (steps + ks - 1) / ks;
  const int NT = p.N / 16;
  // one workgroup per compute unit, the n-tiles dealt out evenly over the fewest rounds: every workgroup loads all the
  // activations of its K slabs, so more workgroups than compute units only multiply that traffic (measured, cold weights,
  // against two workgroups per compute unit: 4096 x 6144 at M = 16 / 32 11.9 / 16.4 -> 10.4 / 12.4 us, 4096 x 28672
  // 31.8 / 38.0 -> 30.4 / 31.9 us, M = 1 unchanged or 3 % faster)
  const int cus = num_cus_current_device();
  const int rounds = (NT + cus - 1) / cus;
  int gx = (NT + rounds - 1) / rounds;
  // One m-block, measured with cold weights: on a layer of many rounds two workgroups per compute unit are ahead
  // (4096 x 28672 at M = 1 / 4 / 16: 28.1 / 28.2 / 29.2 -> 25.7 / 26.1 / 27.8 us; at M = 32 30.5 -> 33.0 us), and with up to
  // four rows a layer of one to two rounds runs one tile per workgroup (4096 x 6144 at M = 1 / 4: 9.3 / 9.4 -> 8.6 / 9.0 us;
  // at M = 16 10.2 -> 10.9 us).
  if (MB == 1 && NT >= 4 * cus) gx = 2 * cus;
  else if (p.M <= 4 && NT > cus && NT <= 2 * cus) gx = NT;
  if (tuning().fp8_gx > 0) gx = tuning().fp8_gx;
  if (gx > NT) gx = NT;
  if (MB == 1) {
    if (ks == 4) launch_stream<BF16_OUT, 4, 1>(p, wk, gx, s);
    else if (ks == 8) launch_stream<BF16_OUT, 8, 1>(p, wk, gx, s);
    else launch_stream<BF16_OUT, 14, 1>(p, wk, gx, s);
  } else if (MB == 2) {
    if (ks == 4) launch_stream<BF16_OUT, 4, 2>(p, wk, gx, s);
    else launch_stream<BF16_OUT, 8, 2>(p, wk, gx, s);
  } else if (MB == 3) {
    launch_stream<BF16_OUT, 4, 3>(p, wk, gx, s);
  } else {
    launch_stream<BF16_OUT, 4, 4>(p, wk, gx, s);
  }
  return true;
}

}  // namespace vaq

extern "C" int vaq_fp8_scaled_mm_workspace(int64_t size_m, int64_t size_n, int64_t size_k, size_t* c_tmp_bytes,
                                           size_t* counter_ints) {
  return vaq_fp8_scaled_mm_workspace_tuned(size_m, size_n, size_k, c_tmp_bytes, counter_ints, nullptr);
}

extern "C" int vaq_fp8_scaled_mm_workspace_tuned(int64_t size_m, int64_t size_n, int64_t size_k, size_t* c_tmp_bytes,
                                                 size_t* counter_ints, const VaqTuning* tuning_or_null) {
  using namespace vaq;
  const TuningScope scope(tuning_or_null);
  VAQ_CHECK_ARG(c_tmp_bytes && counter_ints, "fp8_scaled_mm_workspace: null output pointer");
  VAQ_CHECK_ARG(size_m >= 0 && size_n > 0 && size_k > 0 && size_m < (1ll << 31) && size_n < (1ll << 31) &&
                    size_k < (1ll << 31), "fp8_scaled_mm_workspace: bad shape M=%lld N=%lld K=%lld", (long long)size_m,
                (long long)size_n, (long long)size_k);
  *c_tmp_bytes = 0;
  *counter_ints = 0;
  const bool stream = tuning().fp8_path != 2 && stream_steps_per_wave(size_m, size_n, size_k) != 0;      // needs no scratch
  if (stream) return VAQ_OK;
  if (tuning().fp8_path != 2 && stream_split_steps_per_wave(size_m, size_n, size_k) != 0) {
    const size_t units = (size_t)(size_n / 16) * (size_t)((size_m + 15) / 16);
    *c_tmp_bytes = 2 * units * 1024;
    *counter_ints = units;
    return VAQ_OK;
  }
  if (size_k % 64 != 0 || tuning().fp8_tile_impl != 0 || tuning().fp8_tile_cfg < 0) return VAQ_OK;
  const Fp8TilePlan pl = plan_tile3((int)size_m, (int)size_n, (int)size_k);
  *c_tmp_bytes = (size_t)pl.tmp_bytes();
  *counter_ints = (size_t)pl.counter_ints();
  return VAQ_OK;
}

extern "C" int vaq_fp8_scaled_mm(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb, const float* sa,
                                 int64_t sa_count, const float* sb, int64_t sb_count, const void* bias, void* out,
                                 int64_t ldc, int out_dtype, int64_t size_m, int64_t size_n, int64_t size_k,
                                 void* stream) {
  return vaq_fp8_scaled_mm_ws(a, lda, b, ldb, sa, sa_count, sb, sb_count, bias, out, ldc, out_dtype, size_m, size_n,
                              size_k, nullptr, 0, nullptr, 0, stream);
}

extern "C" int vaq_fp8_scaled_mm_ws(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb, const float* sa,
                                    int64_t sa_count, const float* sb, int64_t sb_count, const void* bias, void* out,
                                    int64_t ldc, int out_dtype, int64_t size_m, int64_t size_n, int64_t size_k,
                                    float* c_tmp, int64_t c_tmp_bytes, int32_t* counters, int64_t counter_ints,
                                    void* stream) {
  return vaq_fp8_scaled_mm_ws_tuned(a, lda, b, ldb, sa, sa_count, sb, sb_count, bias, out, ldc, out_dtype, size_m, size_n,
                                    size_k, c_tmp, c_tmp_bytes, counters, counter_ints, stream, nullptr);
}

extern "C" int vaq_fp8_scaled_mm_ws_tuned(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb, const float* sa,
                                          int64_t sa_count, const float* sb, int64_t sb_count, const void* bias,
                                          void* out, int64_t ldc, int out_dtype, int64_t size_m, int64_t size_n,
                                          int64_t size_k, float* c_tmp, int64_t c_tmp_bytes, int32_t* counters,
                                          int64_t counter_ints, void* stream, const VaqTuning* tuning_or_null) {
  using namespace vaq;
  const TuningScope scope(tuning_or_null);
  VAQ_CHECK_ARG(size_m >= 0 && size_n > 0 && size_k > 0, "fp8_scaled_mm: bad shape M=%lld N=%lld K=%lld",
                (long long)size_m, (long long)size_n, (long long)size_k);
  VAQ_CHECK_ARG(size_m < (1ll << 31) && size_n < (1ll << 31) && size_k < (1ll << 31), "fp8_scaled_mm: shape too large");
  VAQ_CHECK_ARG(size_k % 16 == 0 && size_n % 16 == 0, "fp8_scaled_mm: K = %lld and N = %lld must be multiples of 16",
                (long long)size_k, (long long)size_n);
  VAQ_CHECK_ARG(lda >= size_k && lda % 16 == 0, "fp8_scaled_mm: a row stride %lld must be >= K and a multiple of 16",
                (long long)lda);
  VAQ_CHECK_ARG(ldb >= size_k && ldb % 16 == 0, "fp8_scaled_mm: b column stride %lld must be >= K and a multiple of 16",
                (long long)ldb);
  VAQ_CHECK_ARG(ldc >= size_n && ldc % 8 == 0, "fp8_scaled_mm: out row stride %lld must be >= N and a multiple of 8",
                (long long)ldc);
  VAQ_CHECK_ARG(sa_count == 1 || sa_count == size_m, "fp8_scaled_mm: a_scales count %lld must be 1 or M",
                (long long)sa_count);
  VAQ_CHECK_ARG(sb_count == 1 || sb_count == size_n, "fp8_scaled_mm: b_scales count %lld must be 1 or N",
                (long long)sb_count);
  VAQ_CHECK_ARG(out_dtype == VAQ_F16 || out_dtype == VAQ_BF16, "fp8_scaled_mm: out dtype tag %d", out_dtype);
  if (size_m == 0) return VAQ_OK;
  VAQ_CHECK_ARG(a && b && sa && sb && out, "fp8_scaled_mm: null pointer");
  VAQ_CHECK_ARG(((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0 && ((uintptr_t)out % 8) == 0,
                "fp8_scaled_mm: a and b must be 16-byte aligned, out 8-byte aligned");
  VAQ_CHECK_ARG(((uintptr_t)sb % 16) == 0 && (!bias || ((uintptr_t)bias % 8) == 0),
                "fp8_scaled_mm: b_scales must be 16-byte aligned, bias 8-byte aligned");
  Fp8MMParams p;
  p.a = a; p.lda = lda; p.b = b; p.ldb = ldb;
  p.sa = sa; p.sa_per_row = (sa_count > 1 || size_m == 1) ? 1 : 0;
  p.sb = sb; p.sb_per_col = (sb_count > 1 || size_n == 1) ? 1 : 0;
  p.bias = (const uint16_t*)bias;
  p.out = (uint16_t*)out; p.ldc = ldc;
  p.M = (int)size_m; p.N = (int)size_n; p.K = (int)size_k;
  p.c_tmp = c_tmp;
  p.counters = counters;
  VAQ_CHECK_ARG(c_tmp == nullptr || ((uintptr_t)c_tmp % 16) == 0, "fp8_scaled_mm: c_tmp must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const bool bf16 = out_dtype == VAQ_BF16;
  bool done = false;
  const bool want_stream = tuning().fp8_path != 2 && stream_steps_per_wave(size_m, size_n, size_k) != 0;
  if (tuning().fp8_path != 2) done = bf16 ? dispatch_stream2<true>(p, s) : dispatch_stream2<false>(p, s);
  if (!done && want_stream) done = bf16 ? dispatch_stream<true>(p, s) : dispatch_stream<false>(p, s);
  if (!done && tuning().fp8_path != 2)
    done = bf16 ? dispatch_stream_split<true>(p, c_tmp_bytes, counter_ints, s)
                : dispatch_stream_split<false>(p, c_tmp_bytes, counter_ints, s);
  if (!done) {
    int rc = bf16 ? dispatch_tile<true>(p, c_tmp_bytes, counter_ints, s) : dispatch_tile<false>(p, c_tmp_bytes, counter_ints, s);
    if (rc != VAQ_OK) return rc;
  }
  VAQ_CHECK_LAUNCH("fp8_scaled_mm");
  return VAQ_OK;
}
