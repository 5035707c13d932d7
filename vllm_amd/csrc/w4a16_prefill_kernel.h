// W4A16 prefill-shaped GEMM (M > 32) for gfx950: C[M,N] = A[M,K] . dequant(B[K,N]) (+bias).
//
// MFMA-bound.  One workgroup (4 wavefronts, 2 x 2) computes a BM x BN output tile with v_mfma_f32_32x32x16;
// each wavefront owns (BM/2) x (BN/2) of it as WMB x WNB accumulator blocks of 32 x 32 fp32.
//
//  * K is walked in steps of 64.  A[BM x 64] goes global -> registers -> LDS unchanged.  The weight tile is read
//    in the NATIVE order (one 16-byte load per lane covers 128 k of one column, i.e. two K steps), dequantised
//    *with* its group scale and zero point to the 16-bit activation type and written to LDS as [n][k] so that both
//    MFMA operands are 16-byte, k-contiguous LDS reads.
//  * Dequantisation is exact: code -> fp32 (v_cvt_f32_ubyte), w = fma(code, s, -(z*s)) is the exact real number
//    (code - z) * s (<= 16 significant bits), then one round-to-nearest-even to bf16/fp16.  That is bit-for-bit the
//    weight `(q - z).to(dtype) * s` of the reference's dequantise-then-matmul path.
//  * LDS rows are padded to 72 elements (144 B): 16-byte accesses by 8 consecutive rows hit 8 disjoint bank groups.
//  * LDS is double buffered: while the MFMAs of step i run from buffer i&1, step i+1 is staged into the other
//    buffer; one barrier per step.  Global loads for step i+2 are issued right after the registers are drained.
//  * act_order: the caller passes activations already gathered through `perm` (vaq_permute_cols).
//  * Quantisation groups of 64 / 32 rows: SUBG = 2 / 4 scale (and zero-point) rows per 128-row weight tile; word j of a
//    lane's 16 bytes (rows 32j .. 32j+31 of the tile) takes the values of sub-group j*SUBG/4.
#pragma once
#include "vaq_common.h"
#include "tile_handover.h"

#include <type_traits>

namespace vaq {

struct PrefillParams {
  const uint16_t* a;
  int64_t lda;
  const v4u* b;
  const uint16_t* scales;
  const uint32_t* zeros;
  const uint16_t* bias;
  uint16_t* c;
  float* c_tmp;        // fp32 partial tiles when K is split over workgroups (SK > 1)
  int32_t* counters;   // arrival counters, zero on entry, left zero
  int M, N, K, G, NT, SK;
  int tail_first;      // 0: every tile in SK parts; > 0: only the tiles from this position on (see tile_slot)
  int s_stride, z_stride;   // elements between consecutive rows of scales (N) / zeros (N/8); 0 for channelwise scales
};

constexpr int PF_BK = 64;
constexpr int PF_PITCH = 72;   // LDS row pitch in 16-bit elements

template <bool BF16>
static __device__ inline uint32_t pack2(float lo, float hi) {
  if constexpr (BF16) {
    typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
    v2bf r = {(__bf16)lo, (__bf16)hi};   // v_cvt_pk_bf16_f32, round-to-nearest-even
    return __builtin_bit_cast(uint32_t, r);
  } else {
    return (uint32_t)F16Traits<false>::from_float(lo) | ((uint32_t)F16Traits<false>::from_float(hi) << 16);
  }
}

// float(byte B of x).  One instruction each; written as assembly because the compiler turns `(float)((x >> 8B) & 0xff)`
// of a nibble-masked word into a bit-field extract plus a conversion (two instructions per weight, and the
// dequantisation competes with the MFMAs for issue slots).  The results feed ordinary VALU instructions only.
template <int B>
static __device__ inline float cvt_ubyte(uint32_t x) {
  float f;
  if constexpr (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(x));
  else if constexpr (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(x));
  else if constexpr (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(x));
  else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(x));
  return f;
}

// Four bytes t (elements 0,4,1,5) and u (elements 2,6,3,7) of 8 consecutive k -> 8 scaled 16-bit weights in k order.
template <bool BF16>
static __device__ inline v4u scale_bytes(uint32_t t, uint32_t u, float s, float neg_zs) {
  const float e0 = fmaf(cvt_ubyte<0>(t), s, neg_zs);
  const float e4 = fmaf(cvt_ubyte<1>(t), s, neg_zs);
  const float e1 = fmaf(cvt_ubyte<2>(t), s, neg_zs);
  const float e5 = fmaf(cvt_ubyte<3>(t), s, neg_zs);
  const float e2 = fmaf(cvt_ubyte<0>(u), s, neg_zs);
  const float e6 = fmaf(cvt_ubyte<1>(u), s, neg_zs);
  const float e3 = fmaf(cvt_ubyte<2>(u), s, neg_zs);
  const float e7 = fmaf(cvt_ubyte<3>(u), s, neg_zs);
  v4u r;
  r.x = pack2<BF16>(e0, e1);
  r.y = pack2<BF16>(e2, e3);
  r.z = pack2<BF16>(e4, e5);
  r.w = pack2<BF16>(e6, e7);
  return r;
}

// One native weight word (8 codes of 8 consecutive k) -> 8 scaled 16-bit weights in k order.
template <bool BF16>
static __device__ inline v4u dequant_scaled(uint32_t w, float s, float neg_zs) {
  // nibble positions 0,2,4,6 -> elements 0,4,1,5; nibble positions 1,3,5,7 -> elements 2,6,3,7
  return scale_bytes<BF16>(w & 0x0f0f0f0fu, (w >> 4) & 0x0f0f0f0fu, s, neg_zs);
}

// 8-bit codes stored as two 4-bit planes: the words of the high and of the low nibbles of the same 8 codes.
template <bool BF16>
static __device__ inline v4u dequant_scaled8(uint32_t hi, uint32_t lo, float s, float neg_zs) {
  return scale_bytes<BF16>(((hi & 0x0f0f0f0fu) << 4) | (lo & 0x0f0f0f0fu), (hi & 0xf0f0f0f0u) | ((lo >> 4) & 0x0f0f0f0fu), s, neg_zs);
}

// FP8 e4m3 weights: eight bytes of 8 consecutive k (words wa: 0..3, wb: 4..7) -> 8 scaled 16-bit weights.  The packed
// conversion is exact (its scale operand only contributes a power of two: 1.0), the product with the scale is exact in
// fp32 (4 x 8..11 significant bits) and rounded once to the 16-bit type: the bits of `fp8.to(dtype) * scale`.
template <bool BF16>
static __device__ inline uint32_t fp8_pair_scaled(uint32_t w, bool hi, float s) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  const v2f f = hi ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(w, 1.0f, true) : __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(w, 1.0f, false);
  return pack2<BF16>(f[0] * s, f[1] * s);
}
template <bool BF16>
static __device__ inline v4u dequant_fp8(uint32_t wa, uint32_t wb, float s) {
  v4u r;
  r.x = fp8_pair_scaled<BF16>(wa, false, s);
  r.y = fp8_pair_scaled<BF16>(wa, true, s);
  r.z = fp8_pair_scaled<BF16>(wb, false, s);
  r.w = fp8_pair_scaled<BF16>(wb, true, s);
  return r;
}
// Register t (0..3) of dequant_fp8's result.
template <bool BF16>
static __device__ inline uint32_t dequant_fp8_part(uint32_t wa, uint32_t wb, float s, int t) {
  return fp8_pair_scaled<BF16>((t >> 1) ? wb : wa, (t & 1) != 0, s);
}

// Register t (0..3) of scale_bytes' result: elements 2t and 2t+1.
template <bool BF16>
static __device__ inline uint32_t scale_bytes_part(uint32_t tb, uint32_t ub, float s, float neg_zs, int t) {
  const uint32_t x = (t & 1) ? ub : tb;
  float l, h;
  if (t >> 1) {
    l = cvt_ubyte<1>(x);
    h = cvt_ubyte<3>(x);
  } else {
    l = cvt_ubyte<0>(x);
    h = cvt_ubyte<2>(x);
  }
  return pack2<BF16>(fmaf(l, s, neg_zs), fmaf(h, s, neg_zs));
}

template <bool BF16>
static __device__ inline uint32_t dequant_part8(uint32_t hi, uint32_t lo, float s, float neg_zs, int t) {
  return scale_bytes_part<BF16>(((hi & 0x0f0f0f0fu) << 4) | (lo & 0x0f0f0f0fu), (hi & 0xf0f0f0f0u) | ((lo >> 4) & 0x0f0f0f0fu), s, neg_zs, t);
}

// Quarter t of dequant_scaled: register t of its result (elements 2t and 2t+1).
template <bool BF16>
static __device__ inline uint32_t dequant_part(uint32_t w, float s, float neg_zs, int t) {
  return scale_bytes_part<BF16>(w & 0x0f0f0f0fu, (w >> 4) & 0x0f0f0f0fu, s, neg_zs, t);
}

// fp16 activations, 4-bit codes: the same weights from packed fp16 arithmetic.  (w >> 4t) & 0x000f000f | 0x64006400 is the
// pair (1024 + code[2t], 1024 + code[2t+1]); adding -(1024 + zero) is exact, and the packed multiply by the scale
// rounds the exact product (code - zero) * s once, to nearest even, like the conversion of the fp32 product does:
// the same bits from 15 instead of 23 instructions per 8 weights.  `s2` = the scale in both halves, `nzb2` = -(1024 + zero).
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
static __device__ inline uint32_t dequant_pair_h(uint32_t w, uint32_t s2, uint32_t nzb2, int t) {
  const uint32_t x = ((w >> (4 * t)) & 0x000f000fu) | 0x64006400u;
  const v2h d = __builtin_bit_cast(v2h, x) + __builtin_bit_cast(v2h, nzb2);
  return __builtin_bit_cast(uint32_t, d * __builtin_bit_cast(v2h, s2));
}
static __device__ inline v4u dequant_scaled_h(uint32_t w, uint32_t s2, uint32_t nzb2) {
  v4u r;
  r.x = dequant_pair_h(w, s2, nzb2, 0);
  r.y = dequant_pair_h(w, s2, nzb2, 1);
  r.z = dequant_pair_h(w, s2, nzb2, 2);
  r.w = dequant_pair_h(w, s2, nzb2, 3);
  return r;
}

// value of the sub-group that word j (0..3) of a tile belongs to
template <int SUBG>
static __device__ inline float pick_sub(const float (&a)[SUBG], int j) {
  if constexpr (SUBG == 1) return a[0];
  else if constexpr (SUBG == 2) return j >= 2 ? a[1] : a[0];
  else return j == 0 ? a[0] : (j == 1 ? a[1] : (j == 2 ? a[2] : a[3]));
}

template <bool BF16, int WMB, int WNB, bool HAS_ZP, int SUBG>
__global__ __launch_bounds__(256) void w4a16_prefill_kernel(const PrefillParams p) {
  using T = F16Traits<BF16>;
  constexpr int BM = 64 * WMB, BN = 64 * WNB;
  constexpr int A_CH = BM / 32;    // 16-byte chunks of A per thread per step
  constexpr int W_LD = BN / 64;    // 16-byte weight loads per thread per group
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  uint16_t* As = lds;                           // [2][BM][PITCH]
  uint16_t* Bs = lds + 2 * BM * PF_PITCH;       // [2][BN][PITCH]

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // XCD-aware tile order: consecutive workgroup ids land on different XCDs (round-robin over 8), so give each XCD a
  // contiguous band of tile ids; tiles in a band share A rows / W columns in that XCD's L2.
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  int bid = blockIdx.x;
  {
    const int per = (total + 7) / 8;
    const int xcd = bid & 7, idx = bid >> 3;
    const int remapped = xcd * per + idx;
    // only valid as a bijection when total % 8 == 0; otherwise keep the plain order
    if (total % 8 == 0) bid = remapped;
  }
  // walk tiles column-band-major in groups of 8 m-tiles so that neighbours share weights
  const int tm = bid % tiles_m, tn = bid / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN, nt0 = n0 / 16;

  // ---- per-thread staging state ----
  v4u areg[A_CH];
  v4u wreg[W_LD];
  float ws[W_LD][SUBG], wnz[W_LD][SUBG];     // scale and -(zero*scale) of the current tile's groups, per owned column

  auto load_a = [&](int step) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, ch = c & 7;
      const int m = m0 + row;
      v4u v = {0u, 0u, 0u, 0u};
      if (m < p.M) v = *reinterpret_cast<const v4u*>(p.a + (int64_t)m * p.lda + step * PF_BK + ch * 8);
      areg[i] = v;
    }
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, ch = c & 7;
      *reinterpret_cast<v4u*>(As + ((size_t)buf * BM + row) * PF_PITCH + ch * 8) = areg[i];
    }
  };
  auto load_w = [&](int g) {
#pragma unroll
    for (int i = 0; i < W_LD; ++i) {
      const int ntl = i * 4 + wave;
      const int nt = nt0 + ntl;
      v4u v = {0u, 0u, 0u, 0u};
      if (nt < p.NT) v = p.b[((int64_t)nt * p.G + g) * 64 + lane];
      wreg[i] = v;
#pragma unroll
      for (int sj = 0; sj < SUBG; ++sj) {
        float s = 0.f, z = 8.f;
        if (nt < p.NT) {
          const int n = nt * 16 + (lane & 15);
          const int64_t row = (int64_t)g * SUBG + sj;
          s = T::to_float(p.scales[row * p.s_stride + n]);
          if constexpr (HAS_ZP) {
            const uint32_t zw = p.zeros[row * p.z_stride + (n >> 3)];
            z = (float)((zw >> ((n & 7) * 4)) & 0xFu);
          }
        }
        ws[i][sj] = s;
        wnz[i][sj] = -(z * s);   // exact: <= 4 + 11 significant bits
      }
    }
  };
  auto store_w = [&](int buf, int half) {
    const int o = lane >> 4, r = lane & 15;
#pragma unroll
    for (int i = 0; i < W_LD; ++i) {
      const int ntl = i * 4 + wave;
      const uint32_t w0 = half ? wreg[i].z : wreg[i].x;
      const uint32_t w1 = half ? wreg[i].w : wreg[i].y;
      uint16_t* rowp = Bs + ((size_t)buf * BN + ntl * 16 + r) * PF_PITCH + o * 8;
      *reinterpret_cast<v4u*>(rowp) = dequant_scaled<BF16>(w0, pick_sub<SUBG>(ws[i], half * 2), pick_sub<SUBG>(wnz[i], half * 2));
      *reinterpret_cast<v4u*>(rowp + 32) =
          dequant_scaled<BF16>(w1, pick_sub<SUBG>(ws[i], half * 2 + 1), pick_sub<SUBG>(wnz[i], half * 2 + 1));
    }
  };

  v16f acc[WMB][WNB];
#pragma unroll
  for (int i = 0; i < WMB; ++i)
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int steps = p.K / PF_BK;

  // ---- prologue: stage step 0, issue loads for step 1 ----
  load_a(0);
  load_w(0);
  store_a(0);
  store_w(0, 0);
  if (steps > 1) load_a(1);
  __syncthreads();

  for (int step = 0; step < steps; ++step) {
    const int cur = step & 1;
    // stage step+1 into the other buffer
    if (step + 1 < steps) {
      const int nstep = step + 1;
      store_a(cur ^ 1);
      store_w(cur ^ 1, nstep & 1);
      if (nstep + 1 < steps) {
        load_a(nstep + 1);
        if (nstep & 1) load_w((nstep + 1) >> 1);   // both halves of the group consumed: fetch the next group
      }
    }
    // MFMAs of this step
    const uint16_t* Ab = As + ((size_t)cur * BM + wm * 32 * WMB + (lane & 31)) * PF_PITCH + (lane >> 5) * 8;
    const uint16_t* Bb = Bs + ((size_t)cur * BN + wn * 32 * WNB + (lane & 31)) * PF_PITCH + (lane >> 5) * 8;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      v4u af[WMB], bf[WNB];
#pragma unroll
      for (int i = 0; i < WMB; ++i) af[i] = *reinterpret_cast<const v4u*>(Ab + (size_t)i * 32 * PF_PITCH + kk * 16);
#pragma unroll
      for (int j = 0; j < WNB; ++j) bf[j] = *reinterpret_cast<const v4u*>(Bb + (size_t)j * 32 * PF_PITCH + kk * 16);
#pragma unroll
      for (int i = 0; i < WMB; ++i)
#pragma unroll
        for (int j = 0; j < WNB; ++j) acc[i][j] = T::mfma32(af[i], bf[j], acc[i][j]);
    }
    __syncthreads();
  }

  // ---- epilogue: lane holds column n = lane%32, rows 8*(e/4) + 4*(lane/32) + e%4 of each 32x32 block ----
#pragma unroll
  for (int j = 0; j < WNB; ++j) {
    const int n = n0 + wn * 32 * WNB + j * 32 + (lane & 31);
    if (n >= p.N) continue;
    float bv = 0.f;
    if (p.bias) bv = T::to_float(p.bias[n]);
#pragma unroll
    for (int i = 0; i < WMB; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * 32 * WMB + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (m < p.M) p.c[(int64_t)m * p.N + n] = T::from_float(acc[i][j][e] + bv);
      }
    }
  }
}

// The tail of a tile kernel: (split K) hand the partial tile over and let one wavefront sum (tile_handover.h), then bias,
// rounding and the stores.  `acc[i][j]` = 32 x 32 block (i along m, j along n) of this wavefront's TM x TN part of the
// tile at (m0 + wm * TM, n0 + wn * TN), in the layout of an MFMA whose A operand held the weights: lane = column m, four
// consecutive registers = four consecutive n.  `sl` = the workgroup's (tile, K part); `lds8` = at least
// NW * 32 * (TN * 2 + 16) bytes of LDS that every wavefront is done with.
template <bool BF16, int WMB, int WNB, int NW, int TM, int TN>
static __device__ inline void tile_epilogue(const PrefillParams& p, v16f (&acc)[WMB][WNB], uint8_t* lds8, const TileSlot& sl,
                                            int wave, int lane, int m0, int n0, int wm, int wn) {
  using T = F16Traits<BF16>;
  if (sl.nsplit > 1 && !handover_finish<WMB, WNB, NW>(p.c_tmp, p.counters, acc, sl, wave, lane)) return;

  // ---- epilogue: four consecutive accumulator registers = four consecutive n of one row.  The 16-bit results cross a
  // wavefront-private piece of LDS (32 rows of TN * 2 + 16 bytes, the operand stages being free by now) and leave as
  // 16-byte stores, 4-16 lanes to a row: stored directly, every instruction touches 32 rows with 16 bytes each, and
  // the write requests of a device whose tiles all finish together took 10-17 us per tile. ----
  if (((uintptr_t)p.c & 15) == 0) {
    constexpr int PITCH = TN * 2 + 16;
    constexpr int CPR = TN / 8;                // 16-byte chunks per row
    static_assert((32 * CPR) % 64 == 0, "whole store instructions");
    uint8_t* wave_lds = lds8 + wave * (32 * PITCH);
    v2u bv[WNB][4];
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * TN + j * 32 + 8 * q + 4 * (lane >> 5);
        bv[j][q] = v2u{0u, 0u};
        if (p.bias && n < p.N) bv[j][q] = *reinterpret_cast<const v2u*>(p.bias + n);
      }
#pragma unroll
    for (int i = 0; i < WMB; ++i) {
#pragma unroll
      for (int j = 0; j < WNB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float ov[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) ov[e] = acc[i][j][4 * q + e];
          if (p.bias) {
            ov[0] += T::to_float((uint16_t)(bv[j][q].x & 0xffffu));
            ov[1] += T::to_float((uint16_t)(bv[j][q].x >> 16));
            ov[2] += T::to_float((uint16_t)(bv[j][q].y & 0xffffu));
            ov[3] += T::to_float((uint16_t)(bv[j][q].y >> 16));
          }
          v2u pk;
          pk.x = pack2<BF16>(ov[0], ov[1]);
          pk.y = pack2<BF16>(ov[2], ov[3]);
          *reinterpret_cast<v2u*>(wave_lds + (lane & 31) * PITCH + (j * 32 + 8 * q + 4 * (lane >> 5)) * 2) = pk;
        }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();         // lanes exchange data through LDS; its operations run in program order
#pragma unroll
      for (int it = 0; it < 32 * CPR / 64; ++it) {
        const int idx = it * 64 + lane;
        const int row = idx / CPR, ch = idx % CPR;
        const v4u v = *reinterpret_cast<const v4u*>(wave_lds + row * PITCH + ch * 16);
        const int m = m0 + wm * TM + i * 32 + row;
        const int n = n0 + wn * TN + ch * 8;
        if (m < p.M && n < p.N) *reinterpret_cast<v4u*>(p.c + (int64_t)m * p.N + n) = v;
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < WMB; ++i) {
    const int m = m0 + wm * TM + i * 32 + (lane & 31);
    if (m >= p.M) continue;
    uint16_t* orow = p.c + (int64_t)m * p.N;
#pragma unroll
    for (int j = 0; j < WNB; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * TN + j * 32 + 8 * q + 4 * (lane >> 5);
        if (n >= p.N) continue;
        float ov[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = acc[i][j][4 * q + e];
        if (p.bias) {
          const v2u bb = *reinterpret_cast<const v2u*>(p.bias + n);
          ov[0] += T::to_float((uint16_t)(bb.x & 0xffffu));
          ov[1] += T::to_float((uint16_t)(bb.x >> 16));
          ov[2] += T::to_float((uint16_t)(bb.y & 0xffffu));
          ov[3] += T::to_float((uint16_t)(bb.y >> 16));
        }
        v2u pk;
        pk.x = pack2<BF16>(ov[0], ov[1]);
        pk.y = pack2<BF16>(ov[2], ov[3]);
        *reinterpret_cast<v2u*>(orow + n) = pk;
      }
    }
  }
}

// ----------------------------------------------------------------------------- direct-to-LDS variant
// Same arithmetic, different plumbing:
//  * the activation tile goes global -> LDS with `buffer_load_dwordx4 ... lds` (no registers, no VALU);
//  * LDS tiles are unpadded: a pair of 128-byte rows is one 256-byte line of 16 chunks (16 B each, chunk index
//    (row & 1) * 8 + c), and the chunk index is XOR-ed with (row >> 1) & 15.  The LDS of this architecture has 64 banks
//    (256 bytes per cycle): 16 lanes that touch 16 consecutive rows at the same k chunk -- the operand reads and the
//    dequantised-weight writes -- then hit 16 different 16-byte bank groups, and so do the 16 lanes of a DMA line;
//  * WAVES_M x WAVES_N wavefronts per workgroup (8 = two per SIMD lets one wavefront dequantise while the other one
//    issues MFMAs);
//  * the MFMAs take the weight fragment as A operand, so four consecutive accumulator registers are four consecutive
//    output columns of one row: 8 bytes per lane into the epilogue's LDS staging (16-byte global stores from there);
//  * weight words of group g+1 are requested one K step before they are needed (two register sets, by group parity).
template <bool BF16, int BM, int BN, int WAVES_M, int WAVES_N, bool HAS_ZP, int SUBG, int WT = 0, bool PP = false>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void w4a16_prefill2_kernel(const PrefillParams p) {
  using T = F16Traits<BF16>;
  constexpr bool W8 = WT != 0;      // two 1 KiB blocks per tile: nibble planes of 8-bit codes (WT = 1) or FP8 e4m3 bytes (WT = 2)
  constexpr bool F8 = WT == 2;
  static_assert(!F8 || SUBG == 1, "FP8 weights: channelwise scales or groups of 128 rows");
  static_assert(!PP || (!W8 && SUBG == 1 && (BM / (8 * WAVES_M * WAVES_N)) % 2 == 0 && WAVES_M * WAVES_N == 8),
                "alternating phases: 8 wavefronts, groups of 128 rows, an even number of DMA instructions per step");
  static_assert(!W8 || !HAS_ZP, "8-bit codes: symmetric");
  constexpr int TPG = W8 ? 2 : 1;                 // 1 KiB weight blocks per tile (8-bit: high-nibble plane, low-nibble plane)
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;
  constexpr int WMB = TM / 32, WNB = TN / 32;
  constexpr int W_LD = BN / (16 * NW);            // 16-byte weight loads per thread per group
  constexpr int A_LD = BM / (8 * NW);             // direct-to-LDS instructions per wavefront per step
  constexpr int A_ST = BM * 128, W_ST = BN * 128; // bytes per activation / weight stage
  constexpr int W_BASE = 3 * A_ST;                // three activation stages, then two weight stages
  constexpr int KW = W_LD * (TPG + SUBG * (HAS_ZP ? 2 : 1));   // vector-memory instructions of one load_w
  static_assert(W_LD >= 1 && A_LD >= 1, "tile too small for this many wavefronts");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds8[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  const TileSlot sl = tile_slot(total, p.SK, p.tail_first);          // one contiguous range of tile positions per XCD
  const int t = sl.pos;
  constexpr int GM = 4;                                              // tiles are handed out in bands of 4 tile rows (2 .. 16
                                                                     // measured: 1-3 % ahead of 8 on the large shapes), so
  const int band = t / (GM * tiles_n);                               // that the tiles resident on one XCD share
  const int first_m = band * GM;                                     // activation rows and weight columns in its L2
  const int gsz = min(tiles_m - first_m, GM);
  const int tin = t - band * GM * tiles_n;
  const int tm = first_m + tin % gsz, tn = tin / gsz;
  const int m0 = tm * BM, n0 = tn * BN, nt0 = n0 / 16;

  // ---- activation tile: direct-to-LDS loads ----
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.a), 0, (int)((uint32_t)p.M * (uint32_t)p.lda * 2u), 0x00020000);
  // DMA instruction i of this wavefront fills rows r0 .. r0+7 (r0 = (wave*A_LD + i) * 8): lane l lands in LDS slot
  // r0*8 + l, i.e. row pair j = r0/2 + (l >> 4), swizzled chunk l & 15; it must therefore fetch the element that
  // belongs there: c16 = (l & 15) ^ (j & 15), row = 2j + (c16 >> 3), chunk = c16 & 7.
  uint32_t voff_a[A_LD];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int j = (wave * A_LD + i) * 4 + (lane >> 4);
    const int c16 = (lane & 15) ^ (j & 15);
    const int lrow = 2 * (lane >> 4) + (c16 >> 3);
    voff_a[i] = ((uint32_t)lrow * (uint32_t)p.lda) * 2u + (uint32_t)(c16 & 7) * 16u;
  }
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto issue_a = [&](int step, int buf) {
    uint8_t* Ab = lds8 + (size_t)buf * A_ST;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int r0 = (wave * A_LD + i) * 8;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(Ab + r0 * 128), 16, (int)voff_a[i],
                                               (int)(((uint32_t)(m0 + r0) * (uint32_t)p.lda + (uint32_t)step * 64u) * 2u), 0, 0);
    }
  };

  // ---- weight words: the group being dequantised (cur) and the next one in flight (nxt).  Two named sets with a
  // register copy per group, not one array indexed by the group's parity: a run-time index into a register array turns
  // every access into a select chain, and the loads would have to be waited for as soon as they are issued. ----
  v4u wcur[W_LD], wnxt[W_LD];
  v4u wcur_lo[W8 ? W_LD : 1], wnxt_lo[W8 ? W_LD : 1];      // 8-bit codes: the low-nibble plane (wcur / wnxt hold the high one)
  // scales, and for one group per tile -(zero * scale); with several groups per tile the zero points stay packed as one
  // byte per group (registers are short here) and the product is formed where it is used
  using ZT = std::conditional_t<SUBG == 1, float, uint32_t>;
  float scur[W_LD][SUBG];
  ZT zcur[W_LD];
  constexpr bool HP = !BF16 && !W8 && SUBG == 1;      // packed fp16 dequantisation (see dequant_pair_h)
  uint32_t s2cur[HP ? W_LD : 1], nzb2cur[HP ? W_LD : 1];
  // the next group's scales and zero-point words as loaded; converted in advance_w, a K step after the request (a
  // conversion next to the load makes the wavefront wait for the memory latency in the middle of the step)
  uint16_t snxt_raw[W_LD][SUBG];
  uint32_t znxt_raw[W_LD][SUBG];
  const int o = lane >> 4, r = lane & 15;
  auto load_w = [&](int g) {
#pragma unroll
    for (int i = 0; i < W_LD; ++i) {
      const int ntl = i * NW + wave;
      const int nt = min(nt0 + ntl, p.NT - 1);          // clamped: columns past N are computed but never stored
      wnxt[i] = p.b[(((int64_t)nt * p.G + g) * TPG) * 64 + lane];
      if constexpr (W8) wnxt_lo[i] = p.b[(((int64_t)nt * p.G + g) * TPG + 1) * 64 + lane];
      const int n = nt * 16 + r;
#pragma unroll
      for (int sj = 0; sj < SUBG; ++sj) {
        const int64_t row = (int64_t)g * SUBG + sj;
        snxt_raw[i][sj] = p.scales[row * p.s_stride + n];
        if constexpr (HAS_ZP) znxt_raw[i][sj] = p.zeros[row * p.z_stride + (n >> 3)];
        else znxt_raw[i][sj] = 0u;
      }
    }
  };
  auto advance_w = [&]() {
#pragma unroll
    for (int i = 0; i < W_LD; ++i) {
      wcur[i] = wnxt[i];
      if constexpr (W8) wcur_lo[i] = wnxt_lo[i];
      if constexpr (SUBG > 1) zcur[i] = 0u;
#pragma unroll
      for (int sj = 0; sj < SUBG; ++sj) {
        const float sv = T::to_float(snxt_raw[i][sj]);
        uint32_t zc = F8 ? 0u : (W8 ? 128u : 8u);
        if constexpr (HAS_ZP) zc = (znxt_raw[i][sj] >> ((r & 7) * 4)) & 0xFu;    // column n = 16 * tile + r
        scur[i][sj] = sv;
        if constexpr (HP) {
          const uint32_t sb = snxt_raw[i][sj], zb = 0xE400u | zc;       // -(1024 + zero) as fp16 bits
          s2cur[i] = sb | (sb << 16);
          nzb2cur[i] = zb | (zb << 16);
        }
        if constexpr (SUBG == 1) zcur[i] = -((float)zc * sv);   // exact: <= 4 + 11 significant bits
        else if constexpr (HAS_ZP) zcur[i] |= zc << (8 * sj);
      }
    }
  };
  // scale and -(zero * scale) for word j (0..3) of weight load i
  auto sub_vals = [&](int i, int j, float& sv, float& zv) {
    sv = pick_sub<SUBG>(scur[i], j);
    if constexpr (SUBG == 1) {
      zv = zcur[i];
    } else if constexpr (HAS_ZP) {
      const int sj = (j * SUBG) >> 2;
      zv = -((float)((zcur[i] >> (8 * sj)) & 0xffu) * sv);
    } else {
      zv = -(F8 ? 0.f : (W8 ? 128.f : 8.f)) * sv;
    }
  };
  // Prologue only: dequantise half 0 of the current group into weight stage 0.
  auto store_w0 = [&]() {
    uint8_t* Bb = lds8 + W_BASE;
#pragma unroll
    for (int pc = 0; pc < 2 * W_LD; ++pc) {
      const int i = pc >> 1, which = pc & 1;
      const int row = (i * NW + wave) * 16 + r;
      const uint32_t wsel = which ? wcur[i].y : wcur[i].x;
      float sv, zv;
      sub_vals(i, which, sv, zv);
      const int c0 = (row & 1) * 8 + o + which * 4, sw = (row >> 1) & 15;
      v4u dv;
      if constexpr (F8) dv = dequant_fp8<BF16>(which ? wcur[i].z : wcur[i].x, which ? wcur[i].w : wcur[i].y, sv);      // block 0: words of j = 0, 1
      else if constexpr (W8) dv = dequant_scaled8<BF16>(wsel, which ? wcur_lo[i].y : wcur_lo[i].x, sv, zv);
      else if constexpr (HP) dv = dequant_scaled_h(wsel, s2cur[i], nzb2cur[i]);
      else dv = dequant_scaled<BF16>(wsel, sv, zv);
      *reinterpret_cast<v4u*>(Bb + (row >> 1) * 256 + ((c0 ^ sw) * 16)) = dv;
    }
  };
  auto issue_a_one = [&](int step, int buf, int i) {
    uint8_t* Ab = lds8 + (size_t)buf * A_ST;
    const int r0 = (wave * A_LD + i) * 8;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(Ab + r0 * 128), 16, (int)voff_a[i],
                                             (int)(((uint32_t)(m0 + r0) * (uint32_t)p.lda + (uint32_t)step * 64u) * 2u), 0, 0);
  };

  v16f acc[WMB][WNB];
#pragma unroll
  for (int i = 0; i < WMB; ++i)
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // operand reads: row = lane & 31 of a 32-row block (blocks start at multiples of 32 rows), chunk kk*2 + (lane >> 5)
  const int kh = lane >> 5;
  uint32_t coff[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
    coff[kk] = (uint32_t)(((lane & 31) >> 1) * 256 + ((((lane & 1) * 8 + kk * 2 + kh) ^ ((lane >> 1) & 15)) * 16));
  const uint32_t arow = (uint32_t)(wm * TM * 128);
  const uint32_t brow = (uint32_t)(wn * TN * 128);

  // One K step (64 wide = 4 MFMA k-slices) on activation stage `a_cur` and weight stage `w_cur`, fused with the staging
  // work for later steps: the DMA requests of the activation tile two steps ahead (into stage `a_dst`), and the
  // dequantisation of the next step's weights into the other weight stage.  The fragments of slice kk+1 are read
  // while the MFMAs of slice kk run; the staging work is cut into sub-steps that alternate with shares of the MFMAs
  // (sched_barrier keeps the compiler from regrouping them).
  auto fused_step = [&](int a_cur, int w_cur, auto stage_c, auto dma_c, int a_dst, int a_step, int half) {
    constexpr bool stage_on = decltype(stage_c)::value;
    constexpr bool dma_on = decltype(dma_c)::value;
    constexpr int NM = WMB * WNB;                    // MFMAs per slice
    constexpr int SUB = (NM % 4 == 0) ? 4 : 1;       // sub-steps per slice
    constexpr int PPS = (2 * W_LD + 3) / 4;          // dequantisation pieces per slice (at most)
    const uint8_t* base_a = lds8 + (size_t)a_cur * A_ST;
    const uint8_t* base_b = lds8 + W_BASE + (size_t)w_cur * W_ST;
    uint8_t* Bn = lds8 + W_BASE + (size_t)(w_cur ^ 1) * W_ST;
    if constexpr (dma_on) {
#pragma unroll
      for (int i = 0; i < A_LD; ++i) issue_a_one(a_step, a_dst, i);
    }
    v4u af[WMB], bf[2][WNB];     // weight fragments double-buffered, activation fragments refilled in place
#pragma unroll
    for (int i = 0; i < WMB; ++i) af[i] = *reinterpret_cast<const v4u*>(base_a + arow + i * 4096 + coff[0]);
#pragma unroll
    for (int j = 0; j < WNB; ++j) bf[0][j] = *reinterpret_cast<const v4u*>(base_b + brow + j * 4096 + coff[0]);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int cb = kk & 1, nb = cb ^ 1;
      v4u dq[PPS];
#pragma unroll
      for (int t = 0; t < SUB; ++t) {
        // a share of this slice's MFMAs
#pragma unroll
        for (int q = t * (NM / SUB); q < (t + 1) * (NM / SUB); ++q) {
          const int i = q / WNB, j = q % WNB;
          acc[i][j] = T::mfma32(bf[cb][j], af[i], acc[i][j]);   // rows = n, columns = m
        }
        // a share of the fragment reads of the next slice
        if (kk < 3) {
#pragma unroll
          for (int i = 0; i < WMB; ++i) {
            // activation fragment i has just had its last use in this slice: refill it in place
            const int last_q = i * WNB + WNB - 1;
            if (last_q >= t * (NM / SUB) && last_q < (t + 1) * (NM / SUB))
              af[i] = *reinterpret_cast<const v4u*>(base_a + arow + i * 4096 + coff[kk + 1]);
          }
#pragma unroll
          for (int j = 0; j < WNB; ++j)
            if (j % SUB == t) bf[nb][j] = *reinterpret_cast<const v4u*>(base_b + brow + j * 4096 + coff[kk + 1]);
        }
        // a share of the dequantisation
        if constexpr (stage_on) {
#pragma unroll
          for (int pc = 0; pc < 2 * W_LD; ++pc) {
            if (pc * 4 / (2 * W_LD) != kk) continue;
            const int slot = pc % PPS;
            const int i = pc >> 1, which = pc & 1;
            const uint32_t wsel = half ? (which ? wcur[i].w : wcur[i].z) : (which ? wcur[i].y : wcur[i].x);
            float sv, zv;
            sub_vals(i, half * 2 + which, sv, zv);
            if constexpr (F8) {
              // piece j = 2 * half + which: block `half` of the tile, words 2 * which and 2 * which + 1
              const uint32_t wa = half ? (which ? wcur_lo[i].z : wcur_lo[i].x) : (which ? wcur[i].z : wcur[i].x);
              const uint32_t wb = half ? (which ? wcur_lo[i].w : wcur_lo[i].y) : (which ? wcur[i].w : wcur[i].y);
              if constexpr (SUB == 4) dq[slot][t] = dequant_fp8_part<BF16>(wa, wb, sv, t);
              else dq[slot] = dequant_fp8<BF16>(wa, wb, sv);
            } else if constexpr (W8) {
              const uint32_t wlo = half ? (which ? wcur_lo[i].w : wcur_lo[i].z) : (which ? wcur_lo[i].y : wcur_lo[i].x);
              if constexpr (SUB == 4) dq[slot][t] = dequant_part8<BF16>(wsel, wlo, sv, zv, t);
              else dq[slot] = dequant_scaled8<BF16>(wsel, wlo, sv, zv);
            } else if constexpr (HP) {
              if constexpr (SUB == 4) dq[slot][t] = dequant_pair_h(wsel, s2cur[i], nzb2cur[i], t);
              else dq[slot] = dequant_scaled_h(wsel, s2cur[i], nzb2cur[i]);
            } else if constexpr (SUB == 4) {
              dq[slot][t] = dequant_part<BF16>(wsel, sv, zv, t);
            } else {
              dq[slot] = dequant_scaled<BF16>(wsel, sv, zv);
            }
            if (t == SUB - 1) {
              const int row = (i * NW + wave) * 16 + r;
              const int c0 = (row & 1) * 8 + o + which * 4, sw = (row >> 1) & 15;
              *reinterpret_cast<v4u*>(Bn + (row >> 1) * 256 + ((c0 ^ sw) * 16)) = dq[slot];
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // Vector-memory operations retire in issue order.  At the end of step s the activation tile of step s+1 (requested
  // during step s-1) must have landed, while the requests made during step s -- the tile of step s+2 and, on even
  // steps, the next group's weight words -- may stay in flight: wait until at most that many are outstanding.
  using TT = std::true_type;
  using FF = std::false_type;

  // K may be split over workgroups: this one covers the groups [g_lo, g_hi)
  const int g_lo = (int)(((int64_t)p.G * sl.split) / sl.nsplit), g_hi = (int)(((int64_t)p.G * (sl.split + 1)) / sl.nsplit);

  // ---- prologue: activation tiles of the first two steps, weights of the first step (group g_lo, half 0) ----
  issue_a(2 * g_lo, 0);
  issue_a(2 * g_lo + 1, 1);
  load_w(g_lo);
  advance_w();
  store_w0();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  int a_cur = 0;                      // activation stage of the current step (step mod 3)
  auto nxt = [](int x) { return x == 2 ? 0 : x + 1; };
  // LDS writes of this wavefront done, requests older than the newest `n` landed, then the workgroup barrier.  (A
  // plain __syncthreads() carries a fence that drains every outstanding load.)
  auto sync_step = [&](auto n_c) {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(decltype(n_c)::value) : "memory");
  };
  if constexpr (PP) {
    // Alternating phases.  A K step is two half steps of two MFMA k-slices; a half step is a READ phase (this
    // wavefront's fragments of the two slices, its share of the DMA requests, the LDS writes of two dequantised weight
    // pieces) and an MFMA phase (16 MFMAs with the dequantisation of the next two pieces in their shadow: a wavefront's
    // LDS traffic and its VALU work do not overlap each other, but both overlap the other wavefront's MFMAs), each
    // ended by a workgroup barrier.  The wavefronts w and w + 4 share a SIMD; the second four pass one extra barrier
    // first (and skip their last one), so on every SIMD one wavefront is in its READ phase while the other one keeps
    // the matrix core busy.
    // Weight pieces for step t+1 (four per wavefront): 0,1 dequantised in MFMA phase (t-1, 1), written in READ phase
    // (t, 0); 2,3 dequantised in (t, 0), written in (t, 1).  The next group's words are requested a step and a half
    // before their first use and become current in the middle of the even step.
    // Hazards, with the late half one phase behind: a weight stage written during step t is first read two barriers
    // after its last write; the activation stage requested during step t was last read one barrier before the first
    // request; the tile of step t+1 has landed at the end of the second READ phase of step t of every wavefront, at
    // least one barrier before anyone reads it.
    const bool late = wave >= NW / 2;
    v4u af[2][WMB], bf[2][WNB];
    v4u dq[W_LD];
    // pieces h*W_LD .. of weight half `half` of the current group -> dq
    auto deq = [&](int half, auto h_c) {
      constexpr int h = decltype(h_c)::value;
#pragma unroll
      for (int x = 0; x < W_LD; ++x) {
        const int pc = h * W_LD + x;
        const int i = pc >> 1, which = pc & 1;
        const uint32_t wsel = half ? (which ? wcur[i].w : wcur[i].z) : (which ? wcur[i].y : wcur[i].x);
        float sv, zv;
        sub_vals(i, half * 2 + which, sv, zv);
        if constexpr (HP) dq[x] = dequant_scaled_h(wsel, s2cur[i], nzb2cur[i]);
        else dq[x] = dequant_scaled<BF16>(wsel, sv, zv);
      }
    };
    auto read_phase = [&](int a_cur, int w_cur, auto write_c, auto dma_c, int a_dst, int a_step, auto h_c) {
      constexpr bool write_on = decltype(write_c)::value;
      constexpr bool dma_on = decltype(dma_c)::value;
      constexpr int h = decltype(h_c)::value;
      const uint8_t* base_a = lds8 + (size_t)a_cur * A_ST;
      const uint8_t* base_b = lds8 + W_BASE + (size_t)w_cur * W_ST;
      uint8_t* Bn = lds8 + W_BASE + (size_t)(w_cur ^ 1) * W_ST;
      if constexpr (dma_on) {
#pragma unroll
        for (int i = h * (A_LD / 2); i < (h + 1) * (A_LD / 2); ++i) issue_a_one(a_step, a_dst, i);
      }
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2) {
#pragma unroll
        for (int j = 0; j < WNB; ++j) bf[k2][j] = *reinterpret_cast<const v4u*>(base_b + brow + j * 4096 + coff[2 * h + k2]);
#pragma unroll
        for (int i = 0; i < WMB; ++i) af[k2][i] = *reinterpret_cast<const v4u*>(base_a + arow + i * 4096 + coff[2 * h + k2]);
      }
      if constexpr (write_on) {
        __builtin_amdgcn_sched_barrier(0);        // the writes stay behind the reads (see sync_reads_only)
#pragma unroll
        for (int x = 0; x < W_LD; ++x) {
          const int pc = h * W_LD + x;
          const int i = pc >> 1, which = pc & 1;
          const int row = (i * NW + wave) * 16 + r;
          const int c0 = (row & 1) * 8 + o + which * 4, sw = (row >> 1) & 15;
          *reinterpret_cast<v4u*>(Bn + (row >> 1) * 256 + ((c0 ^ sw) * 16)) = dq[x];
        }
      }
    };
    auto mfma_phase = [&](auto deq_c, int half, auto h_c) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
        for (int i = 0; i < WMB; ++i)
#pragma unroll
          for (int j = 0; j < WNB; ++j) acc[i][j] = T::mfma32(bf[k2][j], af[k2][i], acc[i][j]);   // rows = n, columns = m
      if constexpr (decltype(deq_c)::value) {
        deq(half, h_c);
#pragma unroll
        for (int x = 0; x < 2 * WMB * WNB; ++x) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);     // three VALU instructions in its shadow
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    auto bare_barrier = [&]() { asm volatile("s_barrier" ::: "memory"); };
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    using LGKM_ONLY = std::integral_constant<int, 63>;     // no vector-memory wait in the first half of a step
    // End of the first READ phase of a step: the fragment reads are complete, the W_LD piece writes issued after them
    // may still be queued (LDS operations complete in order); they are waited for at the end of the step's second READ
    // phase, a barrier before the stage they fill is read.
    auto sync_reads_only = [&]() {
      asm volatile("s_waitcnt lgkmcnt(%0)\n\ts_barrier" ::"n"(W_LD) : "memory");
    };
    // (prologue, continued) the next group's words; pieces 0,1 of (g_lo, half 1)
    if (g_lo + 1 < g_hi) load_w(g_lo + 1);
    deq(1, H0{});
    if (late) bare_barrier();
    for (int g = g_lo; g + 1 < g_hi; ++g) {
      // even step 2g reads weight stage 0 and fills stage 1 with (g, half 1); requests the tile of step 2g+2
      read_phase(a_cur, 0, TT{}, TT{}, nxt(nxt(a_cur)), 2 * g + 2, H0{});
      sync_reads_only();
      mfma_phase(TT{}, 1, H1{});                     // pieces 2,3 of (g, half 1)
      bare_barrier();
      read_phase(a_cur, 0, TT{}, TT{}, nxt(nxt(a_cur)), 2 * g + 2, H1{});
      sync_step(std::integral_constant<int, A_LD>{});
      advance_w();                                   // group g+1 becomes current
      mfma_phase(TT{}, 0, H0{});                     // pieces 0,1 of (g+1, half 0)
      bare_barrier();
      a_cur = nxt(a_cur);
      // odd step 2g+1 reads stage 1 and fills stage 0 with (g+1, half 0); requests the tile of step 2g+3 and the words
      // of group g+2 (clamped at the end of this workgroup's range: a repeated load keeps the wait counts uniform)
      load_w(min(g + 2, g_hi - 1));
      read_phase(a_cur, 1, TT{}, TT{}, nxt(nxt(a_cur)), 2 * g + 3, H0{});
      sync_reads_only();
      mfma_phase(TT{}, 0, H1{});                     // pieces 2,3 of (g+1, half 0)
      bare_barrier();
      read_phase(a_cur, 1, TT{}, TT{}, nxt(nxt(a_cur)), 2 * g + 3, H1{});
      sync_step(std::integral_constant<int, A_LD + KW>{});
      mfma_phase(TT{}, 1, H0{});                     // pieces 0,1 of (g+1, half 1)
      bare_barrier();
      a_cur = nxt(a_cur);
    }
    // last group: its second half is still dequantised, nothing is requested any more
    read_phase(a_cur, 0, TT{}, FF{}, 0, 0, H0{});
    sync_reads_only();
    mfma_phase(TT{}, 1, H1{});
    bare_barrier();
    read_phase(a_cur, 0, TT{}, FF{}, 0, 0, H1{});
    sync_step(std::integral_constant<int, 0>{});
    mfma_phase(FF{}, 0, H0{});
    bare_barrier();
    a_cur = nxt(a_cur);
    read_phase(a_cur, 1, FF{}, FF{}, 0, 0, H0{});
    sync_step(LGKM_ONLY{});
    mfma_phase(FF{}, 0, H0{});
    bare_barrier();
    read_phase(a_cur, 1, FF{}, FF{}, 0, 0, H1{});
    sync_step(LGKM_ONLY{});
    mfma_phase(FF{}, 0, H0{});
    if (!late) bare_barrier();
  } else {
  for (int g = g_lo; g + 1 < g_hi; ++g) {
    // even step 2g: dequantise (g, half 1) for step 2g+1; request the tile of step 2g+2 and the words of group g+1
    load_w(g + 1);
    fused_step(a_cur, 0, TT{}, TT{}, nxt(nxt(a_cur)), 2 * g + 2, 1);
    sync_step(std::integral_constant<int, A_LD + KW>{});
    a_cur = nxt(a_cur);
    // odd step 2g+1: dequantise (g+1, half 0) for step 2g+2; request the tile of step 2g+3
    advance_w();
    fused_step(a_cur, 1, TT{}, TT{}, nxt(nxt(a_cur)), 2 * g + 3, 0);
    sync_step(std::integral_constant<int, A_LD>{});
    a_cur = nxt(a_cur);
  }
  // last group: its second half is still dequantised, nothing is requested any more
  fused_step(a_cur, 0, TT{}, FF{}, 0, 0, 1);
  sync_step(std::integral_constant<int, 0>{});
  a_cur = nxt(a_cur);
  fused_step(a_cur, 1, FF{}, FF{}, 0, 0, 0);
  }
  // every wavefront is done with the operand stages: the epilogue reuses them
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  static_assert((3 * BM + 2 * BN) * 128 >= NW * 32 * (TN * 2 + 16), "operand stages too small for the epilogue staging");
  tile_epilogue<BF16, WMB, WNB, NW, TM, TN>(p, acc, lds8, sl, wave, lane, m0, n0, wm, wn);
}

template <bool BF16, int WMB, int WNB, bool HAS_ZP, int SUBG>
static int launch_prefill(const PrefillParams& p, hipStream_t s) {
  constexpr int BM = 64 * WMB, BN = 64 * WNB;
  const size_t lds = (size_t)2 * (BM + BN) * PF_PITCH * sizeof(uint16_t);
  auto kern = w4a16_prefill_kernel<BF16, WMB, WNB, HAS_ZP, SUBG>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (const int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "w4a16_gemm(prefill)"); rc != VAQ_OK) return rc;
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(256), lds, s, p);
  return VAQ_OK;
}

template <bool BF16, int BM, int BN, int WAVES_M, int WAVES_N, bool HAS_ZP, int SUBG, int WT = 0, bool PP = false>
static int launch_prefill2(const PrefillParams& p, hipStream_t s) {
  const size_t lds = (size_t)(3 * BM + 2 * BN) * 128;
  auto kern = w4a16_prefill2_kernel<BF16, BM, BN, WAVES_M, WAVES_N, HAS_ZP, SUBG, WT, PP>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (const int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "w4a16_gemm(prefill)"); rc != VAQ_OK) return rc;
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  const dim3 grid = p.tail_first > 0 ? dim3(p.tail_first + (tiles - p.tail_first) * p.SK) : dim3(tiles, p.SK);
  hipLaunchKernelGGL(kern, grid, dim3(WAVES_M * WAVES_N * 64), lds, s, p);
  return VAQ_OK;
}

// Groups of 64 / 32 rows (sub = 2 / 4 per tile); defined in w4a16_prefill_sub.hip for the tile ids the automatic choice
// uses (10, 12, 14, 15 and 0, 1, 2).
int prefill_launch_sub(const PrefillParams& p, int sub, int tile, bool bf16, bool zp, hipStream_t s);
// 8-bit codes; defined in w4a16_prefill_w8.hip for the direct-to-LDS tile ids 10, 12, 14, 15 (sub = 1, 2 or 4 groups per
// 128 rows).
int prefill_launch_w8(const PrefillParams& p, int sub, int tile, bool bf16, hipStream_t s);
// FP8 e4m3 weights (bytes), channelwise scales or groups of 128 rows; defined in w4a16_prefill_f8.hip (tile ids 10, 12, 14, 15)
int prefill_launch_f8(const PrefillParams& p, int tile, bool bf16, hipStream_t s);

}  // namespace vaq
