// W4A16 decode-shaped GEMM (M <= 32) for gfx950: C[M,N] = A[M,K] . dequant(B[K,N]) (+bias).
//
// Memory-bound: the job is to stream K*N/2 bytes of packed int4 once, at HBM speed, with as little VALU work per
// byte as possible.  Design:
//
//  * Weights arrive in the NATIVE tile order (see w4a16_repack.hip): one 16-byte load per lane = one 1 KiB
//    wavefront load = a 16(n) x 128(k) tile = the A operands of four v_mfma_f32_16x16x32 and exactly one
//    quantisation group.
//  * The weights are the MFMA *A* operand (rows = n), the activations the *B* operand (columns = m), so the cost per
//    weight byte does not depend on M (up to 16 per m-block) and the matrix pipe does all multiply-adds.
//  * Dequantisation is 7 VALU ops per 8 codes: `(w >> 4i) & 0x000f000f | EX` yields the 16-bit numbers BIAS + code
//    (BIAS = 128 for bf16, 1024 for fp16).  The "- BIAS - zero" and the group scale are NOT applied per element:
//        C[m,n] = sum_g s[g,n] * ( P_g[m,n] - (BIAS + z[g,n]) * S_g[m] ),
//        P_g[m,n] = sum_{k in g} a[m,k] * (BIAS + code[k,n])      (4 MFMAs, fp32)
//        S_g[m]   = sum_{k in g} a[m,k]                           (MFMA against an all-ones operand, once per wave)
//    which costs two fp32 FMAs per output per group.  The products a*(BIAS+code) are exact in fp32 and the group
//    scale is applied in fp32, so the result is at least as accurate as scaling every weight in 16 bits first.
//  * Each wavefront owns a fixed slab of TG groups along K, keeps the matching activations in registers for the
//    whole kernel (loaded once; act_order gathers through `perm` here, so no permuted copy of A is needed) and walks
//    a contiguous range of n-tiles, prefetching the next TG tiles while the current ones are consumed.
//  * The WK wavefronts of a workgroup cover WK*TG groups of the same n-tile and reduce through LDS (one barrier per
//    n-tile, double-buffered).  If K needs more than one workgroup (SK > 1) the partial tiles go to `c_tmp` and the
//    last workgroup to arrive at a per-tile counter sums them in a fixed order (deterministic) and resets the counter.
#include "vaq_common.h"

namespace vaq {

struct DecodeParams {
  const uint16_t* a;
  int64_t lda;
  const v4u* b;
  const uint16_t* scales;
  const uint32_t* zeros;
  const int32_t* perm;
  const uint16_t* bias;
  uint16_t* c;
  v4f* c_tmp;
  int32_t* counters;
  int M, N, K, G, NT, SK, WK;
  int GR, s_stride, z_stride;   // rows of scales / zeros and the element strides between them (1 row, strides 0: channelwise)
  uint32_t k_mask, k_ex;   // 0x000f000f and the exponent pattern, passed as run-time values (see and_or)
};

// Split-K partial tiles cross workgroups (and therefore XCDs, whose L2 caches are not coherent with each other)
// through 16-byte buffer stores and loads with the sc1 cache-policy bit (device scope): no L2 write-back / invalidate is
// needed, only a wait for the stores to be acknowledged before the arrival counter is bumped.
constexpr int DEC_SC1 = 16;

// (x & mask) | ex.  mask and ex reach the kernel as run-time arguments: with literal constants the compiler emits two
// instructions (a VOP3 op of this architecture cannot carry two literals); with register operands it selects the
// single v_and_or_b32, and unlike inline assembly the instruction stays visible to the MFMA hazard recogniser.
__device__ inline uint32_t and_or(uint32_t x, uint32_t mask, uint32_t ex) { return (x & mask) | ex; }

template <bool BF16>
__device__ inline v4u dequant_biased_fast(uint32_t w, uint32_t M, uint32_t ex) {
  v4u r;
  r.x = and_or(w, M, ex);
  r.y = and_or(w >> 4, M, ex);
  r.z = and_or(w >> 8, M, ex);
  r.w = and_or(w >> 12, M, ex);
  return r;
}

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint64_t bytes) {
  const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}

// MAXW = upper bound on wavefronts per workgroup (8 leaves 256 registers per lane, 16 leaves 128).
// D    = n-tiles kept in flight per wavefront (prefetch depth of the register ring).
template <bool BF16, int TG, int MB, bool HAS_ZP, int MAXW, int D>
__global__ __launch_bounds__(MAXW * 64) void w4a16_decode_kernel(const DecodeParams p) {
  using T = F16Traits<BF16>;
  extern __shared__ v4f red[];   // [2][WK][MB][64]

  const int lane = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.y);   // wave-uniform: tile offsets stay in scalar registers
  const int o = lane >> 4, r16 = lane & 15;
  const int sk = blockIdx.y;
  const int g0 = (sk * p.WK + w) * TG;

  // ---- contiguous range of n-tiles for this workgroup ----
  const int nt0 = (int)(((int64_t)p.NT * blockIdx.x) / gridDim.x);
  const int nt1 = (int)(((int64_t)p.NT * (blockIdx.x + 1)) / gridDim.x);

  // Weights, scales and zero points are read through buffer descriptors: the per-tile part of the address is a
  // scalar offset, the per-lane part a constant, so a load costs no vector ALU work.
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b, (uint64_t)p.K * p.N / 2);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.scales, (uint64_t)p.GR * p.N * 2);
  const __amdgpu_buffer_rsrc_t rz = make_rsrc(HAS_ZP ? (const void*)p.zeros : (const void*)p.scales, (uint64_t)p.GR * (p.N / 8) * 4);
  const int vo_b = lane * 16, vo_s = o * 8, vo_z = (o >> 1) * 4;

  v4u wq[D][TG];
  v2u sc[D][TG];
  uint32_t zq[D][TG];
  // Groups past the end of K (ragged last wavefront) are clamped for addressing; their activations are zero, so they
  // contribute nothing.
  uint32_t ob[TG], os_[TG], oz[TG];      // scalar byte offsets of this wavefront's groups at n-tile 0
#pragma unroll
  for (int t = 0; t < TG; ++t) {
    const uint32_t g = (uint32_t)min(g0 + t, p.G - 1);
    ob[t] = g * 1024u;
    os_[t] = g * (uint32_t)p.s_stride * 2u;
    oz[t] = g * (uint32_t)p.z_stride * 4u;
  }
  auto issue_load = [&](int u, int nt, int t) {
    wq[u][t] = __builtin_amdgcn_raw_buffer_load_b128(rb, vo_b, (int)(ob[t] + (uint32_t)nt * (uint32_t)p.G * 1024u), 2);
    sc[u][t] = __builtin_amdgcn_raw_buffer_load_b64(rs, vo_s, (int)(os_[t] + (uint32_t)nt * 32u), 0);
    if constexpr (HAS_ZP) zq[u][t] = __builtin_amdgcn_raw_buffer_load_b32(rz, vo_z, (int)(oz[t] + (uint32_t)nt * 8u), 0);
  };
  // ---- activations of this wave's K slab, as MFMA B operands (column = m, 8 consecutive k per lane) ----
  // Loaded unconditionally from clamped addresses and zeroed afterwards, so that all loads are in flight together.
  v4u breg[TG][4][MB];
  if (p.perm == nullptr) {
#pragma unroll
    for (int t = 0; t < TG; ++t) {
      const int g = min(g0 + t, p.G - 1);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = min(mb * 16 + r16, p.M - 1);
        const uint16_t* row = p.a + (int64_t)m * p.lda + g * 128 + o * 8;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) breg[t][jj][mb] = *reinterpret_cast<const v4u*>(row + jj * 32);
      }
    }
  } else {
#pragma unroll
    for (int t = 0; t < TG; ++t) {
      const int g = min(g0 + t, p.G - 1);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = min(mb * 16 + r16, p.M - 1);
        const uint16_t* row = p.a + (int64_t)m * p.lda;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int k = g * 128 + jj * 32 + o * 8;
          const v4i p0 = *reinterpret_cast<const v4i*>(p.perm + k);
          const v4i p1 = *reinterpret_cast<const v4i*>(p.perm + k + 4);
          v4u v;
          v.x = (uint32_t)row[p0.x] | ((uint32_t)row[p0.y] << 16);
          v.y = (uint32_t)row[p0.z] | ((uint32_t)row[p0.w] << 16);
          v.z = (uint32_t)row[p1.x] | ((uint32_t)row[p1.y] << 16);
          v.w = (uint32_t)row[p1.z] | ((uint32_t)row[p1.w] << 16);
          breg[t][jj][mb] = v;
        }
      }
    }
  }
  // The first weight tiles are requested right after the activation loads: loads retire in issue order as far as the
  // wait counter is concerned, so this order lets the wait for the activations leave the weight tiles in flight.
#pragma unroll
  for (int u = 0; u < D; ++u) {
#pragma unroll
    for (int t = 0; t < TG; ++t) {
      wq[u][t] = v4u{0u, 0u, 0u, 0u};
      sc[u][t] = v2u{0u, 0u};
      zq[u][t] = 0u;
    }
    if (nt0 + u < nt1) {
#pragma unroll
      for (int t = 0; t < TG; ++t) issue_load(u, nt0 + u, t);
    }
  }

  // S[t][mb] = sum of the group's activations per column m (identical in the 4 accumulator registers).  For the
  // symmetric type the whole correction -(BIAS + 8) * S is the starting value of the group's MFMA chain.
  v4f Sv[TG][MB];
#pragma unroll
  for (int t = 0; t < TG; ++t) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const bool ok = (g0 + t < p.G) && (mb * 16 + r16 < p.M);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
        if (!ok) breg[t][jj][mb] = v4u{0u, 0u, 0u, 0u};
      const v4u ones = {T::ONE2, T::ONE2, T::ONE2, T::ONE2};
      v4f s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) s4 = T::mfma16(ones, breg[t][jj][mb], s4);
      if constexpr (!HAS_ZP) s4 *= -(T::CODE_BIAS + 8.0f);
      Sv[t][mb] = s4;
    }
  }

  uint32_t ex;     // kept in a vector register so that (x & msk) | ex is a legal single VOP3 instruction (one scalar operand)
  asm volatile("v_mov_b32 %0, %1" : "=v"(ex) : "s"(p.k_ex));
  const uint32_t msk = p.k_mask;
  int parity = 0;
  int red_w = 0;      // wavefront that reduces m-block 0 of the current n-tile; advances by MB per n-tile (mod WK)
  for (int base = nt0; base < nt1; base += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int nt = base + u;
      if (nt >= nt1) break;

      v4f acc[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb] = v4f{0.f, 0.f, 0.f, 0.f};

#pragma unroll
      for (int t = 0; t < TG; ++t) {
        const uint32_t wj[4] = {wq[u][t].x, wq[u][t].y, wq[u][t].z, wq[u][t].w};
        const v2u sct = sc[u][t];
        const uint32_t zqt = zq[u][t];
        if (nt + D < nt1) issue_load(u, nt + D, t);      // refill this ring slot D n-tiles ahead
        v4f P[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) P[mb] = HAS_ZP ? v4f{0.f, 0.f, 0.f, 0.f} : Sv[t][mb];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const v4u aop = dequant_biased_fast<BF16>(wj[jj], msk, ex);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) P[mb] = T::mfma16(aop, breg[t][jj][mb], P[mb]);
        }
        // group epilogue: acc += s * (P - (BIAS + z) * S)   (the subtraction is already inside P when symmetric)
        float s[4];
        if constexpr (BF16) {
          s[0] = __uint_as_float(sct.x << 16);
          s[1] = __uint_as_float(sct.x & 0xffff0000u);
          s[2] = __uint_as_float(sct.y << 16);
          s[3] = __uint_as_float(sct.y & 0xffff0000u);
        } else {
          s[0] = T::to_float((uint16_t)(sct.x & 0xffffu));
          s[1] = T::to_float((uint16_t)(sct.x >> 16));
          s[2] = T::to_float((uint16_t)(sct.y & 0xffffu));
          s[3] = T::to_float((uint16_t)(sct.y >> 16));
        }
        if constexpr (HAS_ZP) {
          const uint32_t z4 = zqt >> ((o & 1) * 16);
          float zc[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) zc[r] = T::CODE_BIAS + (float)((z4 >> (4 * r)) & 0xFu);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mb][r] = fmaf(s[r], fmaf(-zc[r], Sv[t][mb][r], P[mb][r]), acc[mb][r]);
        } else {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mb][r] = fmaf(s[r], P[mb][r], acc[mb][r]);
        }
      }

      // ---- reduce the WK partial tiles of this workgroup through LDS; the reducing wavefront rotates ----
      int my_mb = -1;
      v4f tot = v4f{0.f, 0.f, 0.f, 0.f};
      if (p.WK > 1) {
        v4f* buf = red + (size_t)parity * p.WK * MB * 64;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) buf[(w * MB + mb) * 64 + lane] = acc[mb];
        __syncthreads();
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
        {
          int cand = red_w + mb;
          if (cand >= p.WK) cand -= p.WK;
          if (cand == w) my_mb = mb;
        }
        if (my_mb >= 0) {
          for (int ww = 0; ww < p.WK; ++ww) tot += buf[(ww * MB + my_mb) * 64 + lane];
        }
        parity ^= 1;
        red_w += MB;
        if (red_w >= p.WK) red_w -= p.WK;
      }

      const int mb_lo = (p.WK > 1) ? my_mb : 0;
      const int mb_hi = (p.WK > 1) ? my_mb + 1 : MB;
      if (p.WK == 1 || my_mb >= 0) {
        for (int mb = mb_lo; mb < mb_hi; ++mb) {
          v4f val = (p.WK > 1) ? tot : acc[mb];
          bool write_out = true;
          if (p.SK > 1) {
            const uint32_t unit = (uint32_t)(nt * MB + mb) * 1024u;                  // bytes
            const uint32_t sk_stride = (uint32_t)p.NT * (uint32_t)MB * 1024u;
            const __amdgpu_buffer_rsrc_t rt = make_rsrc(p.c_tmp, (uint64_t)sk_stride * (uint64_t)p.SK);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, val), rt, lane * 16,
                                                   (int)((uint32_t)sk * sk_stride + unit), DEC_SC1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // partial tile acknowledged before the counter moves
            int old = 0;
            if (lane == 0) old = __hip_atomic_fetch_add(&p.counters[nt * MB + mb], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old = __builtin_amdgcn_readfirstlane(old);      // lane 0 holds it; a scalar keeps what depends on it scalar
            write_out = (old == p.SK - 1);
            if (write_out) {
              val = v4f{0.f, 0.f, 0.f, 0.f};
              for (int s0 = 0; s0 < p.SK; s0 += 4) {             // four splits in flight, added in split order
                v4u part[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  part[i] = __builtin_amdgcn_raw_buffer_load_b128(rt, lane * 16,
                                                                  (int)((uint32_t)min(s0 + i, p.SK - 1) * sk_stride + unit), DEC_SC1);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  if (s0 + i < p.SK) val += __builtin_bit_cast(v4f, part[i]);
              }
              if (lane == 0) __hip_atomic_store(&p.counters[nt * MB + mb], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
          }
          const int m = mb * 16 + r16;
          if (write_out && m < p.M) {
            const int n = nt * 16 + o * 4;
            if (p.bias) {
              const v2u bb = *reinterpret_cast<const v2u*>(p.bias + n);
              val[0] += T::to_float((uint16_t)(bb.x & 0xffffu));
              val[1] += T::to_float((uint16_t)(bb.x >> 16));
              val[2] += T::to_float((uint16_t)(bb.y & 0xffffu));
              val[3] += T::to_float((uint16_t)(bb.y >> 16));
            }
            v2u outv;
            outv.x = (uint32_t)T::from_float(val[0]) | ((uint32_t)T::from_float(val[1]) << 16);
            outv.y = (uint32_t)T::from_float(val[2]) | ((uint32_t)T::from_float(val[3]) << 16);
            *reinterpret_cast<v2u*>(p.c + (int64_t)m * p.N + n) = outv;
          }
        }
      }
    }
  }
}

// ----------------------------------------------------------------------------- host side

struct DecodeConfig {
  int tg, wk, sk, gx, maxw, d;
};

// `wk` wavefronts of a workgroup x `sk` workgroups cover the K/128 groups, TG groups per wavefront.
static DecodeConfig pick_decode_config(int M, int N, int K) {
  const int G = K / 128, NT = N / 16;
  const int MB = M <= 16 ? 1 : 2;
  const VaqTuning& tn = tuning();
  DecodeConfig c;
  if (tn.decode_tg > 0) c.tg = tn.decode_tg;
  else if (MB == 2) c.tg = 1;
  else if (G % 7 == 0 && G >= 56) c.tg = 7;      // K = 14336: 7 groups per wavefront, 8 wavefronts, 2 workgroups
  else c.tg = G >= 2 ? 2 : 1;
  if (c.tg != 1 && c.tg != 2 && c.tg != 4 && c.tg != 7) c.tg = 2;
  if (MB == 2 && c.tg >= 4) c.tg = 2;
  const int kw = (G + c.tg - 1) / c.tg;          // wavefronts needed along K
  int wk_max = (c.tg >= 4 || (MB == 2 && c.tg == 2)) ? 8 : 16;
  c.maxw = wk_max > 8 ? 16 : 8;                  // the instantiated launch bound; fewer wavefronts may run under it
  if (tn.decode_wk > 0 && tn.decode_wk < wk_max) wk_max = tn.decode_wk;
  c.sk = (kw + wk_max - 1) / wk_max;
  c.wk = (kw + c.sk - 1) / c.sk;
  const int cus = num_cus_current_device();
  int gx = tn.decode_gx > 0 ? tn.decode_gx : cus / c.sk;
  if (gx < 1) gx = 1;
  if (gx > NT) gx = NT;
  c.gx = gx;
  const int per = (NT + gx - 1) / gx;           // n-tiles per workgroup
  c.d = tn.decode_depth > 0 ? tn.decode_depth : (per >= 2 ? 2 : 1);   // depth 3 spills in the 128-register shapes
  if (c.tg == 7) c.d = 1;
  if (c.d > 3) c.d = 3;
  if (c.d < 1) c.d = 1;
  return c;
}

template <bool BF16, int TG, int MB, bool HAS_ZP, int MAXW, int D>
static void launch_decode(const DecodeParams& p, int gx, hipStream_t s) {
  const size_t lds = p.WK > 1 ? (size_t)2 * p.WK * MB * 64 * sizeof(v4f) : 0;
  hipLaunchKernelGGL((w4a16_decode_kernel<BF16, TG, MB, HAS_ZP, MAXW, D>), dim3(gx, p.SK), dim3(64, p.WK), lds, s, p);
}

template <bool BF16, int TG, int MB, bool HAS_ZP, int MAXW>
static int dispatch_d(const DecodeParams& p, const DecodeConfig& c, hipStream_t s) {
  switch (c.d) {
    case 1: launch_decode<BF16, TG, MB, HAS_ZP, MAXW, 1>(p, c.gx, s); return VAQ_OK;
    case 2: launch_decode<BF16, TG, MB, HAS_ZP, MAXW, 2>(p, c.gx, s); return VAQ_OK;
    case 3: launch_decode<BF16, TG, MB, HAS_ZP, MAXW, 3>(p, c.gx, s); return VAQ_OK;
    default: break;
  }
  set_error("w4a16_gemm(decode): unsupported prefetch depth %d", c.d);
  return VAQ_ERR_UNSUPPORTED;
}

// Instantiated launch shapes: one m-block: (TG,MAXW) in {(1,16), (2,16), (4,8), (7,8; depth 1)}; two m-blocks: {(1,16), (2,8)}.
template <bool BF16, int MB, bool HAS_ZP>
static int dispatch_tg(const DecodeParams& p, const DecodeConfig& c, hipStream_t s) {
  if constexpr (MB == 1) {
    if (c.tg == 1 && c.maxw == 16) return dispatch_d<BF16, 1, 1, HAS_ZP, 16>(p, c, s);
    if (c.tg == 2 && c.maxw == 16) return dispatch_d<BF16, 2, 1, HAS_ZP, 16>(p, c, s);
    if (c.tg == 4 && c.maxw == 8) return dispatch_d<BF16, 4, 1, HAS_ZP, 8>(p, c, s);
    if (c.tg == 7 && c.maxw == 8) { launch_decode<BF16, 7, 1, HAS_ZP, 8, 1>(p, c.gx, s); return VAQ_OK; }
  } else {
    if (c.tg == 1 && c.maxw == 16) return dispatch_d<BF16, 1, 2, HAS_ZP, 16>(p, c, s);
    if (c.tg == 2 && c.maxw == 8) return dispatch_d<BF16, 2, 2, HAS_ZP, 8>(p, c, s);
  }
  set_error("w4a16_gemm(decode): unsupported launch shape TG=%d MAXW=%d for MB=%d", c.tg, c.maxw, MB);
  return VAQ_ERR_UNSUPPORTED;
}

// Called from vaq_w4a16_gemm (w4a16_gemm.hip) after argument validation.
int w4a16_decode_workspace(int M, int N, int K, size_t* c_tmp_bytes, size_t* counter_ints) {
  const DecodeConfig c = pick_decode_config(M, N, K);
  const int MB = M <= 16 ? 1 : 2;
  const int NT = N / 16;
  *c_tmp_bytes = c.sk > 1 ? (size_t)c.sk * NT * MB * 64 * sizeof(v4f) : 0;
  *counter_ints = c.sk > 1 ? (size_t)NT * MB : 0;
  return VAQ_OK;
}

int w4a16_decode_launch(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                        const int32_t* perm, const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes,
                        int32_t* counters, int64_t counter_ints, int M, int N, int K, bool channelwise, int dtype,
                        hipStream_t s) {
  DecodeParams p;
  p.a = (const uint16_t*)a;
  p.lda = lda;
  p.b = (const v4u*)b;
  p.scales = (const uint16_t*)scales;
  p.zeros = (const uint32_t*)zeros;
  p.perm = perm;
  p.bias = (const uint16_t*)bias;
  p.c = (uint16_t*)c;
  p.c_tmp = (v4f*)c_tmp;
  p.counters = counters;
  p.M = M; p.N = N; p.K = K;
  p.G = K / 128;
  p.NT = N / 16;
  p.GR = channelwise ? 1 : p.G;
  p.s_stride = channelwise ? 0 : N;
  p.z_stride = channelwise ? 0 : N / 8;
  p.k_mask = 0x000f000fu;
  p.k_ex = dtype == VAQ_BF16 ? 0x43004300u : 0x64006400u;
  const DecodeConfig cfg = pick_decode_config(M, N, K);
  p.SK = cfg.sk;
  p.WK = cfg.wk;
  const int MB = M <= 16 ? 1 : 2;
  if (cfg.sk > 1) {
    VAQ_CHECK_ARG(c_tmp != nullptr && counters != nullptr, "w4a16_gemm: split-K needs c_tmp and counters");
    VAQ_CHECK_ARG(((uintptr_t)c_tmp % 16) == 0, "w4a16_gemm: c_tmp must be 16-byte aligned");
    VAQ_CHECK_ARG((uint64_t)cfg.sk * (uint64_t)p.NT * 2048u < (1ull << 31), "w4a16_gemm: split-K scratch too large");
    VAQ_CHECK_ARG(counter_ints >= (int64_t)p.NT * MB,
                  "w4a16_gemm: workspace.numel = %lld is below min_workspace_size = %lld", (long long)counter_ints,
                  (long long)p.NT * MB);
    VAQ_CHECK_ARG(c_tmp_bytes >= (int64_t)cfg.sk * p.NT * MB * 1024, "w4a16_gemm: c_tmp holds %lld bytes, the K split needs %lld",
                  (long long)c_tmp_bytes, (long long)cfg.sk * p.NT * MB * 1024);
  }
  const bool bf16 = dtype == VAQ_BF16, zp = zeros != nullptr;
  int rc;
  if (MB == 1) {
    if (bf16) rc = zp ? dispatch_tg<true, 1, true>(p, cfg, s) : dispatch_tg<true, 1, false>(p, cfg, s);
    else rc = zp ? dispatch_tg<false, 1, true>(p, cfg, s) : dispatch_tg<false, 1, false>(p, cfg, s);
  } else {
    if (bf16) rc = zp ? dispatch_tg<true, 2, true>(p, cfg, s) : dispatch_tg<true, 2, false>(p, cfg, s);
    else rc = zp ? dispatch_tg<false, 2, true>(p, cfg, s) : dispatch_tg<false, 2, false>(p, cfg, s);
  }
  if (rc != VAQ_OK) return rc;
  VAQ_CHECK_LAUNCH("w4a16_gemm(decode)");
  return VAQ_OK;
}

}  // namespace vaq
