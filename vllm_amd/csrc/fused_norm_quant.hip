// RMSNorm (+ residual add) fused with dynamic per-token FP8 (OCP e4m3fn) quantisation for gfx950: the step in front of a
// per-token-scaled FP8 GEMM, done in one pass over the activations instead of a norm pass plus a quant pass.
//
// Arithmetic, in the order of the reference kernel (csrc/quantization/fused_kernels/layernorm_utils.cuh:17-130):
//   x   = float(input) (+ float(residual); the sum, rounded to the activation type, is written back to `residual`)
//   rms = rsqrtf(sum(x*x) / hidden + eps)                                   (fp32)
//   y   = float( T(x * rms) * weight )        -- the product with the weight is rounded to the activation type T
//   s   = max(min(max|y|, ub) / 448, 1/(448*512))
//   q   = cvt(clamp(y / s, +-448))            -- a true division, like the unfused per-token quantiser
// Only the order of the fp32 additions inside sum(x*x) is this kernel's own (per-thread partial sums over a strided
// set of 8-element vectors, a butterfly over the 64 lanes, then the wavefronts in order); everything else is fixed by
// the list above, so results agree with the reference up to that last-bit freedom of `rms`.
//
// The static-scale variant (reference: csrc/layernorm_quant_kernels.cu:21-178, ops rms_norm_static_fp8_quant and
// fused_add_rms_norm_static_fp8_quant) differs in two places: with a residual the sum is rounded to the activation type
// first and the statistics are taken from the rounded value, and the quantisation multiplies by 1/scale of the given
// per-tensor scale:  q = cvt(clamp(y * (1/scale), +-448)).
//
// HBM-bound: one workgroup per token; the row (and the residual sum) stays in registers between the three passes when
// it has at most 512 x 8 x 8 = 32768 elements and is 16-byte aligned; other rows re-read global memory.
#include "vaq_common.h"

#include <type_traits>

namespace vaq {

namespace {

constexpr float NQ_FP8_MAX = 448.0f;
constexpr int NQ_T = 512;
// Chunks of 8 elements per thread that the row-in-registers path holds (template parameter NV): 2, 4 or 8, the smallest
// that covers the row -- the register arrays are sized by it, and with them the number of rows a compute unit works on
// at a time.
constexpr int NQ_V_MAX = 8;

template <bool BF16>
__device__ inline float nq_to_float(uint16_t v) { return F16Traits<BF16>::to_float(v); }

// round a float to the 16-bit activation type and come back
template <bool BF16>
__device__ inline float nq_round16(float x) { return F16Traits<BF16>::to_float(F16Traits<BF16>::from_float(x)); }

// a * b rounded to the 16-bit type.  For fp16 the product and its conversion are kept apart: left to the compiler the
// pair becomes v_fma_mixlo_f16(a, b, +0), and a product of -0 plus +0 is +0 -- the sign of a zero result would be lost
// (the reference's half-precision multiply keeps it, and the FP8 code of -0 is 0x80).  The multiply itself stays the
// compiler's: written as an instruction in inline assembly it would read the result of a transcendental instruction
// (the reciprocal in silu) without the wait state that the compiler inserts for its own instructions.
template <bool BF16>
__device__ inline float nq_mul_round16(float a, float b) {
  if constexpr (BF16) {
    return nq_round16<true>(a * b);
  } else {
    float p = a * b;
    asm("" : "+v"(p));      // the product is final here: nothing to fuse the conversion with
    return nq_round16<false>(p);
  }
}

template <int TPB>
__device__ inline float nq_block_sum(float v, float* smem) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float r = smem[0];
#pragma unroll
  for (int i = 1; i < TPB / 64; ++i) r += smem[i];
  __syncthreads();
  return r;
}

template <int TPB>
__device__ inline float nq_block_max(float v, float* smem) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float r = smem[0];
#pragma unroll
  for (int i = 1; i < TPB / 64; ++i) r = fmaxf(r, smem[i]);
  __syncthreads();
  return r;
}

__device__ inline void nq_unpack8(v4u r, float* f, bool bf16) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = bf16 ? nq_to_float<true>((uint16_t)(w[i] & 0xffffu)) : nq_to_float<false>((uint16_t)(w[i] & 0xffffu));
    f[2 * i + 1] = bf16 ? nq_to_float<true>((uint16_t)(w[i] >> 16)) : nq_to_float<false>((uint16_t)(w[i] >> 16));
  }
}

// eight values -> eight e4m3 codes: cvt(clamp(dv(y), +-448))
template <typename F>
__device__ inline v2u nq_quant8(const float (&y)[8], F&& dv) {
  v2u o;
  uint32_t* ow = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    float q[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) q[e] = fmaxf(-NQ_FP8_MAX, fminf(dv(y[4 * h + e]), NQ_FP8_MAX));
    const uint32_t lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false) & 0xffffu;
    const uint32_t hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], 0, false) & 0xffffu;
    ow[h] = lo | (hi << 16);
  }
  return o;
}

// One token per WAVEFRONT (rows of at most 64 x NV x 8 elements, many tokens): the row sits in the wavefront's
// registers, both reductions are butterflies over its lanes -- no LDS, no barrier, NQ_W / 64 independent rows per
// workgroup and every load of a row in flight at once.  DYN: the dynamic per-token quantiser (scale written per token);
// otherwise the static one (`scales` = the given per-tensor scale).  Same arithmetic as the row-per-workgroup kernels
// below; only the order of the additions inside the sum of squares differs (per lane over its chunks, then the butterfly).
constexpr int NQ_W = 256;
template <bool BF16, bool HAS_RES, bool DYN, int NV>
__global__ __launch_bounds__(NQ_W) void rms_norm_fp8_row_per_wave_kernel(uint8_t* __restrict__ out, float* __restrict__ scales,
                                                                         const uint16_t* __restrict__ input,
                                                                         const uint16_t* __restrict__ weight,
                                                                         const float* __restrict__ scale_ub, float eps,
                                                                         uint16_t* __restrict__ residual, int hidden,
                                                                         int64_t in_stride, int64_t tokens) {
  using T = F16Traits<BF16>;
  const int lane = threadIdx.x & 63;
  const int64_t tok = (int64_t)blockIdx.x * (NQ_W / 64) + (threadIdx.x >> 6);
  if (tok >= tokens) return;
  const uint16_t* row = input + tok * in_stride;
  uint16_t* res = HAS_RES ? residual + tok * (int64_t)hidden : nullptr;
  uint8_t* orow = out + tok * (int64_t)hidden;
  const int chunks = hidden / 8;
  v4u xr[NV], rr[HAS_RES ? NV : 1], wv[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int c = lane + v * 64;
    if (c < chunks) {
      xr[v] = *reinterpret_cast<const v4u*>(row + c * 8);
      if constexpr (HAS_RES) rr[v] = *reinterpret_cast<const v4u*>(res + c * 8);
    }
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int c = lane + v * 64;
    if (c < chunks) wv[v] = *reinterpret_cast<const v4u*>(weight + c * 8);
  }
  float x[NV][8];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int c = lane + v * 64;
    if (c < chunks) {
      nq_unpack8(xr[v], x[v], BF16);
      if constexpr (HAS_RES) {
        float r[8];
        nq_unpack8(rr[v], r, BF16);
        v4u back;
        uint32_t* bw = reinterpret_cast<uint32_t*>(&back);
        uint16_t z[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          x[v][e] += r[e];
          z[e] = T::from_float(x[v][e]);
          if constexpr (!DYN) x[v][e] = T::to_float(z[e]);      // static variant: statistics from the rounded sum
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) bw[e] = (uint32_t)z[2 * e] | ((uint32_t)z[2 * e + 1] << 16);
        *reinterpret_cast<v4u*>(res + c * 8) = back;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[v][e] * x[v][e];
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
  const float rms = rsqrtf(ss / (float)hidden + eps);
  float amax = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int c = lane + v * 64;
    if (c < chunks) {
      float w[8];
      nq_unpack8(wv[v], w, BF16);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        x[v][e] = nq_mul_round16<BF16>(nq_mul_round16<BF16>(x[v][e], rms), w[e]);
        if constexpr (DYN) amax = fmaxf(amax, fabsf(x[v][e]));
      }
    }
  }
  if constexpr (DYN) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if (scale_ub) amax = fminf(amax, *scale_ub);
    const float s = fmaxf(amax / NQ_FP8_MAX, 1.0f / (NQ_FP8_MAX * 512.0f));
    if (lane == 0) scales[tok] = s;
    const bool fast = scale_ub == nullptr && s < __builtin_inff();
    const float rcp = 1.0f / s;
    auto store8 = [&](int v, auto&& dv) {
      const int c = lane + v * 64;
      if (c < chunks) *reinterpret_cast<v2u*>(orow + c * 8) = nq_quant8(x[v], dv);
    };
    if (fast) {
#pragma unroll
      for (int v = 0; v < NV; ++v) store8(v, [&](float y) { return div16_exact(y, s, rcp); });
    } else {
#pragma unroll
      for (int v = 0; v < NV; ++v) store8(v, [&](float y) { return y / s; });
    }
  } else {
    const float inv = 1.0f / *scales;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int c = lane + v * 64;
      if (c < chunks) *reinterpret_cast<v2u*>(orow + c * 8) = nq_quant8(x[v], [&](float y) { return y * inv; });
    }
  }
}

template <bool BF16, bool HAS_RES, int NV, int TPB>
__global__ __launch_bounds__(TPB) void rms_norm_per_token_fp8_kernel(uint8_t* __restrict__ out, float* __restrict__ scales,
                                                                      const uint16_t* __restrict__ input,
                                                                      const uint16_t* __restrict__ weight,
                                                                      const float* __restrict__ scale_ub, float eps,
                                                                      uint16_t* __restrict__ residual, int hidden,
                                                                      int64_t in_stride) {
  using T = F16Traits<BF16>;
  __shared__ float smem[TPB / 64];
  const int64_t tok = blockIdx.x;
  const uint16_t* row = input + tok * in_stride;
  uint16_t* res = HAS_RES ? residual + tok * (int64_t)hidden : nullptr;
  uint8_t* orow = out + tok * (int64_t)hidden;
  const int chunks = hidden / 8;
  const bool cached = (hidden % 8 == 0) && chunks <= TPB * NV && (in_stride % 8 == 0) &&
                      ((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(weight) |
                        reinterpret_cast<uintptr_t>(out) | (HAS_RES ? reinterpret_cast<uintptr_t>(residual) : 0)) % 16 == 0);
  const float min_scale = 1.0f / (NQ_FP8_MAX * 512.0f);

  if (cached) {
    float x[NV][8];
    v4u wv[NV];          // the weight chunks, requested together with the row: no dependent load after the reduction
    float ss = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int c = threadIdx.x + v * TPB;
      if (c < chunks) {
        wv[v] = *reinterpret_cast<const v4u*>(weight + c * 8);
        nq_unpack8(*reinterpret_cast<const v4u*>(row + c * 8), x[v], BF16);
        if constexpr (HAS_RES) {
          float r[8];
          nq_unpack8(*reinterpret_cast<const v4u*>(res + c * 8), r, BF16);
          v4u back;
          uint32_t* bw = reinterpret_cast<uint32_t*>(&back);
#pragma unroll
          for (int e = 0; e < 8; ++e) x[v][e] += r[e];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            bw[e] = (uint32_t)T::from_float(x[v][2 * e]) | ((uint32_t)T::from_float(x[v][2 * e + 1]) << 16);
          *reinterpret_cast<v4u*>(res + c * 8) = back;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[v][e] * x[v][e];
      }
    }
    ss = nq_block_sum<TPB>(ss, smem);
    const float rms = rsqrtf(ss / (float)hidden + eps);
    float amax = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int c = threadIdx.x + v * TPB;
      if (c < chunks) {
        float w[8];
        nq_unpack8(wv[v], w, BF16);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          x[v][e] = nq_mul_round16<BF16>(nq_mul_round16<BF16>(x[v][e], rms), w[e]);
          amax = fmaxf(amax, fabsf(x[v][e]));
        }
      }
    }
    amax = nq_block_max<TPB>(amax, smem);
    if (scale_ub) amax = fminf(amax, *scale_ub);
    const float s = fmaxf(amax / NQ_FP8_MAX, min_scale);
    if (threadIdx.x == 0) scales[tok] = s;
    // y is a 16-bit value: without an upper bound on the scale (|y / s| <= 448) and with a finite scale the quotient
    // comes from the exact three-instruction division
    const bool fast = scale_ub == nullptr && s < __builtin_inff();
    const float rcp = 1.0f / s;
    auto store8 = [&](int v, auto&& dv) {
      const int c = threadIdx.x + v * TPB;
      if (c < chunks) *reinterpret_cast<v2u*>(orow + c * 8) = nq_quant8(x[v], dv);
    };
    if (fast) {
#pragma unroll
      for (int v = 0; v < NV; ++v) store8(v, [&](float y) { return div16_exact(y, s, rcp); });
    } else {
#pragma unroll
      for (int v = 0; v < NV; ++v) store8(v, [&](float y) { return y / s; });
    }
    return;
  }

  // general path: three passes over global memory, one element per thread and step
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += TPB) {
    float x = nq_to_float<BF16>(row[i]);
    if constexpr (HAS_RES) {
      x += nq_to_float<BF16>(res[i]);
    }
    ss += x * x;
  }
  ss = nq_block_sum<TPB>(ss, smem);
  const float rms = rsqrtf(ss / (float)hidden + eps);
  float amax = 0.f;
  for (int i = threadIdx.x; i < hidden; i += TPB) {
    float x = nq_to_float<BF16>(row[i]);
    if constexpr (HAS_RES) x += nq_to_float<BF16>(res[i]);
    const float y = nq_mul_round16<BF16>(nq_mul_round16<BF16>(x, rms), nq_to_float<BF16>(weight[i]));
    amax = fmaxf(amax, fabsf(y));
  }
  amax = nq_block_max<TPB>(amax, smem);
  if (scale_ub) amax = fminf(amax, *scale_ub);
  const float s = fmaxf(amax / NQ_FP8_MAX, min_scale);
  if (threadIdx.x == 0) scales[tok] = s;
  for (int i = threadIdx.x; i < hidden; i += TPB) {
    float x = nq_to_float<BF16>(row[i]);
    if constexpr (HAS_RES) {
      x += nq_to_float<BF16>(res[i]);
      res[i] = T::from_float(x);
    }
    const float y = nq_mul_round16<BF16>(nq_mul_round16<BF16>(x, rms), nq_to_float<BF16>(weight[i]));
    const float q = fmaxf(-NQ_FP8_MAX, fminf(y / s, NQ_FP8_MAX));
    orow[i] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(q, q, 0, false) & 0xff);
  }
}

template <bool BF16, bool HAS_RES, int NV, int TPB>
__global__ __launch_bounds__(TPB) void rms_norm_static_fp8_kernel(uint8_t* __restrict__ out,
                                                                   const uint16_t* __restrict__ input,
                                                                   const uint16_t* __restrict__ weight,
                                                                   const float* __restrict__ scale, float eps,
                                                                   uint16_t* __restrict__ residual, int hidden,
                                                                   int64_t in_stride) {
  using T = F16Traits<BF16>;
  __shared__ float smem[TPB / 64];
  const int64_t tok = blockIdx.x;
  const uint16_t* row = input + tok * in_stride;
  uint16_t* res = HAS_RES ? residual + tok * (int64_t)hidden : nullptr;
  uint8_t* orow = out + tok * (int64_t)hidden;
  const int chunks = hidden / 8;
  const bool cached = (hidden % 8 == 0) && chunks <= TPB * NV && (in_stride % 8 == 0) &&
                      ((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(weight) |
                        reinterpret_cast<uintptr_t>(out) | (HAS_RES ? reinterpret_cast<uintptr_t>(residual) : 0)) % 16 == 0);
  const float inv = 1.0f / *scale;

  if (cached) {
    float x[NV][8];
    v4u wv[NV];          // the weight chunks, requested together with the row
    float ss = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int c = threadIdx.x + v * TPB;
      if (c < chunks) {
        wv[v] = *reinterpret_cast<const v4u*>(weight + c * 8);
        nq_unpack8(*reinterpret_cast<const v4u*>(row + c * 8), x[v], BF16);
        if constexpr (HAS_RES) {
          float r[8];
          nq_unpack8(*reinterpret_cast<const v4u*>(res + c * 8), r, BF16);
          v4u back;
          uint32_t* bw = reinterpret_cast<uint32_t*>(&back);
          uint16_t z[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            z[e] = T::from_float(x[v][e] + r[e]);
            x[v][e] = T::to_float(z[e]);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) bw[e] = (uint32_t)z[2 * e] | ((uint32_t)z[2 * e + 1] << 16);
          *reinterpret_cast<v4u*>(res + c * 8) = back;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[v][e] * x[v][e];
      }
    }
    ss = nq_block_sum<TPB>(ss, smem);
    const float rms = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int c = threadIdx.x + v * TPB;
      if (c < chunks) {
        float w[8];
        nq_unpack8(wv[v], w, BF16);
        v2u o;
        uint32_t* ow = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float q[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float y = nq_mul_round16<BF16>(nq_mul_round16<BF16>(x[v][4 * h + e], rms), w[4 * h + e]);
            q[e] = fmaxf(-NQ_FP8_MAX, fminf(y * inv, NQ_FP8_MAX));
          }
          uint32_t lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false) & 0xffffu;
          uint32_t hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], 0, false) & 0xffffu;
          ow[h] = lo | (hi << 16);
        }
        *reinterpret_cast<v2u*>(orow + c * 8) = o;
      }
    }
    return;
  }

  // general path: two passes over global memory, one element per thread and step
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += TPB) {
    float x = nq_to_float<BF16>(row[i]);
    if constexpr (HAS_RES) {
      const uint16_t z = T::from_float(x + nq_to_float<BF16>(res[i]));
      res[i] = z;
      x = T::to_float(z);
    }
    ss += x * x;
  }
  ss = nq_block_sum<TPB>(ss, smem);  // its barrier also orders this workgroup's own writes to `res` before the re-reads
  const float rms = rsqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += TPB) {
    const float x = nq_to_float<BF16>(HAS_RES ? res[i] : row[i]);
    const float y = nq_mul_round16<BF16>(nq_mul_round16<BF16>(x, rms), nq_to_float<BF16>(weight[i]));
    const float q = fmaxf(-NQ_FP8_MAX, fminf(y * inv, NQ_FP8_MAX));
    orow[i] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(q, q, 0, false) & 0xff);
  }
}

// silu(x) * y of the two halves of each row, quantised with a given per-tensor scale.
// reference: csrc/quantization/activation_kernels.cu:35-119 -- silu is rounded to the activation type, so is the product.
// x / (1 + exp(-x)) as x * rcp(1 + exp2(-log2(e) x)): the hardware exponential and reciprocal (one unit in the last place
// each, plus |x| * 6e-8 from the rounded argument) instead of the library exponential and the IEEE division, 6 instead of
// ~25 instructions per element.  The quotient is rounded to a 16-bit type straight away, three orders of magnitude
// coarser than that error: 4096 x 14336 normal values gave the same 58.7 M codes as the library forms, and the kernel is
// no longer bound by its arithmetic (69.6 -> 45.7 us, 6.4 TB/s).  Saturation is the same: exp2 overflows to +inf for
// x < -88 (quotient -0), underflows to 0 for large x (quotient x), and -inf gives NaN like -inf / inf does.
template <bool BF16>
__device__ inline float silu_mul16(float x, float y) {
  const float s = nq_mul_round16<BF16>(x, __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x)));
  return nq_mul_round16<BF16>(s, y);
}

template <bool BF16, bool VEC>
__global__ __launch_bounds__(NQ_T) void silu_and_mul_fp8_kernel(uint8_t* __restrict__ out,
                                                                const uint16_t* __restrict__ input,
                                                                const float* __restrict__ scale, int64_t tokens, int d) {
  const float inv = 1.0f / *scale;
  if constexpr (VEC) {
    const int chunks = d / 8;
    const int64_t total = tokens * chunks;
    for (int64_t idx = (int64_t)blockIdx.x * NQ_T + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * NQ_T) {
      const int64_t tok = idx / chunks;
      const int c = (int)(idx - tok * chunks);
      const uint16_t* xr = input + tok * 2 * (int64_t)d + c * 8;
      float x[8], y[8];
      nq_unpack8(*reinterpret_cast<const v4u*>(xr), x, BF16);
      nq_unpack8(*reinterpret_cast<const v4u*>(xr + d), y, BF16);
      v2u o;
      uint32_t* ow = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float q[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          q[e] = fmaxf(-NQ_FP8_MAX, fminf(silu_mul16<BF16>(x[4 * h + e], y[4 * h + e]) * inv, NQ_FP8_MAX));
        uint32_t lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false) & 0xffffu;
        uint32_t hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], 0, false) & 0xffffu;
        ow[h] = lo | (hi << 16);
      }
      *reinterpret_cast<v2u*>(out + tok * (int64_t)d + c * 8) = o;
    }
  } else {
    const int64_t total = tokens * d;
    for (int64_t idx = (int64_t)blockIdx.x * NQ_T + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * NQ_T) {
      const int64_t tok = idx / d;
      const int i = (int)(idx - tok * d);
      const uint16_t* xr = input + tok * 2 * (int64_t)d;
      const float v = silu_mul16<BF16>(nq_to_float<BF16>(xr[i]), nq_to_float<BF16>(xr[d + i]));
      const float q = fmaxf(-NQ_FP8_MAX, fminf(v * inv, NQ_FP8_MAX));
      out[idx] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(q, q, 0, false) & 0xff);
    }
  }
}

}  // namespace

}  // namespace vaq

namespace vaq {
// A token per wavefront: rows that allow 16-byte loads everywhere, short enough and many enough for it to pay (the
// same bounds as the unfused per-token quantiser, where a wavefront per row measured 1.1-1.8x faster inside them and
// slower outside: at 4096 elements the 64 values per lane no longer overlap their own arithmetic with other rows' loads).
static bool nq_row_per_wave(const void* out, const void* in, const void* w, const void* res, int64_t in_stride,
                            int64_t tokens, int64_t hidden) {
  const bool can = hidden % 8 == 0 && hidden <= 64 * 8 * 4 && in_stride % 8 == 0 &&
                   ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(out) |
                     reinterpret_cast<uintptr_t>(res)) % 16 == 0);
  return can && (hidden <= 1024 ? tokens >= 1024 : tokens >= 2048);
}

// Rows of at most 4096 elements run on workgroups of 256 threads (two chunks of 8 elements per thread): twice the
// workgroups per compute unit, each a dependent chain of load, reduction(s) and store of its own, and half the
// wavefronts in every barrier.  4096 tokens of 4096: dynamic per-token 16.2 -> 13.6 us, with residual and a static scale
// 20.0 -> 19.2 us, static scale 13.5 -> 13.5 us; longer rows are better off with 512 threads (8192: 22.0 against 24.0 us
// static; 14336 with residual 65.7 against 70.5 us).
static bool nq_half_workgroup(int64_t hidden) { return hidden <= (NQ_T / 2) * 8 * 2; }

// run-time (dtype, residual, chunks per thread) -> compile-time template arguments
template <typename F>
static void nq_dispatch(bool bf16, bool has_res, int nv, F&& f) {
  auto with_nv = [&](auto bf, auto rs) {
    if (nv == 2) f(bf, rs, std::integral_constant<int, 2>{});
    else if (nv == 4) f(bf, rs, std::integral_constant<int, 4>{});
    else f(bf, rs, std::integral_constant<int, NQ_V_MAX>{});
  };
  auto with_res = [&](auto bf) {
    if (has_res) with_nv(bf, std::true_type{});
    else with_nv(bf, std::false_type{});
  };
  if (bf16) with_res(std::true_type{});
  else with_res(std::false_type{});
}
}  // namespace vaq

extern "C" int vaq_rms_norm_dynamic_per_token_fp8_quant(uint8_t* out, float* scales, const void* input, int64_t in_stride,
                                                        const void* weight, const float* scale_ub, float epsilon,
                                                        void* residual, int dtype, int64_t tokens, int64_t hidden,
                                                        void* stream) {
  using namespace vaq;
  VAQ_CHECK_ARG(tokens >= 0 && hidden > 0 && hidden < (1ll << 31) && tokens < (1ll << 31),
                "rms_norm_dynamic_per_token_quant: bad shape [%lld, %lld]", (long long)tokens, (long long)hidden);
  VAQ_CHECK_ARG(dtype == VAQ_F16 || dtype == VAQ_BF16, "rms_norm_dynamic_per_token_quant: dtype tag %d", dtype);
  VAQ_CHECK_ARG(in_stride >= hidden, "rms_norm_dynamic_per_token_quant: input row stride %lld < hidden %lld",
                (long long)in_stride, (long long)hidden);
  if (tokens == 0) return VAQ_OK;
  VAQ_CHECK_ARG(out && scales && input && weight, "rms_norm_dynamic_per_token_quant: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)tokens), block(NQ_T);
  const uint16_t* in = (const uint16_t*)input;
  const uint16_t* w = (const uint16_t*)weight;
  uint16_t* res = (uint16_t*)residual;
  const bool bf16 = dtype == VAQ_BF16;
  if (nq_row_per_wave(out, in, w, res, in_stride, tokens, hidden)) {
    const dim3 wgrid((unsigned)((tokens + NQ_W / 64 - 1) / (NQ_W / 64))), wblock(NQ_W);
    auto launch = [&](auto bf, auto rs, auto nvc) {
      hipLaunchKernelGGL((rms_norm_fp8_row_per_wave_kernel<decltype(bf)::value, decltype(rs)::value, true, decltype(nvc)::value>),
                         wgrid, wblock, 0, s, out, scales, in, w, scale_ub, epsilon, res, (int)hidden, in_stride, tokens);
    };
    nq_dispatch(bf16, res != nullptr, hidden <= 64 * 8 * 2 ? 2 : 4, launch);
    VAQ_CHECK_LAUNCH("rms_norm_dynamic_per_token_quant");
    return VAQ_OK;
  }
  const int nv = hidden <= NQ_T * 8 * 2 ? 2 : (hidden <= NQ_T * 8 * 4 ? 4 : NQ_V_MAX);
  const bool half_wg = nq_half_workgroup(hidden);
  auto launch = [&](auto bf, auto rs, auto nvc) {
    if (half_wg)
      hipLaunchKernelGGL((rms_norm_per_token_fp8_kernel<decltype(bf)::value, decltype(rs)::value, 2, NQ_T / 2>), grid,
                         dim3(NQ_T / 2), 0, s, out, scales, in, w, scale_ub, epsilon, res, (int)hidden, in_stride);
    else
      hipLaunchKernelGGL((rms_norm_per_token_fp8_kernel<decltype(bf)::value, decltype(rs)::value, decltype(nvc)::value, NQ_T>),
                         grid, block, 0, s, out, scales, in, w, scale_ub, epsilon, res, (int)hidden, in_stride);
  };
  nq_dispatch(bf16, res != nullptr, nv, launch);
  VAQ_CHECK_LAUNCH("rms_norm_dynamic_per_token_quant");
  return VAQ_OK;
}

extern "C" int vaq_rms_norm_static_fp8_quant(uint8_t* out, const void* input, int64_t in_stride, const void* weight,
                                             const float* scale, float epsilon, void* residual, int dtype,
                                             int64_t tokens, int64_t hidden, void* stream) {
  using namespace vaq;
  VAQ_CHECK_ARG(tokens >= 0 && hidden > 0 && hidden < (1ll << 31) && tokens < (1ll << 31),
                "rms_norm_static_fp8_quant: bad shape [%lld, %lld]", (long long)tokens, (long long)hidden);
  VAQ_CHECK_ARG(dtype == VAQ_F16 || dtype == VAQ_BF16, "rms_norm_static_fp8_quant: dtype tag %d", dtype);
  VAQ_CHECK_ARG(in_stride >= hidden, "rms_norm_static_fp8_quant: input row stride %lld < hidden %lld",
                (long long)in_stride, (long long)hidden);
  if (tokens == 0) return VAQ_OK;
  VAQ_CHECK_ARG(out && input && weight && scale, "rms_norm_static_fp8_quant: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)tokens), block(NQ_T);
  const uint16_t* in = (const uint16_t*)input;
  const uint16_t* w = (const uint16_t*)weight;
  uint16_t* res = (uint16_t*)residual;
  if (nq_row_per_wave(out, in, w, res, in_stride, tokens, hidden)) {
    const dim3 wgrid((unsigned)((tokens + NQ_W / 64 - 1) / (NQ_W / 64))), wblock(NQ_W);
    auto launch = [&](auto bf, auto rs, auto nvc) {
      hipLaunchKernelGGL((rms_norm_fp8_row_per_wave_kernel<decltype(bf)::value, decltype(rs)::value, false, decltype(nvc)::value>),
                         wgrid, wblock, 0, s, out, const_cast<float*>(scale), in, w, nullptr, epsilon, res, (int)hidden,
                         in_stride, tokens);
    };
    nq_dispatch(dtype == VAQ_BF16, res != nullptr, hidden <= 64 * 8 * 2 ? 2 : 4, launch);
    VAQ_CHECK_LAUNCH("rms_norm_static_fp8_quant");
    return VAQ_OK;
  }
  const int nv = hidden <= NQ_T * 8 * 2 ? 2 : (hidden <= NQ_T * 8 * 4 ? 4 : NQ_V_MAX);
  const bool half_wg = nq_half_workgroup(hidden);
  auto launch = [&](auto bf, auto rs, auto nvc) {
    if (half_wg)
      hipLaunchKernelGGL((rms_norm_static_fp8_kernel<decltype(bf)::value, decltype(rs)::value, 2, NQ_T / 2>), grid, dim3(NQ_T / 2),
                         0, s, out, in, w, scale, epsilon, res, (int)hidden, in_stride);
    else
      hipLaunchKernelGGL((rms_norm_static_fp8_kernel<decltype(bf)::value, decltype(rs)::value, decltype(nvc)::value, NQ_T>), grid,
                         block, 0, s, out, in, w, scale, epsilon, res, (int)hidden, in_stride);
  };
  nq_dispatch(dtype == VAQ_BF16, res != nullptr, nv, launch);
  VAQ_CHECK_LAUNCH("rms_norm_static_fp8_quant");
  return VAQ_OK;
}

extern "C" int vaq_silu_and_mul_fp8_quant(uint8_t* out, const void* input, const float* scale, int dtype, int64_t tokens,
                                          int64_t d, void* stream) {
  using namespace vaq;
  VAQ_CHECK_ARG(tokens >= 0 && d >= 0 && d < (1ll << 30) && tokens < (1ll << 31),
                "silu_and_mul_quant: bad shape [%lld, 2*%lld]", (long long)tokens, (long long)d);
  VAQ_CHECK_ARG(dtype == VAQ_F16 || dtype == VAQ_BF16, "silu_and_mul_quant: dtype tag %d", dtype);
  if (tokens == 0 || d == 0) return VAQ_OK;
  VAQ_CHECK_ARG(out && input && scale, "silu_and_mul_quant: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const bool vec = d % 8 == 0 && ((uintptr_t)input % 16) == 0 && ((uintptr_t)out % 8) == 0;
  const int64_t work = vec ? tokens * (d / 8) : tokens * d;
  int64_t blocks = (work + NQ_T - 1) / NQ_T;
  const int64_t cap = (int64_t)num_cus_current_device() * 32;
  if (blocks > cap) blocks = cap;
  const dim3 grid((unsigned)blocks), block(NQ_T);
  const uint16_t* in = (const uint16_t*)input;
  if (dtype == VAQ_BF16) {
    if (vec) hipLaunchKernelGGL((silu_and_mul_fp8_kernel<true, true>), grid, block, 0, s, out, in, scale, tokens, (int)d);
    else hipLaunchKernelGGL((silu_and_mul_fp8_kernel<true, false>), grid, block, 0, s, out, in, scale, tokens, (int)d);
  } else {
    if (vec) hipLaunchKernelGGL((silu_and_mul_fp8_kernel<false, true>), grid, block, 0, s, out, in, scale, tokens, (int)d);
    else hipLaunchKernelGGL((silu_and_mul_fp8_kernel<false, false>), grid, block, 0, s, out, in, scale, tokens, (int)d);
  }
  VAQ_CHECK_LAUNCH("silu_and_mul_quant");
  return VAQ_OK;
}
