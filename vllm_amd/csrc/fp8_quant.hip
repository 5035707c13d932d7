// FP8 (OCP e4m3fn) activation quantisation for gfx950: per-token dynamic, per-tensor dynamic, per-tensor static.
//
// Bit-exactness contract (codes AND scales) with the reference kernels:
//   per token : amax = max|float(x)| ; s = max(min(amax, ub) / 448, 1/(448*512)) ; q = cvt(clamp(float(x) / s, +-448))
//               -- the correctly rounded fp32 quotient per element, not a reciprocal multiply (for 16-bit inputs without
//               an upper bound on the scale it comes from div16_exact: three instructions, the same bits);
//   per tensor: s = amax_all / 448 ; q = cvt(clamp(float(x) * (1 / s), +-448))   (reciprocal multiply);
//   static    : q = cvt(clamp(float(x) * (1 / scale), +-448)).
// cvt is the hardware v_cvt_pk_fp8_f32 (round-to-nearest-even; inputs are already clamped, NaN stays NaN).
// The file is compiled without fast-math, so `/` is the correctly rounded division.
//
// HBM-bound: each row is read ONCE -- a workgroup keeps its whole row in registers between the absmax pass and the
// convert pass whenever the row has at most 512 threads x 4 vectors x 8 elements = 16384 elements and is 16-byte
// aligned; other rows take a two-pass scalar path.
#include "vaq_common.h"

namespace vaq {

constexpr float FP8_MAX = 448.0f;
// (measured: 512 threads with 4 vectors each against 256 x 8: 2.95 -> 2.68 us at 16 rows of 4096, 3.65 -> 3.3 us at 256
// rows, 41.5 -> 39.5 us at 4096 rows of 14336, unchanged at 4096 x 4096; 1024 x 2 and 128 x 16 are slower)
constexpr int QT = 512;         // threads per workgroup of the row-per-workgroup kernel (its TPB: QT or QT / 2)
constexpr int QV = 4;           // cached 8-element vectors per thread
constexpr int QTW = 256;        // threads per workgroup of the row-per-wavefront kernel (four rows)

template <typename T>
__device__ inline float load_as_float(const T* p);
template <>
__device__ inline float load_as_float<float>(const float* p) { return *p; }
struct bf16_t { uint16_t v; };
struct f16_t { uint16_t v; };
template <>
__device__ inline float load_as_float<bf16_t>(const bf16_t* p) { return F16Traits<true>::to_float(p->v); }
template <>
__device__ inline float load_as_float<f16_t>(const f16_t* p) { return F16Traits<false>::to_float(p->v); }

__device__ inline float clamp448(float x) { return fmaxf(-FP8_MAX, fminf(x, FP8_MAX)); }

// two fp32 -> two e4m3fn codes in the low 16 bits
__device__ inline uint32_t cvt2(float a, float b) { return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu; }
__device__ inline uint8_t cvt1(float a) { return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(a, a, 0, false) & 0xff); }

// 8 consecutive elements of a row as floats
template <typename T>
struct Vec8 {
  float f[8];
  __device__ inline void load(const T* p) {
    if constexpr (sizeof(T) == 2) {
      const v4u r = *reinterpret_cast<const v4u*>(p);
      const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        T lo, hi;
        lo.v = (uint16_t)(w[i] & 0xffffu);
        hi.v = (uint16_t)(w[i] >> 16);
        f[2 * i] = load_as_float<T>(&lo);
        f[2 * i + 1] = load_as_float<T>(&hi);
      }
    } else {
      const v4f a = *reinterpret_cast<const v4f*>(p);
      const v4f b = *reinterpret_cast<const v4f*>(p + 4);
      f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
      f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
  }
};

template <int TPB>
__device__ inline float block_max(float v, float* smem) {
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

// MODE 0: dynamic per token (divide by row scale, scale written per row)
// MODE 1: per tensor with a given scale (multiply by reciprocal) -- static, and pass 2 of dynamic per tensor
// MODE 2: absmax only: atomic max of rowmax/448 into *scale (pass 1 of dynamic per tensor)
template <typename T, int MODE, int TPB>
__global__ __launch_bounds__(TPB) void fp8_quant_kernel(const T* __restrict__ in, int64_t in_stride,
                                                        uint8_t* __restrict__ out, int64_t out_stride,
                                                        float* __restrict__ scales, const float* __restrict__ scale_ub,
                                                        int hidden) {
  __shared__ float smem[TPB / 64];
  const int64_t row = blockIdx.x;
  const T* x = in + row * in_stride;
  uint8_t* y = out + row * out_stride;
  const int tid = threadIdx.x;

  const bool vec_ok = (hidden % 8 == 0) && (((uintptr_t)x % 16) == 0) && (((uintptr_t)y % 8) == 0) &&
                      (hidden <= TPB * QV * 8);
  Vec8<T> cache[QV];
  const int nvec = hidden / 8;

  float scale_or_inv;
  if constexpr (MODE != 1) {
    float amax = 0.f;
    if (vec_ok) {
#pragma unroll
      for (int i = 0; i < QV; ++i) {
        const int v = tid + i * TPB;
        if (v < nvec) {
          cache[i].load(x + (int64_t)v * 8);
#pragma unroll
          for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(cache[i].f[e]));
        }
      }
    } else {
      for (int e = tid; e < hidden; e += TPB) amax = fmaxf(amax, fabsf(load_as_float<T>(x + e)));
    }
    amax = block_max<TPB>(amax, smem);
    if constexpr (MODE == 2) {
      // non-negative floats order like their bit patterns
      if (tid == 0) atomicMax(reinterpret_cast<int*>(scales), __float_as_int(amax / FP8_MAX));
      return;
    } else {
      float s = scale_ub ? fminf(amax, *scale_ub) : amax;
      s = fmaxf(s / FP8_MAX, 1.0f / (FP8_MAX * 512.0f));
      if (tid == 0) scales[row] = s;
      scale_or_inv = s;
    }
  } else {
    scale_or_inv = 1.0f / (*scales);
    if (vec_ok) {
#pragma unroll
      for (int i = 0; i < QV; ++i) {
        const int v = tid + i * TPB;
        if (v < nvec) cache[i].load(x + (int64_t)v * 8);
      }
    }
  }

  // MODE 0 on 16-bit inputs whose quotients cannot leave the normal range (no upper bound that could shrink the scale
  // below amax / 448, finite scale): the exact three-instruction division; the same for every thread of the row
  bool fast = false;
  float rcp = 0.f;
  if constexpr (MODE == 0 && sizeof(T) == 2) {
    fast = scale_ub == nullptr && scale_or_inv < __builtin_inff();
    rcp = 1.0f / scale_or_inv;
  }
  auto conv = [&](float v) -> float {
    if constexpr (MODE == 0) return clamp448(v / scale_or_inv);
    else return clamp448(v * scale_or_inv);
  };
  auto conv_fast = [&](float v) -> float { return clamp448(div16_exact(v, scale_or_inv, rcp)); };
  auto pack8 = [&](const float (&f)[8], auto&& cv) {
    v2u o;
    o.x = cvt2(cv(f[0]), cv(f[1])) | (cvt2(cv(f[2]), cv(f[3])) << 16);
    o.y = cvt2(cv(f[4]), cv(f[5])) | (cvt2(cv(f[6]), cv(f[7])) << 16);
    return o;
  };

  if (vec_ok) {
    if (fast) {
#pragma unroll
      for (int i = 0; i < QV; ++i) {
        const int v = tid + i * TPB;
        if (v < nvec) *reinterpret_cast<v2u*>(y + (int64_t)v * 8) = pack8(cache[i].f, conv_fast);
      }
    } else {
#pragma unroll
      for (int i = 0; i < QV; ++i) {
        const int v = tid + i * TPB;
        if (v < nvec) *reinterpret_cast<v2u*>(y + (int64_t)v * 8) = pack8(cache[i].f, conv);
      }
    }
  } else {
    for (int e = tid; e < hidden; e += TPB) y[e] = cvt1(conv(load_as_float<T>(x + e)));
  }
}

// Dynamic per token, one row per WAVEFRONT: the row (at most 64 lanes x NV vectors x 8 elements) sits in the wavefront's
// registers, the absmax is a butterfly over the lanes -- no LDS, no barrier, four rows per workgroup in flight
// independently.  Same arithmetic as MODE 0 above (the maximum is order-independent, the division is the IEEE one).
template <typename T, int NV>
__global__ __launch_bounds__(QTW) void fp8_quant_row_per_wave_kernel(const T* __restrict__ in, int64_t in_stride,
                                                                     uint8_t* __restrict__ out, int64_t out_stride,
                                                                     float* __restrict__ scales,
                                                                     const float* __restrict__ scale_ub, int hidden,
                                                                     int64_t rows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (QTW / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* x = in + row * in_stride;
  uint8_t* y = out + row * out_stride;
  const int nvec = hidden / 8;
  Vec8<T> cache[NV];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + i * 64;
    if (v < nvec) cache[i].load(x + (int64_t)v * 8);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + i * 64;
    if (v < nvec) {
#pragma unroll
      for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(cache[i].f[e]));
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  float s = scale_ub ? fminf(amax, *scale_ub) : amax;
  s = fmaxf(s / FP8_MAX, 1.0f / (FP8_MAX * 512.0f));
  if (lane == 0) scales[row] = s;
  const bool fast = scale_ub == nullptr && s < __builtin_inff();      // see fp8_quant_kernel
  const float rcp = 1.0f / s;
  auto store8 = [&](int i, auto&& cv) {
    const int v = lane + i * 64;
    if (v < nvec) {
      float q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = clamp448(cv(cache[i].f[e]));
      v2u o;
      o.x = cvt2(q[0], q[1]) | (cvt2(q[2], q[3]) << 16);
      o.y = cvt2(q[4], q[5]) | (cvt2(q[6], q[7]) << 16);
      *reinterpret_cast<v2u*>(y + (int64_t)v * 8) = o;
    }
  };
  if (fast) {
#pragma unroll
    for (int i = 0; i < NV; ++i) store8(i, [&](float v) { return div16_exact(v, s, rcp); });
  } else {
#pragma unroll
    for (int i = 0; i < NV; ++i) store8(i, [&](float v) { return v / s; });
  }
}

__global__ void fill_zero_kernel(float* p) { *p = 0.f; }

// The row-per-wavefront kernel takes 16-bit rows of at most 4096 elements whose addresses allow 16-byte loads and
// 8-byte stores on every row (the caller only sends rows of up to 2048 elements).
static bool row_per_wave_ok(const void* in, int in_dtype, int64_t in_stride, const uint8_t* out, int64_t out_stride,
                            int64_t hidden) {
  return (in_dtype == VAQ_BF16 || in_dtype == VAQ_F16) && hidden % 8 == 0 && hidden <= 64 * 8 * 8 &&
         ((uintptr_t)in % 16) == 0 && in_stride % 8 == 0 && ((uintptr_t)out % 8) == 0 && out_stride % 8 == 0;
}

template <typename T>
static void launch_row_per_wave(const void* in, int64_t in_stride, uint8_t* out, int64_t out_stride, float* scales,
                                const float* ub, int64_t rows, int64_t hidden, hipStream_t s) {
  const dim3 grid((unsigned)((rows + QTW / 64 - 1) / (QTW / 64))), block(QTW);
  if (hidden <= 64 * 8 * 2)
    hipLaunchKernelGGL((fp8_quant_row_per_wave_kernel<T, 2>), grid, block, 0, s, (const T*)in, in_stride, out, out_stride,
                       scales, ub, (int)hidden, rows);
  else if (hidden <= 64 * 8 * 4)
    hipLaunchKernelGGL((fp8_quant_row_per_wave_kernel<T, 4>), grid, block, 0, s, (const T*)in, in_stride, out, out_stride,
                       scales, ub, (int)hidden, rows);
  else
    hipLaunchKernelGGL((fp8_quant_row_per_wave_kernel<T, 8>), grid, block, 0, s, (const T*)in, in_stride, out, out_stride,
                       scales, ub, (int)hidden, rows);
}

// Many rows of at most 5120 elements run on workgroups of 256 threads: twice the workgroups per compute unit, each a
// dependent chain of load, reduction and store of its own, and half the wavefronts in every barrier (4096 rows of 3072 /
// 4096 / 5120: 10.5 / 12.4 / 14.2 -> 8.3 / 11.0 / 13.4 us, 8192 x 4096 20.9 -> 17.8 us; rows of 8192: 18.6 against 19.3 us
// with 512 threads; a few hundred rows of 4096: 3.0 against 3.2 us).
template <int MODE, int TPB>
static int launch_quant_tpb(const void* in, int in_dtype, int64_t in_stride, uint8_t* out, int64_t out_stride,
                            float* scales, const float* ub, int64_t rows, int64_t hidden, hipStream_t s) {
  const dim3 grid((unsigned)rows), block(TPB);
  switch (in_dtype) {
    case VAQ_BF16:
      hipLaunchKernelGGL((fp8_quant_kernel<bf16_t, MODE, TPB>), grid, block, 0, s, (const bf16_t*)in, in_stride, out,
                         out_stride, scales, ub, (int)hidden);
      break;
    case VAQ_F16:
      hipLaunchKernelGGL((fp8_quant_kernel<f16_t, MODE, TPB>), grid, block, 0, s, (const f16_t*)in, in_stride, out,
                         out_stride, scales, ub, (int)hidden);
      break;
    case VAQ_F32:
      hipLaunchKernelGGL((fp8_quant_kernel<float, MODE, TPB>), grid, block, 0, s, (const float*)in, in_stride, out,
                         out_stride, scales, ub, (int)hidden);
      break;
    default:
      set_error("fp8_quant: unsupported input dtype tag %d", in_dtype);
      return VAQ_ERR_INVALID_ARG;
  }
  return VAQ_OK;
}

template <int MODE>
static int launch_quant(const void* in, int in_dtype, int64_t in_stride, uint8_t* out, int64_t out_stride,
                        float* scales, const float* ub, int64_t rows, int64_t hidden, hipStream_t s) {
  if (rows >= 1024 && hidden <= 5120)
    return launch_quant_tpb<MODE, QT / 2>(in, in_dtype, in_stride, out, out_stride, scales, ub, rows, hidden, s);
  return launch_quant_tpb<MODE, QT>(in, in_dtype, in_stride, out, out_stride, scales, ub, rows, hidden, s);
}

static int check_quant(const char* who, const void* in, int64_t in_stride, const uint8_t* out, int64_t out_stride,
                       const float* scale, int64_t rows, int64_t hidden) {
  VAQ_CHECK_ARG(rows >= 0 && hidden > 0, "%s: bad shape [%lld, %lld]", who, (long long)rows, (long long)hidden);
  VAQ_CHECK_ARG(rows < (1ll << 31) && hidden < (1ll << 31), "%s: shape too large", who);
  VAQ_CHECK_ARG(in_stride >= hidden && out_stride >= hidden, "%s: row strides (%lld, %lld) smaller than hidden = %lld",
                who, (long long)in_stride, (long long)out_stride, (long long)hidden);
  if (rows > 0) VAQ_CHECK_ARG(in && out && scale, "%s: null pointer", who);
  return VAQ_OK;
}

}  // namespace vaq

extern "C" int vaq_fp8_quant_per_token(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out,
                                       int64_t out_row_stride, float* scales, const float* scale_ub, int64_t rows,
                                       int64_t hidden, void* stream) {
  return vaq_fp8_quant_per_token_tuned(in, in_dtype, in_row_stride, out, out_row_stride, scales, scale_ub, rows, hidden,
                                       stream, nullptr);
}

extern "C" int vaq_fp8_quant_per_token_tuned(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out,
                                             int64_t out_row_stride, float* scales, const float* scale_ub, int64_t rows,
                                             int64_t hidden, void* stream, const VaqTuning* tuning_or_null) {
  using namespace vaq;
  const TuningScope scope(tuning_or_null);
  int rc = check_quant("fp8_quant_per_token", in, in_row_stride, out, out_row_stride, scales, rows, hidden);
  if (rc != VAQ_OK || rows == 0) return rc;
  // Measured: a row per wavefront is 1.1-1.6x faster for short rows in large batches; with few rows a whole workgroup
  // per row has the shorter latency, and from 4096 elements on the 64 registers of row data per lane cost more than the
  // barriers saved.
  const bool many_short_rows = hidden <= 1024 ? rows >= 1024 : (hidden <= 2048 && rows >= 2048);
  const int force = tuning().quant_wg_per_row;      // 1: a workgroup per row, 2: a wavefront per row where it can run
  if ((force == 2 || (force == 0 && many_short_rows)) &&
      row_per_wave_ok(in, in_dtype, in_row_stride, out, out_row_stride, hidden)) {
    if (in_dtype == VAQ_BF16)
      launch_row_per_wave<bf16_t>(in, in_row_stride, out, out_row_stride, scales, scale_ub, rows, hidden, (hipStream_t)stream);
    else
      launch_row_per_wave<f16_t>(in, in_row_stride, out, out_row_stride, scales, scale_ub, rows, hidden, (hipStream_t)stream);
  } else {
    rc = launch_quant<0>(in, in_dtype, in_row_stride, out, out_row_stride, scales, scale_ub, rows, hidden,
                         (hipStream_t)stream);
    if (rc != VAQ_OK) return rc;
  }
  VAQ_CHECK_LAUNCH("fp8_quant_per_token");
  return VAQ_OK;
}

extern "C" int vaq_fp8_quant_static(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out,
                                    int64_t out_row_stride, const float* scale, int64_t rows, int64_t hidden,
                                    void* stream) {
  using namespace vaq;
  int rc = check_quant("fp8_quant_static", in, in_row_stride, out, out_row_stride, scale, rows, hidden);
  if (rc != VAQ_OK || rows == 0) return rc;
  rc = launch_quant<1>(in, in_dtype, in_row_stride, out, out_row_stride, const_cast<float*>(scale), nullptr, rows,
                       hidden, (hipStream_t)stream);
  if (rc != VAQ_OK) return rc;
  VAQ_CHECK_LAUNCH("fp8_quant_static");
  return VAQ_OK;
}

extern "C" int vaq_fp8_quant_dynamic(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out,
                                     int64_t out_row_stride, float* scale, int64_t rows, int64_t hidden,
                                     void* stream) {
  using namespace vaq;
  int rc = check_quant("fp8_quant_dynamic", in, in_row_stride, out, out_row_stride, scale, rows, hidden);
  if (rc != VAQ_OK || rows == 0) return rc;
  hipStream_t s = (hipStream_t)stream;
  // the running maximum starts from zero; a one-thread kernel rather than a memset node keeps the call graph-capturable
  hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(1), 0, s, scale);
  rc = launch_quant<2>(in, in_dtype, in_row_stride, out, out_row_stride, scale, nullptr, rows, hidden, s);
  if (rc != VAQ_OK) return rc;
  rc = launch_quant<1>(in, in_dtype, in_row_stride, out, out_row_stride, scale, nullptr, rows, hidden, s);
  if (rc != VAQ_OK) return rc;
  VAQ_CHECK_LAUNCH("fp8_quant_dynamic");
  return VAQ_OK;
}
