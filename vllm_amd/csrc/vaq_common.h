// Shared host/device helpers for the gfx950 quantized-linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/vllm_amd_qlinear.h"
#include "vaq_tuning.h"

namespace vaq {

// ----------------------------------------------------------------------------- host: error reporting
void set_error(const char* fmt, ...);   // defined in api.hip (thread-local buffer)

#define VAQ_CHECK_ARG(cond, ...)            \
  do {                                      \
    if (!(cond)) {                          \
      ::vaq::set_error(__VA_ARGS__);        \
      return VAQ_ERR_INVALID_ARG;           \
    }                                       \
  } while (0)

#define VAQ_CHECK_SUPPORTED(cond, ...)      \
  do {                                      \
    if (!(cond)) {                          \
      ::vaq::set_error(__VA_ARGS__);        \
      return VAQ_ERR_UNSUPPORTED;           \
    }                                       \
  } while (0)

#define VAQ_CHECK_LAUNCH(what)                                                     \
  do {                                                                             \
    hipError_t e__ = hipGetLastError();                                            \
    if (e__ != hipSuccess) {                                                       \
      ::vaq::set_error("%s: launch failed: %s", what, hipGetErrorString(e__));     \
      return VAQ_ERR_LAUNCH;                                                       \
    }                                                                              \
  } while (0)

int num_cus_current_device();   // cached per device, api.hip

// Kernel-variant overrides of the `_tuned` entry points (tests, benchmarks).  An entry point opens a TuningScope with
// the caller's struct; the host code below it reads `tuning()`, which is all zeros (= automatic) outside a scope.  The
// pointer lives in a thread-local for the duration of that one call: nothing persists between calls or crosses threads.
const VaqTuning& tuning();
class TuningScope {
 public:
  explicit TuningScope(const VaqTuning* t);
  ~TuningScope();
  TuningScope(const TuningScope&) = delete;
  TuningScope& operator=(const TuningScope&) = delete;

 private:
  const VaqTuning* prev_;
};

// Dynamic LDS above the default limit has to be reserved per kernel and per device.  `reserved` is the calling launch
// function's own static array (one per kernel instantiation, zero-initialised): bytes already reserved on each device.
// The attribute is idempotent, so two threads racing here at worst set it twice.
constexpr int VAQ_MAX_DEVICES = 64;
inline int reserve_dynamic_lds(const void* kern, size_t lds, size_t (&reserved)[VAQ_MAX_DEVICES], const char* what) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= VAQ_MAX_DEVICES) {
    set_error("%s: cannot identify the current device", what);
    (void)hipGetLastError();
    return VAQ_ERR_LAUNCH;
  }
  if (lds <= reserved[dev]) return VAQ_OK;
  if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
    set_error("%s: cannot reserve %zu bytes of LDS", what, lds);
    (void)hipGetLastError();
    return VAQ_ERR_LAUNCH;
  }
  reserved[dev] = lds;
  return VAQ_OK;
}

// ----------------------------------------------------------------------------- device: exact division
// x / s, correctly rounded, for x that came from a 16-bit float (bf16 or fp16) and r = 1.0f / s (IEEE division, done
// once per row): the product with the reciprocal is within one step of the quotient, the fused multiply-add forms its
// residual exactly, and one more fused multiply-add lands on the correctly rounded quotient.  Checked against the IEEE
// division for every significand of s and every 7- and 10-bit significand of x (tests/native/exact_div_check.c).
// Three instructions instead of the ten of the general division.  Needs |x / s| and |x| inside the normal range and a
// finite s (callers take the general division otherwise); signed zeros keep their sign.
// The two fused operations are written as instructions: merged into one expression a compiler may rewrite
// -(q*s - x) as (-q)*s + x, which loses the sign of a zero residual (x = -0 must give -0, the code 0x80).
// None of the operands may come straight out of a transcendental instruction (v_rcp_f32, v_exp_f32, v_rsq_f32 ...):
// the wait state that such a result needs before its first use is inserted by the compiler for its own instructions
// only, not in front of inline assembly.  The callers form r by the IEEE division, which ends in v_div_fixup_f32.
__device__ inline float div16_exact(float x, float s, float r) {
  float q, e, o;
  asm("v_mul_f32 %0, %1, %2" : "=v"(q) : "v"(x), "v"(r));
  asm("v_fma_f32 %0, %1, %2, -%3" : "=v"(e) : "v"(q), "v"(s), "v"(x));
  asm("v_fma_f32 %0, -%1, %2, %3" : "=v"(o) : "v"(e), "v"(r), "v"(q));
  return o;
}

// ----------------------------------------------------------------------------- device: vector types
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

// 16-bit float handling is done on raw bit patterns so that bf16 and fp16 share one code path.
template <bool BF16>
struct F16Traits;

template <>
struct F16Traits<true> {
  // (code & 0xF) | EX is the bf16 number 128 + code (7 mantissa bits, exponent 2^7).
  static constexpr uint32_t EX = 0x43004300u;
  static constexpr float CODE_BIAS = 128.0f;
  __device__ static inline float to_float(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
  __device__ static inline uint16_t from_float(float f) {   // v_cvt_pk_bf16_f32: round-to-nearest-even, NaN stays NaN
    return __builtin_bit_cast(uint16_t, (__bf16)f);
  }
  __device__ static inline v4f mfma16(v4u a, v4u b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
  __device__ static inline v16f mfma32(v4u a, v4u b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
  static constexpr uint32_t ONE2 = 0x3f803f80u;   // packed (1.0, 1.0)
};

template <>
struct F16Traits<false> {
  // (code & 0xF) | EX is the fp16 number 1024 + code (10 mantissa bits, exponent 2^10).
  static constexpr uint32_t EX = 0x64006400u;
  static constexpr float CODE_BIAS = 1024.0f;
  __device__ static inline float to_float(uint16_t h) {
    _Float16 x = __builtin_bit_cast(_Float16, h);
    return (float)x;
  }
  __device__ static inline uint16_t from_float(float f) {
    _Float16 x = (_Float16)f;   // v_cvt_f16_f32: round-to-nearest-even
    return __builtin_bit_cast(uint16_t, x);
  }
  __device__ static inline v4f mfma16(v4u a, v4u b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
  __device__ static inline v16f mfma32(v4u a, v4u b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
  static constexpr uint32_t ONE2 = 0x3c003c00u;
};

// One native-layout weight word (8 codes, nibble p holds element {0,2,4,6,1,3,5,7}[p]) -> 8 consecutive 16-bit
// numbers CODE_BIAS + code, i.e. one 16x16x32 MFMA operand register quad.
template <bool BF16>
__device__ inline v4u dequant_biased(uint32_t w) {
  constexpr uint32_t M = 0x000f000fu, EX = F16Traits<BF16>::EX;
  v4u r;
  r.x = (w & M) | EX;
  r.y = ((w >> 4) & M) | EX;
  r.z = ((w >> 8) & M) | EX;
  r.w = ((w >> 12) & M) | EX;
  return r;
}

}  // namespace vaq
