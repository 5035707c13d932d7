/*
 * vllm_amd_qlinear.h -- C ABI of the MI355X (gfx950) quantized-linear library
 * (GPTQ W4A16 + FP8 W8A8).  One shared object: vllm_amd/libvllm_amd_qlinear.so.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless the name ends in _host;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *  - the library never allocates device memory, never synchronises the device
 *    and throws nothing: each call validates its arguments on the host,
 *    enqueues work on `stream` and returns VAQ_OK or a negative status, the
 *    text for which is returned by vaq_last_error() (thread local);
 *  - dtype tags: VAQ_F16 / VAQ_BF16 for 16-bit activations and outputs.
 *
 * Every entry point cites the reference interface it stands in for
 * (paths relative to the reference tree).
 */
#ifndef VLLM_AMD_QLINEAR_H_
#define VLLM_AMD_QLINEAR_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The library is built with hidden visibility; only what this header declares is exported. */
#pragma GCC visibility push(default)

#define VAQ_OK 0
#define VAQ_ERR_INVALID_ARG (-1)   /* shape / stride / alignment / enum check failed (TORCH_CHECK analogue)   */
#define VAQ_ERR_UNSUPPORTED (-2)   /* valid request outside what is built (TORCH_CHECK_NOT_IMPLEMENTED analogue) */
#define VAQ_ERR_LAUNCH (-3)        /* the HIP runtime refused the launch                                       */

#define VAQ_F16 0
#define VAQ_BF16 1
#define VAQ_F32 2

/* Weight layouts produced by vaq_w4a16_repack (both are int32 [K/16, 2N], same bytes). */
#define VAQ_LAYOUT_MARLIN 0 /* the reference's Marlin tile order, bit-exact with gptq_marlin_repack   */
#define VAQ_LAYOUT_NATIVE 1 /* wavefront tile order consumed by vaq_w4a16_gemm (K % 128 == 0 needed) */
#define VAQ_LAYOUT_NATIVE_BYTES 2 /* num_bits 8 only: the same tiles with whole bytes, for wtype FE4M3    */

/* Weight code types (what b_q_type.id selects in the reference, vllm/scalar_type.py:327-351). */
#define VAQ_WTYPE_U4B8 0 /* symmetric: code - 8            */
#define VAQ_WTYPE_U4 1   /* asymmetric: code - zeros[g][n] */
#define VAQ_WTYPE_U8B128 2 /* 8-bit symmetric: code - 128 (weights from vaq_w4a16_repack with num_bits = 8) */
#define VAQ_WTYPE_FE4M3 3  /* FP8 e4m3fn weights, 16-bit activations (the reference's weight-only FP8 path,
                              marlin_utils_fp8.py); weights from vaq_w4a16_repack with num_bits = 8 and
                              VAQ_LAYOUT_NATIVE_BYTES; group_size -1 or 128, no zero points, no act_order */

/* Text of the last error on the calling thread ("" if none). */
const char* vaq_last_error(void);

/* Library / device facts.  vaq_num_cus: compute units of `device` (>0) or a negative status. */
int vaq_abi_version(void);
int vaq_num_cus(int device);

/*
 * GPTQ int4 / int8 repack.  Replaces `gptq_marlin_repack(Tensor b_q_weight, Tensor perm, SymInt size_k,
 * SymInt size_n, int num_bits) -> Tensor` (csrc/torch_bindings.cpp:320-321; device code
 * csrc/quantization/gptq_marlin/gptq_marlin_repack.cu:7-322).
 *   qweight  int32 [size_k/8, size_n] contiguous (8 nibbles along K per word); num_bits 8: [size_k/4, size_n], 4 bytes
 *   perm     int32 [size_k] act_order sort indices (output row r takes input row perm[r]) or NULL
 *   out      int32 [size_k/16, 2*size_n]; num_bits 8: [size_k/16, 4*size_n]
 * num_bits must be 4 or 8.  size_k % 16 == 0, size_n % 64 == 0 (NATIVE additionally size_k % 128 == 0).
 */
int vaq_w4a16_repack(const int32_t* qweight, const int32_t* perm, int32_t* out, int64_t size_k, int64_t size_n,
                     int num_bits, int layout, void* stream);

/*
 * AWQ int4 repack.  Replaces `awq_marlin_repack(Tensor b_q_weight, SymInt size_k, SymInt size_n, int num_bits)
 * -> Tensor` (csrc/torch_bindings.cpp:325-327; device code csrc/quantization/gptq_marlin/awq_marlin_repack.cu:7-268).
 *   qweight  int32 [size_k, size_n/8] contiguous (AutoAWQ: 8 nibbles along N per word, column 8c+{0,2,4,6,1,3,5,7}[p]
 *            in nibble position p)
 *   out      int32 [size_k/16, 2*size_n], same two layouts and the same size rules as vaq_w4a16_repack
 */
int vaq_w4a16_repack_awq(const int32_t* qweight, int32_t* out, int64_t size_k, int64_t size_n, int num_bits, int layout,
                         void* stream);

/*
 * Zero-point repack for the NATIVE layout: GPTQ/compressed-tensors `qzeros` values, packed 8 per int32 along N
 * in natural order, are what vaq_w4a16_gemm reads, so no device work is needed and no entry point exists for
 * it; the reference's marlin_zero_points (marlin_utils.py:326-346) is reproduced on the host side only.
 */

/*
 * Scratch the caller must hand to vaq_w4a16_gemm for a given problem, in bytes:
 *   *c_tmp_bytes   fp32 split-K partials   (reference: c_tmp, gptq_marlin.cu:752-763)
 *   *a_tmp_bytes   permuted activations    (reference: a_tmp, gptq_marlin.cu:799); 0 when has_perm == 0
 *   *counter_ints  int32 arrival counters that must be ZERO on entry and are left zero
 *                  (reference: `workspace`, marlin_utils.py:237-245, marlin_template.h:225-271)
 */
int vaq_w4a16_gemm_workspace(int64_t size_m, int64_t size_n, int64_t size_k, int has_perm, int device,
                             size_t* c_tmp_bytes, size_t* a_tmp_bytes, size_t* counter_ints);

/*
 * W4A16 GEMM  C[M,N] = A[:, perm] . dequant(B) (+ bias), fp32 accumulation, one rounding to the 16-bit dtype.
 * Replaces `gptq_marlin_gemm(...)` (csrc/torch_bindings.cpp:309-315; csrc/quantization/gptq_marlin/gptq_marlin.cu:674-959).
 *   a        [M, K] 16-bit, row stride lda elements (lda % 8 == 0, base 16-byte aligned), unit column stride
 *   b        NATIVE-layout weights from vaq_w4a16_repack (num_bits 8 for wtype U8B128)
 *   scales   [K/group_size, N] ([1, N] for group_size -1) in the activation dtype, contiguous
 *   zeros    int32 [K/group_size, N/8] ([1, N/8] for -1) natural nibble order (wtype U4) or NULL (wtype U4B8)
 *   perm     int32 [K] act_order sort indices or NULL  (is_k_full semantics: group of sorted row r is r / group_size)
 *   bias     [N] activation dtype or NULL
 *   c        [M, N] activation dtype, contiguous
 *   group_size  128, 64, 32, or -1 / K for channelwise scales (the reference's MARLIN_SUPPORTED_GROUP_SIZES,
 *               marlin_utils.py:24), for every wtype; anything else returns VAQ_ERR_UNSUPPORTED
 * M == 0 is a no-op.  Kernel choice (decode: M <= 32, up to 64 for 4-bit codes in groups of 128 rows or channelwise --
 * up to 256 on layers narrow enough that workgroups of 16 rows each make one round -- MFMA GEMV with in-register
 * dequant; prefill: tile kernels, weights dequantised through LDS or in registers)
 * is internal; `force_path` = 0 auto, 1 decode (M <= 64 at most), 2 prefill (tests / benchmarks).
 * Scratch: `c_tmp` holds at least `c_tmp_bytes` bytes and `counters` at least `counter_ints` zeroed ints; a call whose
 * kernel needs more than it was given returns VAQ_ERR_INVALID_ARG (sizes: vaq_w4a16_gemm_workspace) and launches nothing.
 * One use of `c_tmp` is optional: at thousands of rows, 256 x 256 tiles that end in a round of workgroups at most half
 * full run the tiles of that round in K parts when `c_tmp` holds their partial tiles, and whole (same result, slower)
 * when it does not -- the workspace query reports the size with that use included.
 */
int vaq_w4a16_gemm(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                   const int32_t* perm, const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes, void* a_tmp,
                   int32_t* counters, int64_t counter_ints, int64_t size_m, int64_t size_n, int64_t size_k,
                   int group_size, int dtype, int wtype, int force_path, void* stream);

/*
 * vaq_w4a16_gemm on scratch the library owns, for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference, whose GEMM allocates its
 * scratch through the torch allocator (gptq_marlin.cu:752-763, :799).  Same arguments, results and kernels as
 * vaq_w4a16_gemm with force_path 0; the partial tiles, permuted activations and arrival counters live in one
 * file-scope device array of VAQ_STATIC_SCRATCH_COUNTER_INTS ints + VAQ_STATIC_SCRATCH_DATA_BYTES bytes per GPU, which
 * a GPU holds from the library's first use on it until the process ends.  The call allocates and frees nothing.
 * A problem whose scratch (vaq_w4a16_gemm_workspace, without the optional use of c_tmp described above, which this
 * entry point never makes) exceeds that returns VAQ_ERR_INVALID_ARG and launches nothing.
 * Every call on a GPU uses that GPU's one array: calls that may overlap in time on one GPU (different streams or
 * threads) race on it and must be serialised by the caller.  The first call on a GPU looks the array's address up
 * (hipGetSymbolAddress); make it outside any graph capture.
 */
#define VAQ_STATIC_SCRATCH_COUNTER_INTS 65536
#define VAQ_STATIC_SCRATCH_DATA_BYTES (16u << 20)
int vaq_w4a16_gemm_static(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                          const int32_t* perm, const void* bias, void* c, int64_t size_m, int64_t size_n, int64_t size_k,
                          int group_size, int dtype, int wtype, void* stream);

/*
 * out[m, k] = a[m, perm[k]] for 16-bit elements.  Replaces `permute_cols(Tensor A, Tensor perm) -> Tensor`
 * (csrc/torch_bindings.cpp:304; csrc/permute_cols.cu:13-87).
 */
int vaq_permute_cols(const void* a, int64_t lda, const int32_t* perm, void* out, int64_t size_m, int64_t size_k,
                     void* stream);

/*
 * FP8 (OCP e4m3fn) activation quantisation.  `in` is [rows, hidden] F16/BF16/F32 with unit column stride and
 * row stride in_row_stride (elements); `out` is uint8 codes with row stride out_row_stride.
 *
 * vaq_fp8_quant_per_token  replaces `dynamic_per_token_scaled_fp8_quant(Tensor! result, Tensor input, Tensor! scale,
 *     Tensor? scale_ub)` (csrc/torch_bindings.cpp:585-587; csrc/quantization/w8a8/fp8/common.cu:91-131, :213-247):
 *     scales[r] = max(min(amax_r, *scale_ub) / 448, 1/(448*512));  out = cvt(clamp(x / scales[r], +-448))  (true division)
 * vaq_fp8_quant_static     replaces `static_scaled_fp8_quant(Tensor! result, Tensor input, Tensor scale)` (:572; common.cu:11-30, :136-170):
 *     out = cvt(clamp(x * (1 / *scale), +-448))
 * vaq_fp8_quant_dynamic    replaces `dynamic_scaled_fp8_quant(Tensor! result, Tensor input, Tensor! scale)` (:578; common.cu:32-89, :172-211):
 *     *scale = max_all|x| / 448 (written by the call), then as static.
 */
int vaq_fp8_quant_per_token(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out, int64_t out_row_stride,
                            float* scales, const float* scale_ub, int64_t rows, int64_t hidden, void* stream);
int vaq_fp8_quant_static(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out, int64_t out_row_stride,
                         const float* scale, int64_t rows, int64_t hidden, void* stream);
int vaq_fp8_quant_dynamic(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out, int64_t out_row_stride,
                          float* scale, int64_t rows, int64_t hidden, void* stream);

/*
 * FP8 scaled GEMM  out[m,n] = round(sa[m] * (sb[n] * sum_k a[m,k] b[k,n]) + bias[n]).
 * Replaces `cutlass_scaled_mm(Tensor! out, Tensor a, Tensor b, Tensor a_scales, Tensor b_scales, Tensor? bias)`
 * (csrc/torch_bindings.cpp:412-414; csrc/quantization/w8a8/cutlass/scaled_mm_entry.cu:175-245; epilogue
 * csrc/cutlass_extensions/epilogue/scaled_mm_epilogues_c3x.hpp:136-216).
 *   a     e4m3fn [M, K] row-major, row stride lda bytes (lda % 16 == 0)
 *   b     e4m3fn [K, N] COLUMN-major: element (k, n) at b[n * ldb + k]   (ldb % 16 == 0; ldb may exceed K)
 *   sa    fp32, sa_count == 1 (per tensor) or M (per token);  sb fp32, sb_count == 1 or N (per channel)
 *   bias  [N] of out dtype or NULL;  out [M, N] F16/BF16, row stride ldc elements (ldc % 8 == 0)
 * K % 16 == 0 and N % 16 == 0 required (as the reference's cutlass path, vllm/_custom_ops.py:790-791).
 */
int vaq_fp8_scaled_mm(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb, const float* sa, int64_t sa_count,
                      const float* sb, int64_t sb_count, const void* bias, void* out, int64_t ldc, int out_dtype,
                      int64_t size_m, int64_t size_n, int64_t size_k, void* stream);

/*
 * RMSNorm (+ residual add) fused with dynamic per-token FP8 quantisation.  Replaces
 * `rms_norm_dynamic_per_token_quant(Tensor! result, Tensor input, Tensor weight, Tensor! scale, float epsilon,
 * Tensor? scale_ub, Tensor!? residual)` (csrc/torch_bindings.cpp:216-221; device code
 * csrc/quantization/fused_kernels/fused_layernorm_dynamic_per_token_quant.cu, layernorm_utils.cuh:17-130) for FP8 output.
 *   out       e4m3fn [tokens, hidden] contiguous;  scales fp32 [tokens]
 *   input     [tokens, hidden] F16/BF16, row stride in_stride elements;  weight [hidden] same dtype
 *   scale_ub  optional fp32 scalar (device);  residual optional [tokens, hidden] contiguous, updated in place with
 *             input + residual
 */
int vaq_rms_norm_dynamic_per_token_fp8_quant(uint8_t* out, float* scales, const void* input, int64_t in_stride,
                                             const void* weight, const float* scale_ub, float epsilon, void* residual,
                                             int dtype, int64_t tokens, int64_t hidden, void* stream);

/*
 * RMSNorm (+ residual add) fused with static per-tensor FP8 quantisation.  With residual == NULL replaces
 * `rms_norm_static_fp8_quant(Tensor! result, Tensor input, Tensor weight, Tensor scale, float epsilon)`
 * (csrc/torch_bindings.cpp:200-205, device code csrc/layernorm_quant_kernels.cu:21-66); with a residual replaces
 * `fused_add_rms_norm_static_fp8_quant(Tensor! result, Tensor input, Tensor! residual, Tensor weight, Tensor scale,
 * float epsilon)` (csrc/torch_bindings.cpp:208-213, csrc/layernorm_quant_kernels.cu:72-178): residual is updated in
 * place with input + residual, input is left untouched.
 *   out  e4m3fn [tokens, hidden] contiguous;  input row stride in_stride elements;  scale fp32 scalar (device)
 */
int vaq_rms_norm_static_fp8_quant(uint8_t* out, const void* input, int64_t in_stride, const void* weight,
                                  const float* scale, float epsilon, void* residual, int dtype, int64_t tokens,
                                  int64_t hidden, void* stream);

/*
 * out[t, i] = fp8(silu(input[t, i]) * input[t, d + i] / scale).  Replaces
 * `silu_and_mul_quant(Tensor! result, Tensor input, Tensor scale)` (csrc/torch_bindings.cpp:121-123, device code
 * csrc/quantization/activation_kernels.cu:35-119, 560-568).
 *   out  e4m3fn [tokens, d] contiguous;  input [tokens, 2*d] F16/BF16 contiguous;  scale fp32 scalar (device)
 */
int vaq_silu_and_mul_fp8_quant(uint8_t* out, const void* input, const float* scale, int dtype, int64_t tokens, int64_t d,
                               void* stream);

/*
 * The same GEMM with caller-provided scratch, which lets the tile kernel split K over workgroups when M and N alone
 * leave compute units idle (up to a few hundred tokens on the narrow layers), and the weight-streaming kernel run
 * 17 .. 32 tokens with K beyond 8192 (up to 16384) as two halves of K.  Sizes come from the query; both may be 0.
 *   c_tmp     fp32 partial tiles, 16-byte aligned, contents irrelevant on entry
 *   counters  int32 arrival counters that must be ZERO on entry and are left zero (calls sharing them must not overlap)
 * With NULL / too small scratch the call behaves exactly like vaq_fp8_scaled_mm.  (The reference's cutlass_scaled_mm has
 * no workspace argument: CUTLASS allocates its own, scaled_mm_entry.cu.)
 */
int vaq_fp8_scaled_mm_workspace(int64_t size_m, int64_t size_n, int64_t size_k, size_t* c_tmp_bytes,
                                size_t* counter_ints);
int vaq_fp8_scaled_mm_ws(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb, const float* sa, int64_t sa_count,
                         const float* sb, int64_t sb_count, const void* bias, void* out, int64_t ldc, int out_dtype,
                         int64_t size_m, int64_t size_n, int64_t size_k, float* c_tmp, int64_t c_tmp_bytes,
                         int32_t* counters, int64_t counter_ints, void* stream);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif
#endif /* VLLM_AMD_QLINEAR_H_ */
