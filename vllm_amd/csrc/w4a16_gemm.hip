// C-ABI entry of the W4A16 GEMM: argument validation and the decode / prefill dispatch.
#include "vaq_common.h"

#include <mutex>

namespace vaq {
// `sub` = quantisation groups per 128-row weight tile (1, 2, 4); `channelwise` = one scale row for all of K (sub == 1)
int w4a16_decode_workspace(int M, int N, int K, size_t* c_tmp_bytes, size_t* counter_ints);
int w4a16_decode_launch(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                        const int32_t* perm, const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes,
                        int32_t* counters, int64_t counter_ints, int M, int N, int K, bool channelwise, int dtype,
                        hipStream_t s);
int w4a16_decode2_workspace(int M, int N, int K, int sub, bool w8, size_t* c_tmp_bytes, size_t* counter_ints);
bool w4a16_decode2_takes_rows(int M, int N, int K, int sub, int wt, bool has_perm);
int w4a16_decode2_launch(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                         const int32_t* perm, const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes,
                         int32_t* counters, int64_t counter_ints, int M, int N, int K, int sub, bool channelwise,
                         int wt, int dtype, hipStream_t s);      // wt: 0 4-bit codes, 1 8-bit codes, 2 FP8 e4m3 bytes
int w4a16_prefill_workspace(int M, int N, int K, size_t* c_tmp_bytes, size_t* counter_ints);
int w4a16_prefill_launch(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                         const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes, int32_t* counters,
                         int64_t counter_ints, int M, int N, int K, int sub, bool channelwise, int wt, int dtype,
                         hipStream_t s);

constexpr int64_t DECODE_MAX_M = 64;          // up to four m-blocks of 16 rows on the LDS-staged kernel
constexpr int64_t DECODE_MAX_M_2BLK = 32;     // the register-resident kernel, groups below 128 rows and 8-bit codes: two

// Measured on MI355X (cold weights): staging the activations once per workgroup in LDS (one independent task per
// wavefront, no barrier in the K loop) wins on every Llama-3-8B projection and on 8192 x 28672 (30 us against 43.5 us
// for 3 <= M <= 16).  The register-resident kernel, whose wavefronts walk over n-tiles with their slice of the
// activations held in registers, stays ahead only on a vocabulary-sized layer (4096 x 128256, 3 <= M <= 16: 55 us
// against 62 us).
static int decode_impl_for(int64_t size_m, int64_t size_n, int64_t lda, int sub, bool w8) {
  // the LDS-staged kernel addresses A through a 32-bit buffer offset
  if (size_m * lda * 2 >= (1ll << 31)) return 1;
  if (sub > 1 || w8) return 0;    // groups below 128 rows and 8-bit codes are built for the LDS-staged kernel only
  if (tuning().decode_impl > 0) return tuning().decode_impl - 1;   // tests / benchmarks: 1 LDS-staged, 2 register-resident
  return (size_n >= 65536 && size_m > 2 && size_m <= 16) ? 1 : 0;
}

static int check_shape(int64_t size_m, int64_t size_n, int64_t size_k) {
  VAQ_CHECK_ARG(size_m >= 0, "w4a16_gemm: size_m = %lld is negative", (long long)size_m);
  VAQ_CHECK_ARG(size_n > 0 && size_n % 64 == 0, "w4a16_gemm: size_n = %lld, is not divisible by min_thread_n = 64",
                (long long)size_n);
  VAQ_CHECK_ARG(size_k > 0 && size_k % 128 == 0, "w4a16_gemm: size_k = %lld, is not divisible by min_thread_k = 128",
                (long long)size_k);
  VAQ_CHECK_ARG(size_m < (1ll << 31) && size_n < (1ll << 31) && size_k < (1ll << 31) &&
                    size_k * size_n / 2 < (1ll << 32),
                "w4a16_gemm: problem too large");   // (8-bit weights: K*N bytes, still below 2^33; offsets are checked per kernel)
  return VAQ_OK;
}
}  // namespace vaq

extern "C" int vaq_w4a16_gemm_workspace(int64_t size_m, int64_t size_n, int64_t size_k, int has_perm, int device,
                                        size_t* c_tmp_bytes, size_t* a_tmp_bytes, size_t* counter_ints) {
  return vaq_w4a16_gemm_workspace_tuned(size_m, size_n, size_k, has_perm, device, c_tmp_bytes, a_tmp_bytes, counter_ints,
                                        nullptr);
}

extern "C" int vaq_w4a16_gemm_workspace_tuned(int64_t size_m, int64_t size_n, int64_t size_k, int has_perm, int device,
                                              size_t* c_tmp_bytes, size_t* a_tmp_bytes, size_t* counter_ints,
                                              const VaqTuning* tuning_or_null) {
  using namespace vaq;
  (void)device;
  const TuningScope scope(tuning_or_null);
  VAQ_CHECK_ARG(c_tmp_bytes && a_tmp_bytes && counter_ints, "w4a16_gemm_workspace: null output pointer");
  int rc = check_shape(size_m, size_n, size_k);
  if (rc != VAQ_OK) return rc;
  *c_tmp_bytes = 0;
  *a_tmp_bytes = 0;
  *counter_ints = 0;
  if (size_m == 0) return VAQ_OK;
  if (size_m <= DECODE_MAX_M) {
    // Enough for whichever kernel runs: that also depends on the row stride of A, the group size and the weight type,
    // all unknown here.
    size_t t = 0, n = 0, t2 = 0, n2 = 0;
    auto take = [&]() {
      if (t2 > t) t = t2;
      if (n2 > n) n = n2;
    };
    rc = w4a16_decode2_workspace((int)size_m, (int)size_n, (int)size_k, 1, false, &t2, &n2);
    if (rc != VAQ_OK) return rc;
    take();
    if (size_m <= DECODE_MAX_M_2BLK) {
      rc = w4a16_decode_workspace((int)size_m, (int)size_n, (int)size_k, &t2, &n2);
      if (rc != VAQ_OK) return rc;
      take();
      rc = w4a16_decode2_workspace((int)size_m, (int)size_n, (int)size_k, 2, false, &t2, &n2);   // groups below 128 rows
      if (rc != VAQ_OK) return rc;
      take();
      rc = w4a16_decode2_workspace((int)size_m, (int)size_n, (int)size_k, 1, true, &t2, &n2);    // 8-bit codes
      if (rc != VAQ_OK) return rc;
      take();
    } else {
      // those cases take the prefill kernel above 32 rows
      rc = w4a16_prefill_workspace((int)size_m, (int)size_n, (int)size_k, &t2, &n2);
      if (rc != VAQ_OK) return rc;
      take();
      if (has_perm) *a_tmp_bytes = (size_t)size_m * (size_t)size_k * 2;
    }
    *c_tmp_bytes = t;
    *counter_ints = n;
    return VAQ_OK;
  }
  if (has_perm) *a_tmp_bytes = (size_t)size_m * (size_t)size_k * 2;
  return w4a16_prefill_workspace((int)size_m, (int)size_n, (int)size_k, c_tmp_bytes, counter_ints);
}

extern "C" int vaq_w4a16_gemm(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                              const int32_t* perm, const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes,
                              void* a_tmp, int32_t* counters, int64_t counter_ints, int64_t size_m, int64_t size_n,
                              int64_t size_k, int group_size, int dtype, int wtype, int force_path, void* stream) {
  return vaq_w4a16_gemm_tuned(a, lda, b, scales, zeros, perm, bias, c, c_tmp, c_tmp_bytes, a_tmp, counters, counter_ints,
                              size_m, size_n, size_k, group_size, dtype, wtype, force_path, stream, nullptr);
}

extern "C" int vaq_w4a16_gemm_tuned(const void* a, int64_t lda, const int32_t* b, const void* scales,
                                    const int32_t* zeros, const int32_t* perm, const void* bias, void* c, float* c_tmp,
                                    int64_t c_tmp_bytes, void* a_tmp, int32_t* counters, int64_t counter_ints,
                                    int64_t size_m, int64_t size_n, int64_t size_k, int group_size, int dtype, int wtype,
                                    int force_path, void* stream, const VaqTuning* tuning_or_null) {
  using namespace vaq;
  const TuningScope scope(tuning_or_null);
  VAQ_CHECK_ARG(c_tmp_bytes >= 0 && counter_ints >= 0, "w4a16_gemm: negative scratch size");
  int rc = check_shape(size_m, size_n, size_k);
  if (rc != VAQ_OK) return rc;
  VAQ_CHECK_ARG(dtype == VAQ_F16 || dtype == VAQ_BF16, "w4a16_gemm: only supports bfloat16 and float16 (dtype tag %d)",
                dtype);
  VAQ_CHECK_ARG(wtype == VAQ_WTYPE_U4B8 || wtype == VAQ_WTYPE_U4 || wtype == VAQ_WTYPE_U8B128 || wtype == VAQ_WTYPE_FE4M3,
                "w4a16_gemm: unknown weight type tag %d", wtype);
  VAQ_CHECK_ARG((wtype == VAQ_WTYPE_U4) == (zeros != nullptr),
                "w4a16_gemm: b_q_type must be uint4 when has_zp = True and uint4b8, uint8b128 or float8_e4m3fn when has_zp = False");
  const int wt = wtype == VAQ_WTYPE_U8B128 ? 1 : (wtype == VAQ_WTYPE_FE4M3 ? 2 : 0);
  const bool w8 = wt != 0;
  const bool channelwise = group_size == -1 || (group_size == size_k && size_k != 128);
  VAQ_CHECK_SUPPORTED(channelwise || group_size == 128 || group_size == 64 || group_size == 32,
                      "w4a16_gemm: group_size = %d is not built (only -1, 32, 64, 128)", group_size);
  const int sub = channelwise ? 1 : 128 / group_size;
  VAQ_CHECK_SUPPORTED(wt != 2 || (sub == 1 && perm == nullptr),
                      "w4a16_gemm: FP8 weights take channelwise scales or groups of 128 rows, and no act_order");
  VAQ_CHECK_ARG(!w8 || size_k * size_n < (1ll << 32), "w4a16_gemm: problem too large for 8-bit weights");
  VAQ_CHECK_ARG(force_path >= 0 && force_path <= 2, "w4a16_gemm: force_path = %d", force_path);
  if (size_m == 0) return VAQ_OK;
  VAQ_CHECK_ARG(a && b && scales && c, "w4a16_gemm: null pointer");
  VAQ_CHECK_ARG(lda >= size_k && lda % 8 == 0, "w4a16_gemm: A.stride(0) = %lld must be >= size_k and divisible by 8",
                (long long)lda);
  VAQ_CHECK_ARG(((uintptr_t)a % 16) == 0, "w4a16_gemm: A must aligned to 16 bytes");
  VAQ_CHECK_ARG(((uintptr_t)b % 16) == 0 && ((uintptr_t)scales % 8) == 0 && ((uintptr_t)c % 8) == 0,
                "w4a16_gemm: b_q_weight must be 16-byte, b_scales and c 8-byte aligned");
  VAQ_CHECK_ARG(!perm || ((uintptr_t)perm % 16) == 0, "w4a16_gemm: perm must be 16-byte aligned");
  VAQ_CHECK_ARG(!bias || ((uintptr_t)bias % 8) == 0, "w4a16_gemm: bias must be 8-byte aligned");
  hipStream_t s = (hipStream_t)stream;

  // three and four m-blocks exist on the LDS-staged kernel for 4-bit codes in groups of 128 rows / channelwise
  const bool two_blocks_only = sub > 1 || w8 || decode_impl_for(size_m, size_n, lda, sub, w8) != 0;
  // (measured: four m-blocks beat the tile kernel by 1.5-2x on the narrow layers and lose 3 % on a 28672-wide one)
  const int64_t dec_max = two_blocks_only ? DECODE_MAX_M_2BLK : (size_n > 8192 ? 48 : DECODE_MAX_M);
  bool decode = size_m <= dec_max;
  if (force_path == 1) {
    VAQ_CHECK_ARG(size_m <= dec_max, "w4a16_gemm: decode path forced with size_m = %lld > %lld", (long long)size_m,
                  (long long)dec_max);
    decode = true;
  } else if (force_path == 2) {
    decode = false;
  } else if (!decode && !two_blocks_only && size_m <= 256 && size_n < (1 << 24) && size_k < (1 << 24) &&
             w4a16_decode2_takes_rows((int)size_m, (int)size_n, (int)size_k, sub, wt, perm != nullptr)) {
    // more rows than one workgroup of the decode kernel takes, on a layer narrow enough that workgroups of 16 rows each
    // make one round: ahead of the tile kernel there (see row_split_config in w4a16_decode2.hip); needs no scratch
    decode = true;
  }
  if (decode && decode_impl_for(size_m, size_n, lda, sub, w8) == 0)
    return w4a16_decode2_launch(a, lda, b, scales, zeros, perm, bias, c, c_tmp, c_tmp_bytes, counters, counter_ints, (int)size_m,
                                (int)size_n, (int)size_k, sub, channelwise, wt, dtype, s);
  if (decode) {
    VAQ_CHECK_SUPPORTED(sub == 1 && !w8, "w4a16_gemm: group_size = %d / 8-bit weights with an A of 2 GiB or more are not built",
                        group_size);
    return w4a16_decode_launch(a, lda, b, scales, zeros, perm, bias, c, c_tmp, c_tmp_bytes, counters, counter_ints, (int)size_m,
                               (int)size_n, (int)size_k, channelwise, dtype, s);
  }

  const void* a_eff = a;
  int64_t lda_eff = lda;
  if (perm) {
    VAQ_CHECK_ARG(a_tmp != nullptr, "w4a16_gemm: act_order on the prefill path needs a_tmp [size_m, size_k]");
    VAQ_CHECK_ARG(((uintptr_t)a_tmp % 16) == 0, "w4a16_gemm: a_tmp must be 16-byte aligned");
    rc = vaq_permute_cols(a, lda, perm, a_tmp, size_m, size_k, stream);
    if (rc != VAQ_OK) return rc;
    a_eff = a_tmp;
    lda_eff = size_k;
  }
  return w4a16_prefill_launch(a_eff, lda_eff, b, scales, zeros, bias, c, c_tmp, c_tmp_bytes, counters, counter_ints, (int)size_m,
                              (int)size_n, (int)size_k, sub, channelwise, wt, dtype, s);
}

// ----------------------------------------------------------------------------- the GEMM on library-owned scratch
namespace vaq {

// Scratch of vaq_w4a16_gemm_static: arrival counters (zero when the module is loaded, left zero by every kernel), then
// the split-K partial tiles, then the permuted activations.  One copy per GPU, held from the first use of the library
// on that GPU until the process ends.
constexpr size_t STATIC_COUNTER_INTS = VAQ_STATIC_SCRATCH_COUNTER_INTS;
constexpr size_t STATIC_DATA_BYTES = VAQ_STATIC_SCRATCH_DATA_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_COUNTER_INTS * 4 + STATIC_DATA_BYTES];

// `scratch` above is the host-side handle of the array, not an address a kernel can use: the device address is looked up
// once per device, with that device current, and kept here.
static unsigned char* g_scratch_ptr[VAQ_MAX_DEVICES];
static hipError_t g_scratch_err[VAQ_MAX_DEVICES];
static std::once_flag g_scratch_once[VAQ_MAX_DEVICES];

static int static_scratch_of_current_device(unsigned char** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= VAQ_MAX_DEVICES) {
    (void)hipGetLastError();
    set_error("w4a16_gemm_static: cannot identify the current device");
    return VAQ_ERR_LAUNCH;
  }
  std::call_once(g_scratch_once[dev], [dev] {
    void* p = nullptr;
    g_scratch_err[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    g_scratch_ptr[dev] = g_scratch_err[dev] == hipSuccess ? static_cast<unsigned char*>(p) : nullptr;
    if (g_scratch_err[dev] != hipSuccess) (void)hipGetLastError();
  });
  if (g_scratch_ptr[dev] == nullptr) {
    set_error("w4a16_gemm_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(g_scratch_err[dev]));
    return VAQ_ERR_LAUNCH;
  }
  *out = g_scratch_ptr[dev];
  return VAQ_OK;
}

}  // namespace vaq

extern "C" int vaq_w4a16_gemm_static(const void* a, int64_t lda, const int32_t* b, const void* scales,
                                     const int32_t* zeros, const int32_t* perm, const void* bias, void* c, int64_t size_m,
                                     int64_t size_n, int64_t size_k, int group_size, int dtype, int wtype, void* stream) {
  using namespace vaq;
  size_t c_tmp_bytes = 0, a_tmp_bytes = 0, counter_ints = 0;
  // The tile kernel's option of splitting the tiles of a half-empty last round over K is left out here: it is worth
  // tens of MB of partial tiles at thousands of rows, and whole tiles give the same result.
  VaqTuning whole_tiles = {};
  whole_tiles.exp[10] = 1;
  int rc = vaq_w4a16_gemm_workspace_tuned(size_m, size_n, size_k, perm != nullptr, 0, &c_tmp_bytes, &a_tmp_bytes, &counter_ints,
                                          &whole_tiles);
  if (rc != VAQ_OK) return rc;
  const size_t c_tmp_span = (c_tmp_bytes + 255) & ~(size_t)255;
  VAQ_CHECK_ARG(counter_ints <= STATIC_COUNTER_INTS && c_tmp_span + a_tmp_bytes <= STATIC_DATA_BYTES,
                "w4a16_gemm_static: M=%lld N=%lld K=%lld needs %zu counters and %zu + %zu bytes of scratch, the "
                "library-owned scratch holds %zu counters and %zu bytes; use vaq_w4a16_gemm with caller scratch",
                (long long)size_m, (long long)size_n, (long long)size_k, counter_ints, c_tmp_bytes, a_tmp_bytes,
                STATIC_COUNTER_INTS, STATIC_DATA_BYTES);
  unsigned char* base = nullptr;
  if (size_m > 0) {
    rc = static_scratch_of_current_device(&base);
    if (rc != VAQ_OK) return rc;
  }
  int32_t* counters = reinterpret_cast<int32_t*>(base);
  unsigned char* data = base ? base + STATIC_COUNTER_INTS * 4 : nullptr;
  return vaq_w4a16_gemm_tuned(a, lda, b, scales, zeros, perm, bias, c, c_tmp_bytes ? reinterpret_cast<float*>(data) : nullptr,
                              (int64_t)c_tmp_bytes, a_tmp_bytes ? data + c_tmp_span : nullptr, counters,
                              (int64_t)STATIC_COUNTER_INTS, size_m, size_n, size_k, group_size, dtype, wtype, 0, stream,
                              &whole_tiles);
}
