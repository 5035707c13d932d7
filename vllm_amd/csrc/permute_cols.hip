// out[m, k] = a[m, perm[k]] for 16-bit elements (activation reorder for act_order weights).
#include "vaq_common.h"

namespace vaq {

// One workgroup per row; each thread gathers 8 columns and writes them as one 16-byte store.
__global__ __launch_bounds__(256) void permute_cols_kernel(const uint16_t* __restrict__ a, int64_t lda,
                                                            const int32_t* __restrict__ perm,
                                                            uint16_t* __restrict__ out, int64_t size_k) {
  const int64_t m = blockIdx.x;
  const uint16_t* row = a + m * lda;
  uint16_t* orow = out + m * size_k;
  const int64_t chunks = size_k / 8;
  for (int64_t c = threadIdx.x; c < chunks; c += blockDim.x) {
    const v4i p0 = *reinterpret_cast<const v4i*>(perm + c * 8);
    const v4i p1 = *reinterpret_cast<const v4i*>(perm + c * 8 + 4);
    v4u r;
    r.x = (uint32_t)row[p0.x] | ((uint32_t)row[p0.y] << 16);
    r.y = (uint32_t)row[p0.z] | ((uint32_t)row[p0.w] << 16);
    r.z = (uint32_t)row[p1.x] | ((uint32_t)row[p1.y] << 16);
    r.w = (uint32_t)row[p1.z] | ((uint32_t)row[p1.w] << 16);
    *reinterpret_cast<v4u*>(orow + c * 8) = r;
  }
}

}  // namespace vaq

extern "C" int vaq_permute_cols(const void* a, int64_t lda, const int32_t* perm, void* out, int64_t size_m,
                                int64_t size_k, void* stream) {
  using namespace vaq;
  VAQ_CHECK_ARG(size_m >= 0 && size_k > 0, "permute_cols: bad shape [%lld, %lld]", (long long)size_m, (long long)size_k);
  VAQ_CHECK_ARG(size_k % 8 == 0, "permute_cols: size_k = %lld must be divisible by 8", (long long)size_k);
  VAQ_CHECK_ARG(lda >= size_k, "permute_cols: lda = %lld < size_k = %lld", (long long)lda, (long long)size_k);
  VAQ_CHECK_ARG(size_m < (1ll << 31), "permute_cols: size_m too large");
  if (size_m == 0) return VAQ_OK;
  VAQ_CHECK_ARG(a && perm && out, "permute_cols: null pointer");
  VAQ_CHECK_ARG(((uintptr_t)out % 16) == 0 && ((uintptr_t)perm % 16) == 0, "permute_cols: out/perm must be 16-byte aligned");
  hipLaunchKernelGGL(permute_cols_kernel, dim3((unsigned)size_m), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)a, lda, perm, (uint16_t*)out, size_k);
  VAQ_CHECK_LAUNCH("permute_cols");
  return VAQ_OK;
}
