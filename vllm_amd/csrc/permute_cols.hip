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

// Rows staged in LDS: a workgroup copies PC_ROWS rows (as many as fit 32 KiB, so that several workgroups share a compute
// unit and one's loads overlap another's gathers) with coalesced 16-byte loads, then every thread gathers 8 columns
// per row from LDS (the permutation entries are read once and reused for all the rows) and writes 16-byte stores.
// The scattered 2-byte reads thus hit LDS instead of going out as 64 separate addresses per global load instruction.
template <int PC_ROWS>
__global__ __launch_bounds__(256) void permute_cols_lds_kernel(const uint16_t* __restrict__ a, int64_t lda,
                                                                const int32_t* __restrict__ perm,
                                                                uint16_t* __restrict__ out, int64_t size_m, int size_k) {
  extern __shared__ __attribute__((aligned(16))) uint16_t rows[];      // [PC_ROWS][size_k]
  const int64_t m0 = (int64_t)blockIdx.x * PC_ROWS;
  const int chunks = size_k / 8;
  const bool aligned = (lda % 8 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0);
#pragma unroll
  for (int r = 0; r < PC_ROWS; ++r) {
    const int64_t m = m0 + r < size_m ? m0 + r : size_m - 1;
    const uint16_t* row = a + m * lda;
    if (aligned) {
      for (int c = threadIdx.x; c < chunks; c += 256)
        *reinterpret_cast<v4u*>(rows + (size_t)r * size_k + c * 8) = *reinterpret_cast<const v4u*>(row + c * 8);
    } else {
      for (int k = threadIdx.x; k < size_k; k += 256) rows[(size_t)r * size_k + k] = row[k];
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < chunks; c += 256) {
    const v4i p0 = *reinterpret_cast<const v4i*>(perm + c * 8);
    const v4i p1 = *reinterpret_cast<const v4i*>(perm + c * 8 + 4);
#pragma unroll
    for (int r = 0; r < PC_ROWS; ++r) {
      if (m0 + r >= size_m) break;
      const uint16_t* row = rows + (size_t)r * size_k;
      v4u v;
      v.x = (uint32_t)row[p0.x] | ((uint32_t)row[p0.y] << 16);
      v.y = (uint32_t)row[p0.z] | ((uint32_t)row[p0.w] << 16);
      v.z = (uint32_t)row[p1.x] | ((uint32_t)row[p1.y] << 16);
      v.w = (uint32_t)row[p1.z] | ((uint32_t)row[p1.w] << 16);
      *reinterpret_cast<v4u*>(out + (m0 + r) * (int64_t)size_k + c * 8) = v;
    }
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
  const size_t row_bytes = (size_t)size_k * 2;
  if (row_bytes <= 128 * 1024) {
    const int rows = row_bytes * 4 <= 32 * 1024 ? 4 : (row_bytes * 2 <= 32 * 1024 ? 2 : 1);
    const size_t lds = rows * row_bytes;
    const void* kern = rows == 4 ? reinterpret_cast<const void*>(permute_cols_lds_kernel<4>)
                                 : (rows == 2 ? reinterpret_cast<const void*>(permute_cols_lds_kernel<2>)
                                              : reinterpret_cast<const void*>(permute_cols_lds_kernel<1>));
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      set_error("permute_cols: cannot reserve %zu bytes of LDS", lds);
      (void)hipGetLastError();
      return VAQ_ERR_LAUNCH;
    }
    const dim3 grid((unsigned)((size_m + rows - 1) / rows));
    if (rows == 4)
      hipLaunchKernelGGL(permute_cols_lds_kernel<4>, grid, dim3(256), lds, (hipStream_t)stream, (const uint16_t*)a, lda, perm,
                         (uint16_t*)out, size_m, (int)size_k);
    else if (rows == 2)
      hipLaunchKernelGGL(permute_cols_lds_kernel<2>, grid, dim3(256), lds, (hipStream_t)stream, (const uint16_t*)a, lda, perm,
                         (uint16_t*)out, size_m, (int)size_k);
    else
      hipLaunchKernelGGL(permute_cols_lds_kernel<1>, grid, dim3(256), lds, (hipStream_t)stream, (const uint16_t*)a, lda, perm,
                         (uint16_t*)out, size_m, (int)size_k);
  } else {
    hipLaunchKernelGGL(permute_cols_kernel, dim3((unsigned)size_m), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t*)a, lda, perm, (uint16_t*)out, size_k);
  }
  VAQ_CHECK_LAUNCH("permute_cols");
  return VAQ_OK;
}
