// Instances of the LDS-staged decode kernel for three and four m-blocks (32 < M <= 64).
#include "w4a16_decode2_kernel.h"

namespace vaq {

template <bool BF16, int MB, bool HAS_ZP>
static int mb34_dispatch_gs(const Decode2Params& p, int gs, hipStream_t s) {
  switch (gs) {
    case 1: return launch_decode2<BF16, 1, MB, HAS_ZP, 16, 1>(p, s);
    case 2: return launch_decode2<BF16, 2, MB, HAS_ZP, 16, 1>(p, s);
    case 4: return launch_decode2<BF16, 4, MB, HAS_ZP, 16, 1>(p, s);
    case 7: return launch_decode2<BF16, 7, MB, HAS_ZP, 16, 1>(p, s);
    case 8: return launch_decode2<BF16, 8, MB, HAS_ZP, 16, 1>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(decode): unsupported groups per wavefront %d for %d m-blocks", gs, MB);
  return VAQ_ERR_UNSUPPORTED;
}

template <int MB>
static int mb34_dispatch_types(const Decode2Params& p, int gs, bool bf16, bool zp, hipStream_t s) {
  if (bf16) return zp ? mb34_dispatch_gs<true, MB, true>(p, gs, s) : mb34_dispatch_gs<true, MB, false>(p, gs, s);
  return zp ? mb34_dispatch_gs<false, MB, true>(p, gs, s) : mb34_dispatch_gs<false, MB, false>(p, gs, s);
}

int decode2_launch_mb34(const Decode2Params& p, int gs, int MB, bool bf16, bool zp, hipStream_t s) {
  if (MB == 3) return mb34_dispatch_types<3>(p, gs, bf16, zp, s);
  if (MB == 4) return mb34_dispatch_types<4>(p, gs, bf16, zp, s);
  set_error("w4a16_gemm(decode): %d m-blocks", MB);
  return VAQ_ERR_UNSUPPORTED;
}

}  // namespace vaq
