// Instances of the LDS-staged decode kernel for quantisation groups of 64 and 32 rows (2 / 4 groups per 128-row tile).
#include "w4a16_decode2_kernel.h"

namespace vaq {

template <bool BF16, int MB, bool HAS_ZP, int SUBG>
static int sub_dispatch_gs(const Decode2Params& p, int gs, hipStream_t s) {
  switch (gs) {
    case 1: return launch_decode2<BF16, 1, MB, HAS_ZP, 16, SUBG>(p, s);
    case 2: return launch_decode2<BF16, 2, MB, HAS_ZP, 16, SUBG>(p, s);
    case 4: return launch_decode2<BF16, 4, MB, HAS_ZP, 16, SUBG>(p, s);
    case 8: return launch_decode2<BF16, 8, MB, HAS_ZP, 16, SUBG>(p, s);
    case 16: return launch_decode2<BF16, 16, MB, HAS_ZP, 16, SUBG>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(decode): unsupported groups per wavefront %d", gs);
  return VAQ_ERR_UNSUPPORTED;
}

template <int MB, int SUBG>
static int sub_dispatch_types(const Decode2Params& p, int gs, bool bf16, bool zp, hipStream_t s) {
  if (bf16) return zp ? sub_dispatch_gs<true, MB, true, SUBG>(p, gs, s) : sub_dispatch_gs<true, MB, false, SUBG>(p, gs, s);
  return zp ? sub_dispatch_gs<false, MB, true, SUBG>(p, gs, s) : sub_dispatch_gs<false, MB, false, SUBG>(p, gs, s);
}

int decode2_launch_sub(const Decode2Params& p, int sub, int gs, int MB, bool bf16, bool zp, hipStream_t s) {
  if (sub == 2) return MB == 1 ? sub_dispatch_types<1, 2>(p, gs, bf16, zp, s) : sub_dispatch_types<2, 2>(p, gs, bf16, zp, s);
  if (sub == 4) return MB == 1 ? sub_dispatch_types<1, 4>(p, gs, bf16, zp, s) : sub_dispatch_types<2, 4>(p, gs, bf16, zp, s);
  set_error("w4a16_gemm(decode): %d quantisation groups per 128 rows", sub);
  return VAQ_ERR_UNSUPPORTED;
}

}  // namespace vaq
