// Instances of the LDS-staged decode kernel with the rows split over workgroups (16 < M <= 64 as independent m-blocks,
// one per blockIdx.z; see the kernel): 4-bit codes, groups of 128 rows or channelwise scales.
#include "w4a16_decode2_kernel.h"

namespace vaq {

template <bool BF16, bool HAS_ZP, int GS>
static int msp_dispatch_rc(const Decode2Params& p, int rc, hipStream_t s) {
  if (rc == 1) return launch_decode2<BF16, GS, 1, HAS_ZP, 16, 1, 0, 1, true>(p, s);
  if (rc == 2) return launch_decode2<BF16, GS, 1, HAS_ZP, 16, 1, 0, 2, true>(p, s);
  return launch_decode2<BF16, GS, 1, HAS_ZP, 16, 1, 0, 0, true>(p, s);
}

template <bool BF16, bool HAS_ZP>
static int msp_dispatch_gs(const Decode2Params& p, int gs, int rc, hipStream_t s) {
  switch (gs) {
    case 1: return launch_decode2<BF16, 1, 1, HAS_ZP, 16, 1, 0, 0, true>(p, s);
    case 2: return launch_decode2<BF16, 2, 1, HAS_ZP, 16, 1, 0, 0, true>(p, s);
    case 4: return launch_decode2<BF16, 4, 1, HAS_ZP, 16, 1, 0, 0, true>(p, s);
    case 7: return msp_dispatch_rc<BF16, HAS_ZP, 7>(p, rc, s);
    case 8: return msp_dispatch_rc<BF16, HAS_ZP, 8>(p, rc, s);
    case 14: return msp_dispatch_rc<BF16, HAS_ZP, 14>(p, rc, s);
    case 16: return msp_dispatch_rc<BF16, HAS_ZP, 16>(p, rc, s);
    default: break;
  }
  set_error("w4a16_gemm(decode): unsupported groups per wavefront %d", gs);
  return VAQ_ERR_UNSUPPORTED;
}

int decode2_launch_msp(const Decode2Params& p, int gs, int rc, bool bf16, bool zp, hipStream_t s) {
  if (p.SK != 1 || p.perm != nullptr) {
    set_error("w4a16_gemm(decode): rows split over workgroups need an unsplit K and no act_order");
    return VAQ_ERR_UNSUPPORTED;
  }
  if (bf16) return zp ? msp_dispatch_gs<true, true>(p, gs, rc, s) : msp_dispatch_gs<true, false>(p, gs, rc, s);
  return zp ? msp_dispatch_gs<false, true>(p, gs, rc, s) : msp_dispatch_gs<false, false>(p, gs, rc, s);
}

}  // namespace vaq
