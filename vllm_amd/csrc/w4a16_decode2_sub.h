// Dispatch of the LDS-staged decode kernel's instances for quantisation groups of 64 or 32 rows (SUBG = 2 / 4 groups
// per 128-row tile); one translation unit per SUBG instantiates it (w4a16_decode2_sub2.hip, w4a16_decode2_sub4.hip).
#pragma once
#include "w4a16_decode2_kernel.h"

namespace vaq {

template <bool BF16, int MB, bool HAS_ZP, int MR, int SUBG>
static int sub_dispatch_gs(const Decode2Params& p, int gs, hipStream_t s) {
  switch (gs) {
    case 1: return launch_decode2<BF16, 1, MB, HAS_ZP, MR, SUBG>(p, s);
    case 2: return launch_decode2<BF16, 2, MB, HAS_ZP, MR, SUBG>(p, s);
    case 4: return launch_decode2<BF16, 4, MB, HAS_ZP, MR, SUBG>(p, s);
    case 8: return launch_decode2<BF16, 8, MB, HAS_ZP, MR, SUBG>(p, s);
    case 16: return launch_decode2<BF16, 16, MB, HAS_ZP, MR, SUBG>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(decode): unsupported groups per wavefront %d", gs);
  return VAQ_ERR_UNSUPPORTED;
}

template <int MB, int MR, int SUBG>
static int sub_dispatch_types(const Decode2Params& p, int gs, bool bf16, bool zp, hipStream_t s) {
  if (bf16) return zp ? sub_dispatch_gs<true, MB, true, MR, SUBG>(p, gs, s) : sub_dispatch_gs<true, MB, false, MR, SUBG>(p, gs, s);
  return zp ? sub_dispatch_gs<false, MB, true, MR, SUBG>(p, gs, s) : sub_dispatch_gs<false, MB, false, MR, SUBG>(p, gs, s);
}

template <int SUBG>
static int sub_dispatch_rows(const Decode2Params& p, int gs, int MB, int mr, bool bf16, bool zp, hipStream_t s) {
  if (MB == 2) return sub_dispatch_types<2, 16, SUBG>(p, gs, bf16, zp, s);
  switch (mr) {
    case 1: return sub_dispatch_types<1, 1, SUBG>(p, gs, bf16, zp, s);
    case 4: return sub_dispatch_types<1, 4, SUBG>(p, gs, bf16, zp, s);
    default: return sub_dispatch_types<1, 16, SUBG>(p, gs, bf16, zp, s);
  }
}

}  // namespace vaq
