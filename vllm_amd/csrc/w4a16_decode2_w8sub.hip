// Instances of the LDS-staged decode kernel for 8-bit codes with quantisation groups of 64 or 32 rows (two 4-bit planes
// per 128 rows, SUBG = 2 / 4 groups per plane tile).
#include "w4a16_decode2_kernel.h"

namespace vaq {

template <bool BF16, int MB, int MR, int SUBG>
static int w8sub_dispatch_gs(const Decode2Params& p, int gs, hipStream_t s) {
  switch (gs) {
    case 2: return launch_decode2<BF16, 2, MB, false, MR, SUBG, true>(p, s);
    case 4: return launch_decode2<BF16, 4, MB, false, MR, SUBG, true>(p, s);
    case 8: return launch_decode2<BF16, 8, MB, false, MR, SUBG, true>(p, s);
    case 16: return launch_decode2<BF16, 16, MB, false, MR, SUBG, true>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(decode, 8-bit): unsupported tiles per wavefront %d", gs);
  return VAQ_ERR_UNSUPPORTED;
}

template <bool BF16, int SUBG>
static int w8sub_dispatch_rows(const Decode2Params& p, int gs, int MB, int mr, hipStream_t s) {
  if (MB == 2) return w8sub_dispatch_gs<BF16, 2, 16, SUBG>(p, gs, s);
  switch (mr) {
    case 1: return w8sub_dispatch_gs<BF16, 1, 1, SUBG>(p, gs, s);
    case 4: return w8sub_dispatch_gs<BF16, 1, 4, SUBG>(p, gs, s);
    default: return w8sub_dispatch_gs<BF16, 1, 16, SUBG>(p, gs, s);
  }
}

int decode2_launch_w8sub(const Decode2Params& p, int sub, int gs, int MB, int mr, bool bf16, hipStream_t s) {
  if (sub == 2) return bf16 ? w8sub_dispatch_rows<true, 2>(p, gs, MB, mr, s) : w8sub_dispatch_rows<false, 2>(p, gs, MB, mr, s);
  if (sub == 4) return bf16 ? w8sub_dispatch_rows<true, 4>(p, gs, MB, mr, s) : w8sub_dispatch_rows<false, 4>(p, gs, MB, mr, s);
  set_error("w4a16_gemm(decode, 8-bit): %d groups per 128 rows are not built", sub);
  return VAQ_ERR_UNSUPPORTED;
}

}  // namespace vaq
