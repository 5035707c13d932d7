// Instances of the LDS-staged decode kernel for quantisation groups of 64 rows (2 groups per 128-row tile).
#include "w4a16_decode2_sub.h"

namespace vaq {

int decode2_launch_sub2(const Decode2Params& p, int gs, int MB, int mr, bool bf16, bool zp, hipStream_t s) {
  return sub_dispatch_rows<2>(p, gs, MB, mr, bf16, zp, s);
}

}  // namespace vaq
