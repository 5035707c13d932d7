// Instances of the LDS-staged decode kernel for quantisation groups of 32 rows (4 groups per 128-row tile).
#include "w4a16_decode2_sub.h"

namespace vaq {

int decode2_launch_sub4(const Decode2Params& p, int gs, int MB, int mr, bool bf16, bool zp, hipStream_t s) {
  return sub_dispatch_rows<4>(p, gs, MB, mr, bf16, zp, s);
}

}  // namespace vaq
