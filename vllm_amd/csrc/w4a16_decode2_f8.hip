// Instances of the LDS-staged decode kernel for FP8 e4m3 weights with 16-bit activations (whole bytes, two 1 KiB blocks
// per tile), channelwise scales or quantisation groups of 128 rows.
#include "w4a16_decode2_kernel.h"

namespace vaq {

template <bool BF16, int MB, int MR>
static int f8_dispatch_gs(const Decode2Params& p, int gs, hipStream_t s) {
  switch (gs) {
    case 2: return launch_decode2<BF16, 2, MB, false, MR, 1, 2>(p, s);
    case 4: return launch_decode2<BF16, 4, MB, false, MR, 1, 2>(p, s);
    case 8: return launch_decode2<BF16, 8, MB, false, MR, 1, 2>(p, s);
    case 14: return launch_decode2<BF16, 14, MB, false, MR, 1, 2>(p, s);
    case 16: return launch_decode2<BF16, 16, MB, false, MR, 1, 2>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(decode, FP8 weights): unsupported blocks per wavefront %d", gs);
  return VAQ_ERR_UNSUPPORTED;
}

template <bool BF16>
static int f8_dispatch_rows(const Decode2Params& p, int gs, int MB, int mr, hipStream_t s) {
  if (MB == 2) return f8_dispatch_gs<BF16, 2, 16>(p, gs, s);
  switch (mr) {
    case 1: return f8_dispatch_gs<BF16, 1, 1>(p, gs, s);
    case 4: return f8_dispatch_gs<BF16, 1, 4>(p, gs, s);
    default: return f8_dispatch_gs<BF16, 1, 16>(p, gs, s);
  }
}

int decode2_launch_f8(const Decode2Params& p, int gs, int MB, int mr, bool bf16, hipStream_t s) {
  return bf16 ? f8_dispatch_rows<true>(p, gs, MB, mr, s) : f8_dispatch_rows<false>(p, gs, MB, mr, s);
}

}  // namespace vaq
