// Instances of the direct-to-LDS prefill kernel for 8-bit codes (uint8b128: two 4-bit planes per tile), quantisation
// groups of 128 rows / channelwise (SUBG = 1) and of 64 / 32 rows (SUBG = 2 / 4).
#include "w4a16_prefill_kernel.h"

namespace vaq {

template <bool BF16, int SUBG>
static int w8_dispatch_tile(const PrefillParams& p, int tile, hipStream_t s) {
  switch (tile) {
    case 10: return launch_prefill2<BF16, 256, 256, 2, 4, false, SUBG, true>(p, s);
    case 12: return launch_prefill2<BF16, 128, 128, 2, 2, false, SUBG, true>(p, s);
    case 14: return launch_prefill2<BF16, 64, 128, 2, 2, false, SUBG, true>(p, s);
    case 15: return launch_prefill2<BF16, 128, 64, 2, 2, false, SUBG, true>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(prefill): tile id %d is not built for 8-bit weights", tile);
  return VAQ_ERR_UNSUPPORTED;
}

int prefill_launch_w8(const PrefillParams& p, int sub, int tile, bool bf16, hipStream_t s) {
  switch (sub) {
    case 1: return bf16 ? w8_dispatch_tile<true, 1>(p, tile, s) : w8_dispatch_tile<false, 1>(p, tile, s);
    case 2: return bf16 ? w8_dispatch_tile<true, 2>(p, tile, s) : w8_dispatch_tile<false, 2>(p, tile, s);
    case 4: return bf16 ? w8_dispatch_tile<true, 4>(p, tile, s) : w8_dispatch_tile<false, 4>(p, tile, s);
    default: break;
  }
  set_error("w4a16_gemm(prefill, 8-bit): %d groups per 128 rows are not built", sub);
  return VAQ_ERR_UNSUPPORTED;
}

}  // namespace vaq
