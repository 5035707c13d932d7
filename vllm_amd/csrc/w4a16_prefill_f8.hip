// Instances of the direct-to-LDS prefill kernel for FP8 e4m3 weights with 16-bit activations (whole bytes, two 1 KiB
// blocks per tile), channelwise scales or quantisation groups of 128 rows.
#include "w4a16_prefill_kernel.h"

namespace vaq {

template <bool BF16>
static int f8_dispatch_tile(const PrefillParams& p, int tile, hipStream_t s) {
  switch (tile) {
    case 10: return launch_prefill2<BF16, 256, 256, 2, 4, false, 1, 2>(p, s);
    case 12: return launch_prefill2<BF16, 128, 128, 2, 2, false, 1, 2>(p, s);
    case 14: return launch_prefill2<BF16, 64, 128, 2, 2, false, 1, 2>(p, s);
    case 15: return launch_prefill2<BF16, 128, 64, 2, 2, false, 1, 2>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(prefill): tile id %d is not built for FP8 weights", tile);
  return VAQ_ERR_UNSUPPORTED;
}

int prefill_launch_f8(const PrefillParams& p, int tile, bool bf16, hipStream_t s) {
  return bf16 ? f8_dispatch_tile<true>(p, tile, s) : f8_dispatch_tile<false>(p, tile, s);
}

}  // namespace vaq
