// Instances of the prefill kernels for quantisation groups of 64 and 32 rows (2 / 4 groups per 128-row tile).
#include "w4a16_prefill_kernel.h"

namespace vaq {

template <bool BF16, bool HAS_ZP, int SUBG>
static int sub_dispatch_tile(const PrefillParams& p, int tile, hipStream_t s) {
  switch (tile) {
    case 10: return launch_prefill2<BF16, 256, 256, 2, 4, HAS_ZP, SUBG>(p, s);
    case 12: return launch_prefill2<BF16, 128, 128, 2, 2, HAS_ZP, SUBG>(p, s);
    case 14: return launch_prefill2<BF16, 64, 128, 2, 2, HAS_ZP, SUBG>(p, s);
    case 15: return launch_prefill2<BF16, 128, 64, 2, 2, HAS_ZP, SUBG>(p, s);
    case 0: return launch_prefill<BF16, 4, 4, HAS_ZP, SUBG>(p, s);
    case 1: return launch_prefill<BF16, 2, 2, HAS_ZP, SUBG>(p, s);
    case 2: return launch_prefill<BF16, 1, 2, HAS_ZP, SUBG>(p, s);
    default: break;
  }
  set_error("w4a16_gemm(prefill): tile id %d is not built for group sizes below 128", tile);
  return VAQ_ERR_UNSUPPORTED;
}

template <int SUBG>
static int sub_dispatch_types(const PrefillParams& p, int tile, bool bf16, bool zp, hipStream_t s) {
  if (bf16) return zp ? sub_dispatch_tile<true, true, SUBG>(p, tile, s) : sub_dispatch_tile<true, false, SUBG>(p, tile, s);
  return zp ? sub_dispatch_tile<false, true, SUBG>(p, tile, s) : sub_dispatch_tile<false, false, SUBG>(p, tile, s);
}

int prefill_launch_sub(const PrefillParams& p, int sub, int tile, bool bf16, bool zp, hipStream_t s) {
  if (sub == 2) return sub_dispatch_types<2>(p, tile, bf16, zp, s);
  if (sub == 4) return sub_dispatch_types<4>(p, tile, bf16, zp, s);
  set_error("w4a16_gemm(prefill): %d quantisation groups per 128 rows", sub);
  return VAQ_ERR_UNSUPPORTED;
}

}  // namespace vaq
