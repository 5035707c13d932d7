// Instances of the register-dequantising tile kernel (w4a16_prefill3_kernel.h): 4-bit codes, groups of 128 rows or
// channelwise scales, bf16 / fp16, with and without zero points.
#include "w4a16_prefill3_kernel.h"

namespace vaq {

int prefill_launch_reg(const PrefillParams& p, bool bf16, bool zp, hipStream_t s) {
  if (bf16) return zp ? launch_prefill3<true, true>(p, s) : launch_prefill3<true, false>(p, s);
  return zp ? launch_prefill3<false, true>(p, s) : launch_prefill3<false, false>(p, s);
}

}  // namespace vaq
