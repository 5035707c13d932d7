// Library-wide pieces of the C ABI: error text, ABI version, cached device facts.
#include "vaq_common.h"

#include <mutex>

namespace vaq {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

static thread_local const VaqTuning* g_tuning = nullptr;
static const VaqTuning g_no_tuning = {};

const VaqTuning& tuning() { return g_tuning ? *g_tuning : g_no_tuning; }
TuningScope::TuningScope(const VaqTuning* t) : prev_(g_tuning) { g_tuning = t; }
TuningScope::~TuningScope() { g_tuning = prev_; }

// Immutable per-device cache (the only host-visible state of the library).
static int g_cus[64];
static std::once_flag g_cus_once[64];

static int cus_of(int dev) {
  if (dev < 0 || dev >= 64) return -1;
  std::call_once(g_cus_once[dev], [dev] {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) v = -1;
    g_cus[dev] = v;
  });
  return g_cus[dev];
}

int num_cus_current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  int c = cus_of(dev);
  return c > 0 ? c : 256;
}

}  // namespace vaq

extern "C" const char* vaq_last_error(void) { return vaq::g_err; }

extern "C" int vaq_abi_version(void) { return 1; }

extern "C" int vaq_num_cus(int device) {
  int c = vaq::cus_of(device);
  if (c <= 0) {
    vaq::set_error("vaq_num_cus: cannot query device %d", device);
    return VAQ_ERR_INVALID_ARG;
  }
  return c;
}
