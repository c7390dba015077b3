// Host-side plumbing of the C ABI: error reporting and device queries.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>

#include "kvq_internal.h"

namespace kvq {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return KVQ_OK;
  return fail(KVQ_EHIP, "%s: %s", what, hipGetErrorString(e));
}

int num_cus() {
  static thread_local int cached_dev = -1;
  static thread_local int cached_cus = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached_dev = dev;
    cached_cus = n;
  }
  return cached_cus;
}

static std::atomic<int> g_batch_invariant{0};
bool batch_invariant() { return g_batch_invariant.load(std::memory_order_relaxed) != 0; }

}  // namespace kvq

extern "C" {

int kvq_set_batch_invariant(int on) { return kvq::g_batch_invariant.exchange(on != 0 ? 1 : 0); }
int kvq_get_batch_invariant(void) { return kvq::batch_invariant() ? 1 : 0; }

int kvq_abi_version(void) { return KVQ_ABI_VERSION; }
const char* kvq_last_error(void) { return kvq::g_err; }
int kvq_device_num_cus(void) { return kvq::num_cus(); }

}  // extern "C"
