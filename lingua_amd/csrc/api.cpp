// Host-side plumbing shared by the entry points: thread-local error text,
// device identification, cached device properties.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>

#include "l8_common.h"

namespace l8 {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static std::atomic<int> g_scale_rule{L8_SCALE_RULE_DIVIDE};
int scale_rule() { return g_scale_rule.load(std::memory_order_relaxed); }

static int g_cus[kMaxDev];  // 0 = not queried yet; benign race: every thread writes the same value

int device_slot() {
  int dev = 0;
  return (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDev) ? dev : -1;
}

int num_cus() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
  int c = g_cus[dev];
  if (c == 0) {
    if (hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || c <= 0) c = 256;
    g_cus[dev] = c;
  }
  return c;
}

}  // namespace l8

extern "C" int l8_version(void) { return 1; }

extern "C" const char *l8_last_error(void) { return l8::g_err; }

extern "C" int l8_set_scale_rule(int rule) {
  if (rule != L8_SCALE_RULE_DIVIDE && rule != L8_SCALE_RULE_TIMES_INVERSE)
    return l8::fail(L8_EINVAL, "l8_set_scale_rule: unknown rule %d", rule);
  l8::g_scale_rule.store(rule, std::memory_order_relaxed);
  return L8_OK;
}

extern "C" int l8_get_scale_rule(void) { return l8::scale_rule(); }

extern "C" int l8_device_check(int device) {
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return l8::fail(L8_EHIP, "hipGetDeviceProperties(%d): %s", device, hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return l8::fail(L8_EARCH, "device %d is %s; this library contains gfx950 code only", device, prop.gcnArchName);
  // per-device set-up, with that device current for its duration
  int prev = -1;
  if (hipGetDevice(&prev) != hipSuccess) prev = -1;
  if (prev != device) {
    e = hipSetDevice(device);
    if (e != hipSuccess) return l8::fail(L8_EHIP, "hipSetDevice(%d): %s", device, hipGetErrorString(e));
  }
  const int rc = l8::noalloc_setup_current_device();
  if (prev != device && prev >= 0) (void)hipSetDevice(prev);
  return rc;
}
