// Error reporting shared by every entry point of libhils_amd.so.
#include <stdarg.h>
#include <stdio.h>
#include <atomic>
#include <hip/hip_runtime.h>
#include "../../include/hils_amd.h"
#include "common.h"

static thread_local char g_err[512] = "";

void hils_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* hils_last_error(void) { return g_err; }
extern "C" int hils_version(void) { return 1; }

// ---- per-device launch state shared by the launchers ------------------------------------------
// Both are keyed by the current device and held in atomics: entry points may be called from
// several host threads and on several devices of one process.
#define HILS_MAX_DEVICES 64

int hils_device_cus() {
  static std::atomic<int> cus[HILS_MAX_DEVICES];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= HILS_MAX_DEVICES) dev = 0;
  int v = cus[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    v = 256;
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) v = n;
    cus[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

int hils_reserve_lds(HilsLdsReserve* state, const void* kernel, size_t bytes, const char* who) {
  int dev = 0;
  const bool known = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < HILS_LDS_RESERVE_DEVICES;
  if (bytes <= 48 * 1024) return HILS_OK;  // within the limit every kernel has without asking
  if (known && state->bytes[dev].load(std::memory_order_acquire) >= bytes) return HILS_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
    (void)hipGetLastError();
    hils_set_error("%s: cannot reserve %zu bytes of LDS", who, bytes);
    return HILS_ERR_LAUNCH;
  }
  if (known) {  // keep the maximum: a racing thread that reserved more must not be undone
    size_t cur = state->bytes[dev].load(std::memory_order_relaxed);
    while (cur < bytes && !state->bytes[dev].compare_exchange_weak(cur, bytes, std::memory_order_release)) {}
  }
  return HILS_OK;
}
