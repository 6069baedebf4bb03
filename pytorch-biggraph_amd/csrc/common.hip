// Error reporting and version of libpbg_hip.
#include <cstdarg>
#include <cstdio>

#include "pbg_internal.h"

namespace pbg {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    return fail(PBG_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
  }
  return PBG_OK;
}

int reserve_lds(const void* kernel, LdsLimit* limit, size_t bytes) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(PBG_ERR_UNSUPPORTED, "device %d: the library keeps state for devices 0 .. %d", dev, kMaxDevices - 1);
  if (bytes <= limit->allowed[dev].load(std::memory_order_acquire)) return PBG_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
    (void)hipGetLastError();
    return fail(PBG_ERR_LAUNCH, "cannot reserve %zu bytes of LDS", bytes);
  }
  // (two threads at once both set the attribute; the larger request is the one that must stay recorded)
  size_t seen = limit->allowed[dev].load(std::memory_order_relaxed);
  while (seen < bytes && !limit->allowed[dev].compare_exchange_weak(seen, bytes, std::memory_order_release)) {
  }
  return PBG_OK;
}

int compute_units() {
  static std::atomic<int> cached[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    cached[dev].store(cus, std::memory_order_relaxed);
  }
  return cus;
}

}  // namespace pbg

extern "C" int pbg_version(void) { return 1; }
extern "C" const char* pbg_last_error(void) { return pbg::g_error; }
