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

}  // namespace pbg

extern "C" int pbg_version(void) { return 1; }
extern "C" const char* pbg_last_error(void) { return pbg::g_error; }
