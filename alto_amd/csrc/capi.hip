// Error reporting and version query of the C ABI.
#include "common.h"

namespace alto {
namespace {
thread_local char g_err[512] = "";
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return ALTO_MXFP4_ELAUNCH;
  }
  return ALTO_MXFP4_OK;
}
}  // namespace alto

extern "C" int alto_mxfp4_version(void) { return 1; }
extern "C" const char* alto_mxfp4_last_error(void) { return alto::g_err; }
