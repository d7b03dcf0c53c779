// Error reporting shared by every entry point of libsga_hip.so.
#include <stdarg.h>
#include <stdio.h>

#include "common.hpp"

namespace sga {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return SGA_ERR_LAUNCH;
  }
  return SGA_OK;
}

}  // namespace sga

extern "C" int sga_version(void) { return 1; }
extern "C" const char* sga_last_error(void) { return sga::g_err; }
