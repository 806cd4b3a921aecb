// Error plumbing and version query shared by every entry point of libtprime_hip.so.
#include "common.hpp"

namespace tp {

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
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return TP_ERR_LAUNCH;
  }
  return TP_OK;
}

}  // namespace tp

extern "C" int tp_version(void) { return 100; }
extern "C" const char* tp_last_error(void) { return tp::g_err; }
