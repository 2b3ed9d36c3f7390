// Error reporting and version query of the C ABI.
#include "kitty_common.h"

namespace kitty {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

}  // namespace kitty

extern "C" int kitty_abi_version(void) { return KITTY_ABI_VERSION; }
extern "C" const char* kitty_last_error(void) { return kitty::g_err; }
