// Error reporting shared by every entry point of the C-ABI.
#include "common.h"

namespace pt {

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
    return PT_ERR_LAUNCH;
  }
  return PT_OK;
}

}  // namespace pt

extern "C" const char* pt_last_error(void) { return pt::g_err; }
extern "C" int pt_abi_version(void) { return 1; }
