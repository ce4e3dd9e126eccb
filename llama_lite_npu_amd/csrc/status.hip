// Thread-local error string and launch-status helper of liblitekv.
#include <stdarg.h>
#include <string.h>

#include "common.h"

namespace litekv {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_last_error[0] = '\0'; }

int check_launch(const char *what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    return fail(LITEKV_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(err));
  }
  clear_error();
  return LITEKV_OK;
}

}  // namespace litekv

extern "C" int litekv_abi_version(void) { return LITEKV_ABI_VERSION; }

extern "C" const char *litekv_last_error(void) { return litekv::g_last_error; }
