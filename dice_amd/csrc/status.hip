// Error text and ABI version of the C boundary.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace dice {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace dice

extern "C" int dice_abi_version(void) { return DICE_MOE_ABI_VERSION; }

extern "C" const char *dice_last_error(void) { return dice::g_err; }
