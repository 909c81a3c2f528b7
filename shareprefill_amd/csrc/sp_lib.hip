// Library identity and the per-thread error string of libshareprefill_hip.
#include <stdarg.h>

#include "sp_common.h"

static thread_local char g_sp_error[512] = "";

void sp_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_sp_error, sizeof(g_sp_error), fmt, ap);
  va_end(ap);
}

extern "C" int sp_version(void) { return 1; }
extern "C" const char* sp_arch(void) { return "gfx950"; }
extern "C" const char* sp_last_error(void) { return g_sp_error; }

