// Error text of the last refused call, and a version probe for the loader.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_last_error[512] = "";

void mi_set_error(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, args);
  va_end(args);
}

extern "C" const char* mi_last_error() { return g_last_error; }

// Bumped whenever an entry point's arguments change, so a stale library is refused.
extern "C" int mi_abi_version() { return 18; }
