// Error channel and identification of the kernel library.  Every entry point returns 0 on
// success; on failure it returns non-zero after storing a message that blm_last_error() gives back.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

static thread_local char g_error[512];

int blm_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

extern "C" const char* blm_last_error() { return g_error; }

// ABI version: bumped when an entry point's signature changes, checked by the Python loader.
extern "C" int blm_abi_version() { return 24; }
