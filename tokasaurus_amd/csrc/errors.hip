// Error reporting of a kernel library: every entry point returns 0 or a negative
// code and leaves a message that the Python side reads with tk_last_error().
// This file is part of each library, so each keeps its own message.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512];

void tk_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

TK_API const char* tk_last_error() { return g_error; }
