// The error message of the last failed entry point of this library (per thread).
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";
extern "C" const char* pico_last_error() { return g_error; }
void pico_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
