// Version and error text of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/iron_hip.h"
#include "common.h"

namespace iron {
static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace iron

extern "C" int iron_version(void) { return 100; }
extern "C" const char* iron_last_error(void) { return iron::g_error; }
