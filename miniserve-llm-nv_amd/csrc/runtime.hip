// Error reporting shared by every entry point of the library.
#include "common.hpp"

#include <stdarg.h>
#include <stdio.h>

namespace {
thread_local char g_last_error[512] = "";
}

int ms_fail(const char* format, ...) {
  va_list args;
  va_start(args, format);
  vsnprintf(g_last_error, sizeof(g_last_error), format, args);
  va_end(args);
  return 1;
}

extern "C" const char* ms_last_error() { return g_last_error; }

// Build probe: the architecture this library was compiled for.
extern "C" const char* ms_target_arch() { return "gfx950"; }
