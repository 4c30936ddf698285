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

// Compute units of the current device, asked once per device (launch rules fill the chip
// by this number; it changes how work is cut, never a result's value beyond rounding).
int ms_compute_units() {
  static thread_local int cached_device = -1, cached_units = 0;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 256;
  if (device != cached_device) {
    int units = 0;
    if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0) units = 256;
    cached_device = device;
    cached_units = units;
  }
  return cached_units;
}

extern "C" int ms_device_compute_units() { return ms_compute_units(); }
