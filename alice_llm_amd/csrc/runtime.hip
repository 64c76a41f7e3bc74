// Host-side error channel and library identification.
#include "common.h"
#include "alice_hip.h"
#include <stdarg.h>
#include <string.h>

static thread_local char g_error[1024] = "";

void alice_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* alice_last_error() { return g_error; }

extern "C" int alice_abi_version() { return ALICE_ABI_VERSION; }

// The digest of the sources that this library was built from (given by the build script).
#ifndef ALICE_SOURCE_DIGEST
#define ALICE_SOURCE_DIGEST ""
#endif
extern "C" const char* alice_source_digest() { return ALICE_SOURCE_DIGEST; }

// The architecture name of the current device, e.g. "gfx950:sramecc+:xnack-".
extern "C" int alice_device_arch(char* out, int cap) {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    alice_set_error("no HIP device is available");
    return 1;
  }
  strncpy(out, prop.gcnArchName, cap - 1);
  out[cap - 1] = 0;
  return 0;
}
