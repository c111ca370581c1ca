// Error channel, version and device queries of libtlq.
#include <stdarg.h>
#include <stdio.h>

#include "tlq_common.h"

namespace tlq {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// Called right after a kernel launch: turns a launch failure into an error string.
bool check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return false;
  }
  return true;
}

}  // namespace tlq

extern "C" {

int tlq_abi_version(void) { return TLQ_ABI_VERSION; }

const char* tlq_last_error(void) { return tlq::g_error; }

int tlq_device_cu_count(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  return n;
}

}  // extern "C"
