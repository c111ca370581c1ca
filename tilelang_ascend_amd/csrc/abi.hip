// Error channel, version and device queries of libtlq.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "tlq_common.h"

namespace tlq {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// Launch log of the calling thread (tlq_debug_launch_log): which kernels an entry point really launched, for benchmarks
// and tests that name the kernel they measured.  Off by default; a repeated entry is written once.
static thread_local bool g_log_on = false;
static thread_local char g_log[1024] = "";
static thread_local char g_log_last[160] = "";
static void log_launch(const char* what, const char* detail) {
  char entry[160];
  if (detail && detail[0])
    snprintf(entry, sizeof(entry), "%s [%s]", what, detail);
  else
    snprintf(entry, sizeof(entry), "%s", what);
  if (strcmp(entry, g_log_last) == 0) return;
  snprintf(g_log_last, sizeof(g_log_last), "%s", entry);
  const size_t used = strlen(g_log);
  if (used + strlen(entry) + 4 >= sizeof(g_log)) return;
  snprintf(g_log + used, sizeof(g_log) - used, "%s%s", used ? " + " : "", entry);
}

// Called right after a kernel launch: turns a launch failure into an error string.  detail: the kernel and its
// variant, for the launch log.  launch_count: how often the calling thread has come through here -- an entry point that
// returned an error without the count moving has refused its arguments and launched nothing.
static thread_local uint64_t g_launches = 0;
uint64_t launch_count() { return g_launches; }

bool check_launch(const char* what, const char* detail) {
  ++g_launches;
  if (g_log_on) log_launch(what, detail);
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

void tlq_debug_launch_log(int on) {
  tlq::g_log_on = on != 0;
  if (on) tlq::g_log[0] = 0, tlq::g_log_last[0] = 0;
}

const char* tlq_debug_launch_log_text(void) { return tlq::g_log; }

int tlq_device_cu_count(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  return n;
}

}  // extern "C"
