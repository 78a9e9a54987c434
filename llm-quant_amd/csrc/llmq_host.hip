// Host-side plumbing of the C ABI: version, per-thread error text, launch checking.
#include <stdarg.h>
#include <stdio.h>

#include "llmq_device.h"

namespace {
thread_local char g_error[512] = "";
}

namespace llmq_host {

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int fail_invalid(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return static_cast<int>(hipErrorInvalidValue);
}

int check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(err));
    return static_cast<int>(err);
  }
  return 0;
}

}  // namespace llmq_host

extern "C" int llmq_abi_version(void) { return 1; }
extern "C" const char* llmq_last_error(void) { return g_error; }
