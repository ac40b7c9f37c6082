// Status / error-string plumbing of the C ABI.
#include "status.h"

#include <cstring>

namespace rafhip {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_error[0] = '\0'; }

}  // namespace rafhip

extern "C" {

int rafhip_abi_version(void) { return RAFHIP_ABI_VERSION; }

const char* rafhip_last_error(void) { return rafhip::g_error; }

int rafhip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();  // a host without a GPU is not an error here
    return 0;
  }
  return n;
}

}  // extern "C"
