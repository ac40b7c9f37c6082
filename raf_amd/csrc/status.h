// Error reporting shared by the C-ABI entry points: a status code plus a thread-local message.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <exception>
#include <new>

#include "rafhip_optim.h"

namespace rafhip {

// Stores a printf-style message for rafhip_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// A plan's tables live on the device that was current when it was made; running it with another
// device current would hand the kernels pointers into the wrong address space.
inline int check_plan_device(const char* who, int plan_device) {
  int now = -1;
  if (hipGetDevice(&now) != hipSuccess) {
    (void)hipGetLastError();
    return fail(RAFHIP_ERR_NO_DEVICE, "%s: no HIP device available", who);
  }
  if (now != plan_device)
    return fail(RAFHIP_ERR_INVALID_ARG, "%s: the plan was made on device %d, the current device is %d", who,
                plan_device, now);
  return RAFHIP_OK;
}

// No C++ exception may cross the C boundary: entry points that allocate host memory (work lists,
// tables) run their body through this and report a failure as RAFHIP_ERR_HOST instead.
template <typename F>
int guarded(const char* who, F&& body) noexcept {
  try {
    return body();
  } catch (const std::bad_alloc&) {
    return fail(RAFHIP_ERR_HOST, "%s: out of host memory", who);
  } catch (const std::exception& e) {
    return fail(RAFHIP_ERR_HOST, "%s: %s", who, e.what());
  } catch (...) {
    return fail(RAFHIP_ERR_HOST, "%s: unknown C++ exception", who);
  }
}

}  // namespace rafhip

#define RAFHIP_HIP_TRY(expr)                                                                \
  do {                                                                                      \
    hipError_t _e = (expr);                                                                 \
    if (_e != hipSuccess)                                                                   \
      return ::rafhip::fail(RAFHIP_ERR_HIP, "%s failed: %s (%s:%d)", #expr,                 \
                            hipGetErrorString(_e), __FILE__, __LINE__);                     \
  } while (0)
