// Error bookkeeping and small host-only entry points of the C ABI.
#include "pa_host.hpp"

#include <stdio.h>
#include <string.h>

namespace pa {

static thread_local char g_last_error[512] = "";

int fail(int code, const char* msg) {
  snprintf(g_last_error, sizeof(g_last_error), "%s", msg);
  return code;
}

int check_launch(const char* where) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return PA_OK;
  snprintf(g_last_error, sizeof(g_last_error), "%s: HIP error %d (%s)", where, (int)e,
           hipGetErrorString(e));
  return PA_ERR_LAUNCH;
}

}  // namespace pa

extern "C" int pa_version(void) { return 3; }

extern "C" const char* pa_last_error(void) { return pa::g_last_error; }
