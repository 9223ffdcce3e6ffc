// Error text of the measuring library (its own copy of the helpers in pa_host.hpp, so that
// libpa_probes.so does not depend on libpaged_attn.so).
#include "pa_host.hpp"
#include "pa_probes.h"

#include <stdio.h>

namespace pa {

static thread_local char g_last_error[512] = "";

int fail(int code, const char* msg) {
  snprintf(g_last_error, sizeof(g_last_error), "%s", msg);
  return code;
}

int check_launch(const char* where) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return PA_OK;
  snprintf(g_last_error, sizeof(g_last_error), "%s: HIP error %d (%s)", where, (int)e, hipGetErrorString(e));
  return PA_ERR_LAUNCH;
}

}  // namespace pa

extern "C" const char* pa_probes_last_error(void) { return pa::g_last_error; }
