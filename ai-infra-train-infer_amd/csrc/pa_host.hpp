// Host-side helpers shared by the C-ABI entry points: per-thread error text and launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "paged_attn.h"

namespace pa {

// Stores `msg` as this thread's last error and returns `code`.
int fail(int code, const char* msg);
// Returns PA_OK, or records hipGetLastError() under `where` and returns PA_ERR_LAUNCH.
int check_launch(const char* where);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace pa
