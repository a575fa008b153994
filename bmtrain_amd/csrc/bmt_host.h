// Host-side helpers shared by the launchers: per-thread error text, device properties.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bmt {

// Records `what` (plus the HIP error string when `e` is given) as the calling
// thread's last error and returns `code`.
int fail(int code, const char *what, hipError_t e = hipSuccess);
// Same for code that does not see the HIP headers.
int fail_message(int code, const char *what);

// Number of compute units of the current device (cached per device).
int device_cu_count();

}  // namespace bmt
