// Host-side plumbing of libbmt_hip.so that is not tied to one kernel file.
#include "bmt_host.h"
#include "../../include/bmt_hip.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace bmt {

static thread_local char g_last_error[256] = "";

int fail(int code, const char *what, hipError_t e) {
    if (e != hipSuccess)
        snprintf(g_last_error, sizeof(g_last_error), "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
    else
        snprintf(g_last_error, sizeof(g_last_error), "%s", what);
    return code;
}

int fail_message(int code, const char *what) { return fail(code, what); }

int device_cu_count() {
    static int cached[64];  // zero-initialised: 0 = not yet queried
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

}  // namespace bmt

extern "C" int is_bf16_supported(void) { return 1; }

extern "C" const char *bmt_hip_last_error(void) { return bmt::g_last_error; }
