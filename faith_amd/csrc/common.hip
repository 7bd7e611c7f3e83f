// Error bookkeeping of the C ABI (no kernels here).
#include "common.h"

namespace faith {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: HIP error %d (%s)", what, static_cast<int>(e), hipGetErrorString(e));
        return FAITH_ERR_LAUNCH;
    }
    return FAITH_OK;
}

}  // namespace faith

extern "C" const char *faith_last_error(void) { return faith::g_error; }

extern "C" int faith_version(void) { return 1; }
