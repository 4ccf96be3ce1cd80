// Error text and version entry points of libmoe_gfx950.so.
#include "common.h"

static thread_local char g_err[512] = {0};

char* moe_err_buf() { return g_err; }

int moe_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int moe_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return moe_fail(MOE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MOE_OK;
}

extern "C" int moe_abi_version(void) { return 3; }

extern "C" const char* moe_last_error(void) { return g_err; }
