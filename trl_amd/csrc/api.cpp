// Host-only part of the C ABI: version, thread-local error text, launch status.
#include <stdarg.h>
#include <stdio.h>

#include "common.hpp"

namespace trlk {
namespace {
thread_local char g_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_error[0] = '\0'; }

int launch_status(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return TRLK_OK;
    snprintf(g_error, sizeof(g_error), "%s: launch failed: %s", what, hipGetErrorString(e));
    return int(e);
}
}  // namespace trlk

extern "C" int trlk_version(void) { return TRLK_VERSION; }

extern "C" const char* trlk_last_error(void) { return trlk::g_error; }
