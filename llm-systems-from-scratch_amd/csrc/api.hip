// Error bookkeeping and version string of the C ABI.
#include <hip/hip_runtime.h>
#include <string.h>

#include "launch.hpp"

static thread_local char g_last_error[256] = "";

int set_error(int code, const char* msg) {
    strncpy(g_last_error, msg ? msg : "", sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return code;
}

extern "C" const char* mi355_last_error(void) { return g_last_error; }

extern "C" const char* mi355_version(void) { return "mi355attn 0.1 (gfx950)"; }
