// Error text of the last refused call, per host thread, and the launch check every entry point
// ends with. The library never prints and never aborts: the caller decides.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

void mllm_set_error(const char* format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(g_error, sizeof(g_error), format, args);
    va_end(args);
}

int mllm_check_launch(const char* what) {
    hipError_t status = hipGetLastError();
    if (status != hipSuccess) {
        mllm_set_error("%s: launch failed: %s", what, hipGetErrorString(status));
        return 2;
    }
    return 0;
}

MLLM_API const char* mllm_last_error() { return g_error; }

// Lets the loader check that it holds the library built from the sources it sees.
MLLM_API int mllm_abi_version() { return 1; }
