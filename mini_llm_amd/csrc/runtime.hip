// Error text of the last refused call, per host thread, and the launch check every entry point
// ends with. The library never prints and never aborts: the caller decides.
#include "common.h"

#include <atomic>
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

static std::atomic<unsigned long long> g_launches[MLLM_K_KINDS];
static const char* const g_kernel_names[MLLM_K_KINDS] = {
    "embed", "layernorm", "add", "cache_write", "attention_general", "attention_decode", "attention_prefill",
    "attention_prefill_stream", "pack", "convert", "decode_attention_half", "decode_mlp_half", "pending_sum",
    "pending_layernorm", "gemm_skinny", "gemm_tiled", "gemm_stream", "static_sum", "probe", "sample", "gemm_best", "choose",
};

void mllm_count_kernel(MllmKernel kind) { g_launches[kind].fetch_add(1, std::memory_order_relaxed); }

// The kinds of kernel this library launches, and how often each has been launched by this process
// (kind < 0: all together). A launch recorded into a graph counts once, at its capture.
MLLM_API int mllm_kernel_kinds() { return MLLM_K_KINDS; }
MLLM_API const char* mllm_kernel_name(int kind) { return kind >= 0 && kind < MLLM_K_KINDS ? g_kernel_names[kind] : ""; }
MLLM_API unsigned long long mllm_launch_count(int kind) {
    if (kind >= 0) return kind < MLLM_K_KINDS ? g_launches[kind].load(std::memory_order_relaxed) : 0ull;
    unsigned long long total = 0;
    for (int k = 0; k < MLLM_K_KINDS; ++k) total += g_launches[k].load(std::memory_order_relaxed);
    return total;
}

// Lets the loader check that it holds the library built from the sources it sees.
MLLM_API int mllm_abi_version() { return 1; }
