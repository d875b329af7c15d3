// Error reporting shared by the entry points.
#include "api.h"
#include "common.h"
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

static thread_local char g_error[512] = "";

void fllm_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int fllm_check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fllm_set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return -2;
    }
    return 0;
}

static int g_fast_kernels = 1;
int fllm_fast_kernels_enabled(void) { return g_fast_kernels; }
extern "C" void fllm_set_fast_kernels(int on) { g_fast_kernels = on ? 1 : 0; }

// Kernel variants that can be switched for measurements and for tests that compare them.
static int g_tile32 = 1;
int fllm_option_tile32(void) { return g_tile32; }
extern "C" int fllm_set_option(const char *name, int value) {
    if (strcmp(name, "attention.tile32") == 0) {
        g_tile32 = value ? 1 : 0;
        return 0;
    }
    fllm_set_error("unknown option %s", name);
    return -1;
}

extern "C" const char *fllm_last_error(void) { return g_error; }
extern "C" int fllm_abi_version(void) { return 1; }
