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
static int g_linear_slices = 0;
static int g_dual_k = 1;
static int g_x_direct = 1;
int fllm_option_x_direct(void) { return g_x_direct; }
static int g_fused_merge = 1;
int fllm_option_fused_merge(void) { return g_fused_merge; }
static int g_prefill_parts = 1;
int fllm_option_prefill_parts(void) { return g_prefill_parts; }
int fllm_option_dual_k(void) { return g_dual_k; }
int fllm_option_tile32(void) { return g_tile32; }
int fllm_option_linear_slices(void) { return g_linear_slices; }
extern "C" int fllm_set_option(const char *name, int value) {
    if (strcmp(name, "attention.fused_merge") == 0) {
        g_fused_merge = value ? 1 : 0;
        return 0;
    }
    if (strcmp(name, "attention.prefill_parts") == 0) {
        g_prefill_parts = value > 0 ? value : 0;
        return 0;
    }
    if (strcmp(name, "linear.x_direct") == 0) {
        g_x_direct = value ? 1 : 0;
        return 0;
    }
    if (strcmp(name, "linear.dual_k") == 0) {
        g_dual_k = value ? 1 : 0;
        return 0;
    }
    if (strcmp(name, "linear.slices") == 0) {
        g_linear_slices = value > 0 ? value : 0;
        return 0;
    }
    if (strcmp(name, "attention.tile32") == 0) {
        g_tile32 = value ? 1 : 0;
        return 0;
    }
    fllm_set_error("unknown option %s", name);
    return -1;
}

// Device memory handed over by the host program, one block per device: counters first, partial results behind them.
static struct {
    void *base;
    size_t bytes;
} g_workspace[16];

bool fllm_device_workspace(void **base, size_t *bytes) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16 || g_workspace[dev].base == nullptr) return false;
    *base = g_workspace[dev].base;
    *bytes = g_workspace[dev].bytes;
    return true;
}

extern "C" int fllm_set_device_workspace(void *workspace, size_t bytes) {
    int dev = 0;
    FLLM_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 16, "set_device_workspace: no current device");
    FLLM_REQUIRE(workspace == nullptr || (bytes > kWorkspaceCounterBytes && ((uintptr_t)workspace & 255) == 0),
                 "set_device_workspace: the workspace must be 256-byte aligned and larger than %zu bytes",
                 (size_t)kWorkspaceCounterBytes);
    g_workspace[dev].base = workspace;
    g_workspace[dev].bytes = workspace ? bytes : 0;
    return 0;
}

extern "C" const char *fllm_last_error(void) { return g_error; }
extern "C" int fllm_abi_version(void) { return 1; }
