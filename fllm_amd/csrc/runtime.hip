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
static int g_tile32_rows = 0;     // 0: chosen by the launch; 128 or 256
int fllm_option_tile32_rows(void) { return g_tile32_rows; }
static int g_wide_waves = 0;      // 0: planned
int fllm_option_wide_waves(void) { return g_wide_waves; }
static int g_resident_tiles = 1;  // q/k/v of up to 16 rows behind a prepared norm streams its tile-major copy (16-row tiles)
int fllm_option_resident_tiles(void) { return g_resident_tiles; }
static int g_slab = 1;
int fllm_option_slab(void) { return g_slab; }
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
    if (strcmp(name, "linear.slab") == 0) {
        g_slab = value < 0 ? 0 : (value > 2 ? 2 : value);
        return 0;
    }
    if (strcmp(name, "attention.tile32_rows") == 0) {
        g_tile32_rows = (value == 128 || value == 256) ? value : 0;
        return 0;
    }
    if (strcmp(name, "linear.resident_tiles") == 0) {
        g_resident_tiles = value != 0;
        return 0;
    }
    if (strcmp(name, "linear.wide_waves") == 0) {
        g_wide_waves = (value == 4 || value == 7 || value == 8) ? value : 0;
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

// ---------------------------------------------------------------------------------------------
// Probes of what the device delivers, for measurements that state a share of a measured ceiling beside the share
// of the published one.
// ---------------------------------------------------------------------------------------------
namespace {
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

// every workgroup reads a contiguous stretch with 16-byte loads, eight of them in flight a lane
__global__ void __launch_bounds__(256) probe_read_kernel(const u32x4_t *__restrict__ src, size_t chunks, unsigned int *sink) {
    const size_t per_block = (chunks + gridDim.x - 1) / gridDim.x;
    const size_t begin = (size_t)blockIdx.x * per_block, end = begin + per_block < chunks ? begin + per_block : chunks;
    u32x4_t acc = {0u, 0u, 0u, 0u};
    size_t i = begin + threadIdx.x;
    for (; i + 7 * 256 < end; i += 8 * 256) {
        u32x4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < 8; u++) acc ^= v[u];
    }
    for (; i < end; i += 256) acc ^= src[i];
    const unsigned int x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (x == 0x9e3779b9u) sink[blockIdx.x] = x;     // keeps the loads alive; written next to never
}

// four independent chains of 32x32x16 bfloat16 products a wave, two waves a SIMD
__global__ void __launch_bounds__(512) probe_mfma_kernel(float *sink, int iters) {
    bf16x8_t a, b;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = (bf16_t)(0.001f * (float)((threadIdx.x + i) & 15));
        b[i] = (bf16_t)(0.002f * (float)((threadIdx.x * 3 + i) & 7));
    }
    f32x16_t acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[c][i] = 0.f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int i = 0; i < 16; i++) s += acc[c][i];
    if (s == 12345.678f) sink[blockIdx.x * 512 + threadIdx.x] = s;
}
}  // namespace

extern "C" int fllm_probe_read(const void *src, size_t bytes, void *sink, int blocks, hipStream_t stream) {
    FLLM_REQUIRE(src != nullptr && sink != nullptr && bytes >= 16 && ((uintptr_t)src & 15) == 0, "probe_read: a 16-byte aligned buffer is required");
    FLLM_REQUIRE(blocks > 0 && blocks <= 65535 * 16, "probe_read: bad number of workgroups %d", blocks);
    hipLaunchKernelGGL(probe_read_kernel, dim3(blocks), dim3(256), 0, stream, (const u32x4_t *)src, bytes / 16, (unsigned int *)sink);
    return fllm_check_launch("probe_read");
}

extern "C" double fllm_probe_mfma_bf16(void *sink, int blocks, int iters, hipStream_t stream) {
    if (sink == nullptr || blocks <= 0 || iters <= 0) {
        fllm_set_error("probe_mfma: bad arguments");
        return -1.0;
    }
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(512), 0, stream, (float *)sink, iters);
    if (fllm_check_launch("probe_mfma") != 0) return -1.0;
    return 2.0 * 32 * 32 * 16 * 16.0 * iters * 8.0 * blocks;      // floating-point operations of the launch
}

extern "C" const char *fllm_last_error(void) { return g_error; }
extern "C" int fllm_abi_version(void) { return 11; }   // 11: fllm_linear_f32_tiled.  10: fllm_logprobs_processed, fllm_prepare_norm.  9: tiles for 17 to 64 rows, fllm_scaled_* take w_tiles.  8: weight tiles.  7: fllm_random_fill.  2: fllm_attention takes single_from; probes.  3: fllm_sample takes kinds.  4: fllm_logprobs.  5: FllmAdjustLists.  6: fllm_linear_add_normed, fllm_scaled_*
