// Shared helpers of the gfx950 kernels: element types, wave64 reductions, error reporting.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define FLLM_F32 0
#define FLLM_BF16 1

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int kWave = 64;

// Records the first failure of a call; every entry point returns 0 or a negative code and the
// text is read back through fllm_last_error().
void fllm_set_error(const char *fmt, ...);
int fllm_check_launch(const char *what);
// 0 when the MFMA kernels are switched off (tests compare them with the plain kernels)
int fllm_fast_kernels_enabled(void);
// 1: prompt portions of heads of 64 and 128 use the 128-row attention kernel (default); 0: the 64-row kernel
int fllm_option_tile32(void);
// 0: the decode-shaped products choose their number of K slices themselves (default); n: n slices where that is possible
int fllm_option_linear_slices(void);
// 1: the parts of a split decode context are merged by the split that arrives last (default); 0: by a second kernel
int fllm_option_fused_merge(void);
// 1: prompt portions with long contexts and few rows share a row tile's keys among workgroups (default); 0: one workgroup a row tile
int fllm_option_prefill_parts(void);
// 1: decode-shaped products read bfloat16 activations straight from global memory (default); 0: they stage them in LDS
int fllm_option_x_direct(void);
// products of 17 to 64 rows: 1 (default) the kernel that suits the shape; 0 activations pass through LDS in chunks wherever
// that kernel can serve; 2 a K slice of the activations stays in LDS wherever that kernel can serve
int fllm_option_slab(void);
int fllm_option_wide_waves(void);
int fllm_option_resident_tiles(void);
int fllm_option_tile32_rows(void);
// 1: decode-shaped products of up to 8 rows use 8-row weight tiles with two K halves a product (default); 0: 16-row tiles
int fllm_option_dual_k(void);

// The device workspace of the current device (fllm_set_device_workspace): its first kWorkspaceCounterBytes are
// counters that every kernel leaves at zero, the rest is for partial results of the kernel that is running.
constexpr size_t kWorkspaceCounterBytes = 64 * 1024;      // plans.h counts with the same number (checked where both are seen)
bool fllm_device_workspace(void **base, size_t *bytes);

// Workgroups of one launch that meet in the workspace: a workgroup leaves its partial results there (relaxed
// agent-scope atomic stores, or the sc0 sc1 buffer stores of linear_skinny.hip), calls parts_published() and then
// counts itself with a relaxed agent-scope add; the workgroup that counts last calls parts_visible() and reads the
// parts of all (relaxed agent-scope atomic loads, sc0 sc1 buffer loads).
//
// FLLM_HANDOVER_SCOPE "agent" makes the two calls the release and acquire fences at agent scope that the HIP memory
// model asks for.  On gfx950 such a release writes the die's whole L2 back and the acquire drops it, and a decode
// step of 8 rows at the Llama-3.1-8B sizes takes 4.76 ms instead of 3.73 (measured; its K-sliced products and split
// contexts hand over 200 times a step), 3.41 instead of 3.34 ms at one row.  The default is therefore the form that
// rests on what the hardware does with these particular accesses, which is all the hand-over needs:
//   1. every part is written by stores with the sc1 bit (what an agent-scope atomic store is on gfx950): they are
//      written through to the memory side, which all eight dies share, and do not stay in the writer's L2;
//   2. s_waitcnt vmcnt(0) returns when those stores have been acknowledged from there;
//   3. only then is the counter's add issued, an atomic performed at the same memory-side point;
//   4. the reader issues its loads after the add that told it it is last has returned, and they carry sc1 too: they
//      are served from the memory side, not from a line its own die's L2 may still hold.
// A compiler fence at workgroup scope keeps the compiler from moving the stores, the add and the loads across each other.
// What this depends on and a change of hardware or compiler could break: that sc1 stores are acknowledged only once
// visible to the other dies (2), and that agent-scope atomic loads never hit in a die's L2 (4).
#ifndef FLLM_HANDOVER_SCOPE
#define FLLM_HANDOVER_SCOPE "workgroup"
#endif
__device__ __forceinline__ void parts_published() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, FLLM_HANDOVER_SCOPE);
    __builtin_amdgcn_s_waitcnt(0);
}
__device__ __forceinline__ void parts_visible() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, FLLM_HANDOVER_SCOPE); }

#define FLLM_REQUIRE(cond, ...)            \
    do {                                   \
        if (!(cond)) {                     \
            fllm_set_error(__VA_ARGS__);   \
            return -1;                     \
        }                                  \
    } while (0)

// Where a key's value lies in the pages.  Inside a page the keys of a key/value head are stored chunk by chunk:
// [kv_head][head_dim / 8][token][8], so that the 8 neighbouring values (16 bytes in bfloat16) of all tokens of the page lie
// together.  A decode step's products take 16 keys x 8 values a lane group: from this order that is 256 bytes in a row
// (two cache lines), from [token][head_dim] it would be 16 bytes of each of 16 rows (sixteen lines), which is what the
// memory pipeline of a compute unit is short of, not bytes (decode attention 8 x 32,768 keys: 182 -> 148 us).
// head_dim must be a multiple of 8.  Values are stored [kv_head][head_dim][token].
__host__ __device__ __forceinline__ size_t key_offset(size_t page, int kv_heads, int kvh, int page_size, int head_dim, int token, int d) {
    return ((((size_t)page * kv_heads + kvh) * (head_dim >> 3) + (d >> 3)) * page_size + token) * 8 + (d & 7);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Sum over a workgroup of NW waves, the same value in every thread; the waves' partial sums
// are added in wave order, so the result depends only on the data and the launch shape.
template <int NW> __device__ __forceinline__ float block_sum(float v, float *scratch /* NW floats */) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < NW; i++) total += scratch[i];
    return total;
}
template <int NW> __device__ __forceinline__ float block_max(float v, float *scratch) {
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float total = -INFINITY;
#pragma unroll
    for (int i = 0; i < NW; i++) total = fmaxf(total, scratch[i]);
    return total;
}

// Philox-4x32 with ten rounds (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3"): the counter words in,
// the output words in their place.  The sampler's draws and the random-weights generator use it.
struct Philox {
    uint32_t c0, c1, c2, c3;
    __device__ __forceinline__ void ten_rounds(uint32_t key_lo, uint32_t key_hi) {
#pragma unroll
        for (int round = 0; round < 10; round++) {
            const uint64_t left = (uint64_t)0xD2511F53u * c0;
            const uint64_t right = (uint64_t)0xCD9E8D57u * c2;
            const uint32_t next0 = (uint32_t)(right >> 32) ^ c1 ^ key_lo;
            const uint32_t next2 = (uint32_t)(left >> 32) ^ c3 ^ key_hi;
            c1 = (uint32_t)right;
            c3 = (uint32_t)left;
            c0 = next0;
            c2 = next2;
            key_lo += 0x9E3779B9u;
            key_hi += 0xBB67AE85u;
        }
    }
};
