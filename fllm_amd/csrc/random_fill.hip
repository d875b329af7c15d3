// Random weights on the device: the generator of fllm_amd/weights/random_init.py (its module text is the
// specification), evaluated with the same integer operations and the same single float32 operations, each
// rounded on its own (__fadd_rn, __fmul_rn, __fdiv_rn, __fsqrt_rn: never fused into a multiply-add), so that a tensor
// drawn here equals the one drawn on the host bit for bit.  The reference draws its test models on the host
// (rust/engine/src/tiny_model.rs:44-60); a model of many gigabytes is drawn where it will live.
#include "api.h"
#include "common.h"

namespace {

__device__ __forceinline__ float bits(uint32_t b) { return __uint_as_float(b); }

// acc = ((t0 x2 + t1) x2 + t2) ... x2 + last, two rounded operations a step
template <int N> __device__ __forceinline__ float horner(float x2, const uint32_t (&terms)[N], float last) {
    float acc = bits(terms[0]);
#pragma unroll
    for (int i = 1; i < N; i++) {
        const float product = acc * x2;
        acc = product + bits(terms[i]);
    }
    const float product = acc * x2;
    return product + last;
}

__device__ __forceinline__ float value_of(uint64_t index, uint32_t key_lo, uint32_t key_hi, int kind) {
    Philox g = {(uint32_t)index, (uint32_t)(index >> 32), 0u, 0u};
    g.ten_rounds(key_lo, key_hi);
    if (kind == 1) {   // 1 + U(-0.1, 0.1)
        const float u = ((float)(g.c0 >> 9) + 0.5f) / 8388608.0f;
        const float scaled = u * 0.2f;
        return 1.0f + (scaled - 0.1f);
    }
    // 0.02 sqrt(-2 ln u1) cos(2 pi u2)
    const uint32_t LOG_TERMS[4] = {0x3DE38E39u, 0x3E124925u, 0x3E4CCCCDu, 0x3EAAAAABu};                              // 1/9 ... 1/3
    const uint32_t SIN_TERMS[5] = {0xB2D7322Bu, 0x3638EF1Du, 0xB9500D01u, 0x3C088889u, 0xBE2AAAABu};                 // -1/11! ... -1/3!
    const uint32_t COS_TERMS[6] = {0x310F76C7u, 0xB493F27Eu, 0x37D00D01u, 0xBAB60B61u, 0x3D2AAAABu, 0xBF000000u};    // 1/12! ... -1/2!
    const float v = (float)((g.c0 >> 9) * 2u + 1u);      // odd and below 2^24: exact
    int e;
    float m = frexpf(v, &e);                              // v = m 2^e, m in [1/2, 1)
    if (m < bits(0x3F3504F3u)) {                          // below sqrt(1/2)
        m = m * 2.0f;
        e -= 1;
    }
    const float s = (m - 1.0f) / (m + 1.0f);
    const float exponent_part = (float)(e - 24) * bits(0x3F317218u);          // ln 2
    const float series = horner(s * s, LOG_TERMS, 1.0f);
    const float mantissa_part = (2.0f * s) * series;
    const float log_u = exponent_part + mantissa_part;
    const float radius = sqrtf(fmaxf(-2.0f * log_u, 0.0f));
    const uint32_t angle = g.c1 >> 9;
    const uint32_t quadrant = angle >> 21;
    const float j = (float)(angle & ((1u << 21) - 1u));
    const float x = ((j + 0.5f) / 2097152.0f) * bits(0x3FC90FDBu);            // pi / 2
    const float x2 = x * x;
    const float sine = x * horner(x2, SIN_TERMS, 1.0f);
    const float cosine = horner(x2, COS_TERMS, 1.0f);
    const float turn = quadrant == 0 ? cosine : quadrant == 1 ? -sine : quadrant == 2 ? -cosine : sine;
    const float unit = radius * turn;
    return 0.02f * unit;
}

template <typename T>
__global__ __launch_bounds__(256) void random_fill_kernel(T *out, uint64_t count, uint32_t key_lo, uint32_t key_hi, int kind) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride)
        out[i] = from_f32<T>(value_of(i, key_lo, key_hi, kind));
}

}  // namespace

extern "C" int fllm_random_fill(void *out, uint64_t count, uint32_t key_lo, uint32_t key_hi, int kind, int dtype,
                                hipStream_t stream) {
    FLLM_REQUIRE(kind == 0 || kind == 1, "fllm_random_fill: kind %d is neither 0 (normal) nor 1 (norm weight)", kind);
    FLLM_REQUIRE(dtype == FLLM_F32 || dtype == FLLM_BF16, "fllm_random_fill: element type %d unsupported", dtype);
    if (count == 0) return 0;
    FLLM_REQUIRE(out != nullptr, "fllm_random_fill: no output");
    const uint64_t blocks = (count + 255) / 256;
    const int grid = (int)(blocks < 256 * 64 ? blocks : 256 * 64);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(random_fill_kernel<float>, dim3(grid), dim3(256), 0, stream, (float *)out, count, key_lo, key_hi, kind);
    else
        hipLaunchKernelGGL(random_fill_kernel<bf16_t>, dim3(grid), dim3(256), 0, stream, (bf16_t *)out, count, key_lo, key_hi, kind);
    return fllm_check_launch("fllm_random_fill");
}
