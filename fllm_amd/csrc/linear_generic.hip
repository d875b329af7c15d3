// Plain tiled matrix product y = x w^T with float32 arithmetic: the true 32-bit path, and the
// fallback of the bfloat16 path for shapes the MFMA kernels refuse.  Every output element is one
// chain of fused multiply-adds over k = 0..K-1 in order, so its bits do not depend on how many
// rows the call has or on where the row sits in the batch.
#include "api.h"
#include "common.h"

int fllm_linear_bf16_fast(const void *x, int ldx, const void *w, const float *bias, void *out, int ldo, int M, int N, int K,
                          int out_mode, hipStream_t stream);   // linear_mfma.hip; returns 1 when it declines the shape

namespace {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;
constexpr int kThreads = (BM / TM) * (BN / TN);   // 256

template <typename T>
__global__ void __launch_bounds__(kThreads)
linear_tiled_kernel(const T *__restrict__ x, int ldx, const T *__restrict__ w, const float *__restrict__ bias,
                    void *__restrict__ out, int ldo, int M, int N, int K, int out_mode) {
    __shared__ float xs[BK][BM + 1];
    __shared__ float ws[BK][BN + 1];
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int tx = threadIdx.x % (BN / TN), ty = threadIdx.x / (BN / TN);
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
        // 64 rows x 16 k per operand: 1024 elements, 4 per thread
#pragma unroll
        for (int e = 0; e < (BM * BK) / kThreads; e++) {
            const int idx = threadIdx.x + e * kThreads;
            const int row = idx / BK, kk = idx % BK;
            const int gm = m0 + row, gn = n0 + row, gk = k0 + kk;
            xs[kk][row] = (gm < M && gk < K) ? to_f32<T>(x[(size_t)gm * ldx + gk]) : 0.f;
            ws[kk][row] = (gn < N && gk < K) ? to_f32<T>(w[(size_t)gn * K + gk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; kk++) {
            float a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = xs[kk][ty * TM + i];
#pragma unroll
            for (int j = 0; j < TN; j++) b[j] = ws[kk][tx * TN + j];
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int gm = m0 + ty * TM + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int gn = n0 + tx * TN + j;
            if (gn >= N) continue;
            float v = acc[i][j];
            if (bias) v += bias[gn];
            const size_t o = (size_t)gm * ldo + gn;
            if (out_mode == 0) ((T *)out)[o] = from_f32<T>(v);
            else if (out_mode == 1) ((float *)out)[o] = v;
            else ((float *)out)[o] += v;
        }
    }
}

}  // namespace

extern "C" int fllm_linear(const void *x, int ldx, const void *w, const float *bias, void *out, int ldo, int M, int N,
                           int K, int dtype, int out_mode, hipStream_t stream) {
    FLLM_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
    FLLM_REQUIRE(ldx >= K && ldo >= N, "linear: row strides ldx=%d ldo=%d are shorter than K=%d N=%d", ldx, ldo, K, N);
    FLLM_REQUIRE(out_mode >= 0 && out_mode <= 2, "linear: unknown out_mode %d", out_mode);
    if (M == 0) return 0;
    const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (dtype == FLLM_F32) {
        hipLaunchKernelGGL(linear_tiled_kernel<float>, grid, dim3(kThreads), 0, stream, (const float *)x, ldx,
                           (const float *)w, bias, out, ldo, M, N, K, out_mode);
    } else if (dtype == FLLM_BF16) {
        const int fast = fllm_linear_bf16_fast(x, ldx, w, bias, out, ldo, M, N, K, out_mode, stream);
        if (fast <= 0) return fast;
        hipLaunchKernelGGL(linear_tiled_kernel<bf16_t>, grid, dim3(kThreads), 0, stream, (const bf16_t *)x, ldx,
                           (const bf16_t *)w, bias, out, ldo, M, N, K, out_mode);
    } else {
        FLLM_REQUIRE(false, "linear: unknown dtype %d", dtype);
    }
    return fllm_check_launch("linear");
}
