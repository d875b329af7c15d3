// bfloat16 matrix products y = x w^T on the MFMA units of gfx950, float32 accumulation.
//
// Calls of up to 64 rows (decode steps) go to the weight-streaming kernel of linear_skinny.hip.
// `tiled` (M > 64, prompt portions) is a 128x128x64 LDS-tiled kernel, four waves of 64x64 each on
// v_mfma_f32_32x32x16_bf16, with register prefetch of the next tile.
//
// MFMA operand layouts used here (wave64):
//   16x16x32: A lane l holds A[m = l%16][k = 8*(l/16) .. +7]; B lane l holds B[k = 8*(l/16) .. +7][n = l%16];
//             D lane l holds D[m = 4*(l/16) + i][n = l%16], i = 0..3.
//   32x32x16: A lane l holds A[m = l%32][k = 8*(l/32) .. +7]; B likewise with n = l%32;
//             D lane l holds D[m = 8*(i/4) + 4*(l/32) + i%4][n = l%32], i = 0..15.
#include "api.h"
#include "common.h"

int fllm_linear_bf16_skinny(const void *x, int ldx, const void *w, const float *bias, void *out, int ldo, int M, int N,
                            int K, int out_mode, hipStream_t stream, const void *w_tiles = nullptr);   // linear_skinny.hip; 1: shape declined

namespace {

__device__ __forceinline__ bf16x8_t zero8() {
    bf16x8_t z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16_t)0.0f;
    return z;
}

__device__ __forceinline__ void store_out(void *out, size_t o, float v, int out_mode) {
    if (out_mode == 0) ((bf16_t *)out)[o] = (bf16_t)v;
    else if (out_mode == 1) ((float *)out)[o] = v;
    else ((float *)out)[o] += v;
}

// ---------------------------------------------------------------------------------------------
// tiled: any M
// ---------------------------------------------------------------------------------------------
constexpr int BM = 128, BN = 128, BK = 64, LDT = BK + 8;   // LDT: row pitch in LDS, padded against bank conflicts
constexpr int kTiledThreads = 256;
constexpr int kChunksPerThread = (BM * BK / 8) / kTiledThreads;   // 16-byte chunks per operand tile and thread: 4

__global__ void __launch_bounds__(kTiledThreads)
linear_tiled_mfma_kernel(const bf16_t *__restrict__ x, int ldx, const bf16_t *__restrict__ w, const float *__restrict__ bias,
                         void *__restrict__ out, int ldo, int M, int N, int K, int out_mode, int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDT];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDT];
    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous range of tiles so
    // that the tiles sharing a weight tile meet in one L2.
    int pid = blockIdx.x;
    const int total = tiles_m * tiles_n;
    if (total % 8 == 0) pid = (pid % 8) * (total / 8) + pid / 8;
    const int tile_m = pid % tiles_m, tile_n = pid / tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lg = lane >> 5;

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    bf16x8_t ra[kChunksPerThread], rb[kChunksPerThread];
    auto load_tile = [&](int k0) {
#pragma unroll
        for (int c = 0; c < kChunksPerThread; c++) {
            const int chunk = threadIdx.x + c * kTiledThreads;
            const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
            const int k = k0 + kc * 8;
            const int gm = m0 + row, gn = n0 + row;
            ra[c] = (gm < M && k < K) ? *(const bf16x8_t *)(x + (size_t)gm * ldx + k) : zero8();
            rb[c] = (gn < N && k < K) ? *(const bf16x8_t *)(w + (size_t)gn * K + k) : zero8();
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int c = 0; c < kChunksPerThread; c++) {
            const int chunk = threadIdx.x + c * kTiledThreads;
            const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
            *(bf16x8_t *)(As + row * LDT + kc * 8) = ra[c];
            *(bf16x8_t *)(Bs + row * LDT + kc * 8) = rb[c];
        }
    };

    load_tile(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        store_tile();
        __syncthreads();
        if (k0 + BK < K) load_tile(k0 + BK);   // in flight while this tile is multiplied
#pragma unroll
        for (int kk = 0; kk < BK / 16; kk++) {
            bf16x8_t a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++) a[i] = *(const bf16x8_t *)(As + (wm * 64 + i * 32 + l32) * LDT + kk * 16 + lg * 8);
#pragma unroll
            for (int j = 0; j < 2; j++) b[j] = *(const bf16x8_t *)(Bs + (wn * 64 + j * 32 + l32) * LDT + kk * 16 + lg * 8);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n0 + wn * 64 + j * 32 + l32;
            if (n >= N) continue;
            const float bv = bias ? bias[n] : 0.f;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (v / 4) + 4 * lg + (v % 4);
                if (m >= M) continue;
                store_out(out, (size_t)m * ldo + n, acc[i][j][v] + bv, out_mode);
            }
        }
}

}  // namespace

// 0: launched, negative: error, 1: shape declined (the caller uses the plain kernel)
int fllm_linear_bf16_fast(const void *x, int ldx, const void *w, const float *bias, void *out, int ldo, int M, int N, int K,
                          int out_mode, hipStream_t stream) {
    if (!fllm_fast_kernels_enabled()) return 1;
    // 16-byte operand loads: K and the row strides must be multiples of 8 elements, the bases aligned
    if (K % 8 != 0 || ldx % 8 != 0 || ((uintptr_t)x & 15) != 0 || ((uintptr_t)w & 15) != 0) return 1;
    const bf16_t *xb = (const bf16_t *)x, *wb = (const bf16_t *)w;
    if (M <= 64) {
        const int rc = fllm_linear_bf16_skinny(x, ldx, w, bias, out, ldo, M, N, K, out_mode, stream);
        if (rc != 1) return rc;
    }
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(linear_tiled_mfma_kernel, dim3(tiles_m * tiles_n), dim3(kTiledThreads), 0, stream, xb, ldx, wb, bias,
                       out, ldo, M, N, K, out_mode, tiles_m, tiles_n);
    return fllm_check_launch("linear_tiled");
}
