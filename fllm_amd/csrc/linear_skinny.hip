// Decode-step matrix products (M <= 64 rows) in bfloat16: y = f(x) w^T with the weight matrix
// streamed exactly once from HBM, and the work around the product folded into the same kernel:
//
//   prologue  BF16      x is bfloat16 [M, K]
//             NORM_F32  x is the float32 residual stream; the operand is x * norm_weight and the row's
//                       rsqrt(mean(x^2) + eps) is applied to the sums afterwards (a row scale commutes
//                       with the product), so RMSNorm costs no pass of its own
//   epilogue  STORE / STORE_F32 / ADD (add to the float32 residual stream)
//             QKV       rotate query and key lanes (pairs (2l, 2l+1)), write queries to a buffer and
//                       keys and values straight into the pages of each row's request
//             SWIGLU    rows n and I + n of the concatenated gate/up matrix go to one workgroup, which
//                       writes silu(gate) * up
//
// A weight row tile is 16 rows (32 for SWIGLU: 16 gate, 16 up).  The waves of a workgroup split K;
// weights go from global memory straight into MFMA A operands; partial sums are added in wave
// order through LDS, so the result does not depend on timing.  Up to 16 rows the activations are
// staged in LDS once per workgroup, which then walks over several row tiles; from 17 rows on a
// workgroup takes one tile and reads its B operands from global memory.
#include "api.h"
#include "common.h"

namespace {

enum { PRO_BF16 = 0, PRO_NORM_F32 = 1 };
enum { EPI_STORE = 0, EPI_STORE_F32 = 1, EPI_ADD = 2, EPI_QKV = 3, EPI_SWIGLU = 4 };

struct SkinnyArgs {
    const void *x;
    int ldx;
    const float *norm_w;
    float eps;
    const bf16_t *w;
    const float *bias;
    void *out;
    int ldo;
    int M, N, K;
    int kc;        // K chunk staged in LDS, a multiple of 128
    int ssq_off;   // byte offset of the sums of squares in LDS (behind the staging / reduction area)
    // QKV epilogue
    const int32_t *row_pos, *row_seg, *tables;
    int table_stride;
    const float *cos_t, *sin_t;
    int rope_dims;
    bf16_t *k_pages, *v_pages;
    int heads, kv_heads, head_dim, page_size, store_kv;
};

__device__ __forceinline__ bf16x8_t zero8() {
    bf16x8_t z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16_t)0.0f;
    return z;
}

// The epilogue of one output group: row m, columns nb .. nb + 3, sums s[t] (t: weight row tile).
template <int MT, int WAVES, int PRO, int EPI, int RT>
__device__ __forceinline__ void finish_group(const SkinnyArgs &a, const f32x4_t *red, const float *ssq_part, int mt, int l,
                                             int n0, int n_out) {
    const int M = a.M, N = a.N, K = a.K;
    do {
        const int m = mt * 16 + (l & 15);
        const int nb = n0 + (l >> 4) * 4;   // four consecutive output columns
        if (m >= M || nb >= n_out) continue;
        f32x4_t s[RT];
#pragma unroll
        for (int t = 0; t < RT; t++) {
            s[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int wv = 0; wv < WAVES; wv++) s[t] += red[((wv * RT + t) * MT + mt) * kWave + l];
        }
        if (PRO == PRO_NORM_F32) {
            float ss = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; wv++) ss += ssq_part[wv * 16 * MT + m];
            const float inv = 1.0f / sqrtf(ss / (float)K + a.eps);
#pragma unroll
            for (int t = 0; t < RT; t++) s[t] *= inv;
        }
        if (a.bias) {
#pragma unroll
            for (int t = 0; t < RT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (nb + i < n_out) s[t][i] += a.bias[t * n_out + nb + i];
        }
        if (EPI == EPI_STORE || EPI == EPI_STORE_F32 || EPI == EPI_ADD) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = nb + i;
                if (n >= N) continue;
                const size_t o = (size_t)m * a.ldo + n;
                if (EPI == EPI_STORE) ((bf16_t *)a.out)[o] = (bf16_t)s[0][i];
                else if (EPI == EPI_STORE_F32) ((float *)a.out)[o] = s[0][i];
                else ((float *)a.out)[o] += s[0][i];
            }
        } else if (EPI == EPI_SWIGLU) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = nb + i;
                if (n >= n_out) continue;
                const float gt = s[0][i], up = s[RT - 1][i];
                ((bf16_t *)a.out)[(size_t)m * a.ldo + n] = (bf16_t)(gt / (1.0f + expf(-gt)) * up);
            }
        } else {   // EPI_QKV: N = (heads + 2 kv_heads) * head_dim, head_dim a multiple of 4, so nb..nb+3 lie in one head
            const int seg = a.row_seg[m];
            if (seg < 0) continue;
            const int pos = a.row_pos[m];
            const int d = a.head_dim;
            const int hd = nb / d, j = nb - hd * d;          // head (q heads, then k heads, then v heads), lane in head
            float v[4] = {s[0][0], s[0][1], s[0][2], s[0][3]};
            if (hd < a.heads + a.kv_heads && j < a.rope_dims) {   // rope_dims is even; j is a multiple of 4
                const float *cs = a.cos_t + (size_t)pos * (a.rope_dims / 2), *sn = a.sin_t + (size_t)pos * (a.rope_dims / 2);
#pragma unroll
                for (int p = 0; p < 2; p++) {
                    if (j + 2 * p < a.rope_dims) {
                        const int l2 = (j + 2 * p) / 2;
                        const float x0 = v[2 * p], x1 = v[2 * p + 1];
                        v[2 * p] = x0 * cs[l2] - x1 * sn[l2];
                        v[2 * p + 1] = x1 * cs[l2] + x0 * sn[l2];
                    }
                }
            }
            if (hd < a.heads) {
                bf16_t *q = (bf16_t *)a.out + (size_t)m * a.ldo + nb;
#pragma unroll
                for (int i = 0; i < 4; i++) q[i] = (bf16_t)v[i];
            } else if (a.store_kv) {
                const int page = a.tables[(size_t)seg * a.table_stride + pos / a.page_size];
                const int off = pos % a.page_size;
                if (hd < a.heads + a.kv_heads) {
                    const int kvh = hd - a.heads;
                    bf16_t *kd = a.k_pages + (((size_t)page * a.kv_heads + kvh) * a.page_size + off) * d + j;
#pragma unroll
                    for (int i = 0; i < 4; i++) kd[i] = (bf16_t)v[i];
                } else {
                    const int kvh = hd - a.heads - a.kv_heads;
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        a.v_pages[(((size_t)page * a.kv_heads + kvh) * d + j + i) * a.page_size + off] = (bf16_t)v[i];
                }
            }
        }
        } while (false);
}

// ---------------------------------------------------------------------------------------------
// up to 16 rows: activations stay in LDS, workgroups walk over the weight row tiles
// ---------------------------------------------------------------------------------------------
// A workgroup of 8 waves stages the activations once (all of K when they fit, which is the case of
// the model's own shapes; else K chunk by K chunk for every tile) and then takes weight row tiles
// blockIdx.x, blockIdx.x + gridDim.x, ...: its waves split K, read their B operands from LDS and
// stream the weights with one block of loads in flight ahead of the products, across tile borders.
template <int PRO, int EPI>
__global__ void __launch_bounds__(8 * kWave) __attribute__((amdgpu_waves_per_eu(4, 4)))   // two workgroups per CU: 128 registers
skinny_resident_kernel(SkinnyArgs a, int red_off) {
    constexpr int MT = 1, WAVES = 8;
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int THREADS = WAVES * kWave;
    constexpr int U = 4 / RT;                      // k-steps of 32 per wave iteration: four weight loads in flight, four ahead
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N, K = a.K;
    const int n_out = EPI == EPI_SWIGLU ? N / 2 : N;
    const int ntiles = (n_out + 15) / 16;
    const int pitch = a.kc + 8;
    bf16_t *xs = (bf16_t *)smem;                                  // [M][pitch]
    f32x4_t *red = (f32x4_t *)(smem + red_off);                   // [WAVES][RT][64]
    float *ssq_part = (float *)(smem + a.ssq_off);                // [WAVES][16]
    const bool resident = a.kc >= K;                              // one chunk: staged once for all tiles
    const int kstep = WAVES * 32 * U;

    auto row_pointers = [&](int tile, const bf16_t *(&wp)[RT]) {
#pragma unroll
        for (int t = 0; t < RT; t++) {
            int row = tile * 16 + r;
            if (row >= n_out) row = n_out - 1;    // past the end: computed from a valid row, never stored
            wp[t] = a.w + (size_t)(row + t * n_out) * K + g * 8;
        }
    };
    auto load_w = [&](bf16x8_t (&wf)[RT][U], const bf16_t *const (&wp)[RT], int kabs, int kend) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool in = kabs + u * 32 + g * 8 < kend;
#pragma unroll
            for (int t = 0; t < RT; t++) wf[t][u] = in ? *(const bf16x8_t *)(wp[t] + kabs + u * 32) : zero8();
        }
    };

    int tile = blockIdx.x;
    const bf16_t *wp[RT];
    row_pointers(tile, wp);
    bf16x8_t wnext[RT][U];
    int have_tile = tile, have_k = wave * 32 * U;         // which block of weights `wnext` holds
    load_w(wnext, wp, wave * 32 * U, min(a.kc, K));     // in flight while the activations are staged
    if (PRO == PRO_NORM_F32 && lane < 16) ssq_part[wave * 16 + lane] = 0.f;
    bool staged = false;

    for (; tile < ntiles; tile += gridDim.x) {
        const bf16_t *wp_next[RT];
        row_pointers(tile + gridDim.x < ntiles ? tile + gridDim.x : tile, wp_next);
        f32x4_t acc[RT];
#pragma unroll
        for (int t = 0; t < RT; t++) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        for (int kc0 = 0; kc0 < K; kc0 += a.kc) {
            const int kcn = min(a.kc, K - kc0);           // a multiple of 8
            if (!staged) {
                __syncthreads();                           // whoever still reads the staging area is done
                if (PRO == PRO_BF16) {
                    const bf16_t *x = (const bf16_t *)a.x;
                    const int per_row = kcn / 8;
                    for (int idx = threadIdx.x; idx < M * per_row; idx += THREADS) {
                        const int m = idx / per_row, c = idx - m * per_row;
                        *(bf16x8_t *)(xs + m * pitch + c * 8) = *(const bf16x8_t *)(x + (size_t)m * a.ldx + kc0 + c * 8);
                    }
                } else {
                    const float *x = (const float *)a.x;
                    const int per_row = kcn / 8;
                    const int per_row_pad = (per_row + kWave - 1) / kWave * kWave;   // a wave never straddles two rows
                    const int total = M * per_row_pad;
                    constexpr int PASSES = 2;                                         // loads of two passes are in flight together
                    for (int base = threadIdx.x; base < total; base += PASSES * THREADS) {
                        f32x4_t xv[PASSES][2], wv[PASSES][2];
                        int mrow[PASSES], col[PASSES];
                        bool ok[PASSES];
#pragma unroll
                        for (int j = 0; j < PASSES; j++) {
                            const int idx = base + j * THREADS;
                            mrow[j] = idx / per_row_pad;
                            col[j] = (idx - mrow[j] * per_row_pad) * 8;
                            ok[j] = idx < total && col[j] < kcn;
                            if (ok[j]) {
                                const float *xp = x + (size_t)mrow[j] * a.ldx + kc0 + col[j];
                                xv[j][0] = *(const f32x4_t *)xp;
                                xv[j][1] = *(const f32x4_t *)(xp + 4);
                                wv[j][0] = *(const f32x4_t *)(a.norm_w + kc0 + col[j]);
                                wv[j][1] = *(const f32x4_t *)(a.norm_w + kc0 + col[j] + 4);
                            }
                        }
#pragma unroll
                        for (int j = 0; j < PASSES; j++) {
                            if (base - threadIdx.x + j * THREADS + wave * kWave >= total) continue;   // the whole wave is past the end
                            float ss = 0.f;
                            if (ok[j]) {
                                bf16x8_t v;
#pragma unroll
                                for (int i = 0; i < 4; i++) {
                                    ss += xv[j][0][i] * xv[j][0][i] + xv[j][1][i] * xv[j][1][i];
                                    v[i] = (bf16_t)(xv[j][0][i] * wv[j][0][i]);
                                    v[4 + i] = (bf16_t)(xv[j][1][i] * wv[j][1][i]);
                                }
                                *(bf16x8_t *)(xs + mrow[j] * pitch + col[j]) = v;
                            }
                            ss = wave_sum(ss);
                            if (lane == 0) ssq_part[wave * 16 + mrow[j]] += ss;
                        }
                    }
                }
                __syncthreads();
                staged = resident;
            }
            for (int k0 = wave * 32 * U; k0 < kcn; k0 += kstep) {
                bf16x8_t wf[RT][U], xf[U];
                if (have_tile != tile || have_k != kc0 + k0) load_w(wnext, wp, kc0 + k0, kc0 + kcn);   // not prefetched
#pragma unroll
                for (int t = 0; t < RT; t++)
#pragma unroll
                    for (int u = 0; u < U; u++) wf[t][u] = wnext[t][u];
                // the next weights of this wave: the rest of this chunk, the next chunk, or the next tile
                if (k0 + kstep < kcn) {
                    load_w(wnext, wp, kc0 + k0 + kstep, kc0 + kcn);
                    have_tile = tile, have_k = kc0 + k0 + kstep;
                } else if (kc0 + a.kc < K) {
                    load_w(wnext, wp, kc0 + a.kc + wave * 32 * U, min(kc0 + 2 * a.kc, K));
                    have_tile = tile, have_k = kc0 + a.kc + wave * 32 * U;
                } else if (tile + gridDim.x < ntiles) {
                    load_w(wnext, wp_next, wave * 32 * U, min(a.kc, K));
                    have_tile = tile + gridDim.x, have_k = wave * 32 * U;
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int k = k0 + u * 32 + g * 8;
                    xf[u] = (k < kcn && r < M) ? *(const bf16x8_t *)(xs + r * pitch + k) : zero8();
                }
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int t = 0; t < RT; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[t][u], xf[u], acc[t], 0, 0, 0);
            }
        }
#pragma unroll
        for (int t = 0; t < RT; t++) red[(wave * RT + t) * kWave + lane] = acc[t];
        __syncthreads();
        if (threadIdx.x < kWave) finish_group<MT, WAVES, PRO, EPI, RT>(a, red, ssq_part, 0, threadIdx.x, tile * 16, n_out);
        __syncthreads();      // the sums have been read: the next tile may overwrite them
        if (PRO == PRO_NORM_F32 && !resident && lane < 16) ssq_part[wave * 16 + lane] = 0.f;
#pragma unroll
        for (int t = 0; t < RT; t++) wp[t] = wp_next[t];
    }
}

// ---------------------------------------------------------------------------------------------
// 17 to 64 rows: operands straight from global memory, one weight row tile per workgroup
// ---------------------------------------------------------------------------------------------
template <int MT, int WAVES, int EPI>
__global__ void __launch_bounds__(WAVES * kWave)
skinny_direct_kernel(SkinnyArgs a) {
    constexpr int RT = 1, PRO = PRO_BF16;
    constexpr int THREADS = WAVES * kWave;
    constexpr int U = 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N, K = a.K;
    const int n0 = blockIdx.x * 16;
    int wrow = n0 + r;
    if (wrow >= N) wrow = N - 1;   // past the end: computed from a valid row, never stored
    const bf16_t *wp = a.w + (size_t)wrow * K + g * 8;
    const bf16_t *x = (const bf16_t *)a.x;
    f32x4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    for (int k0 = wave * 32 * U; k0 < K; k0 += WAVES * 32 * U) {
        bf16x8_t wf[U], xf[MT][U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + u * 32 + g * 8;
            const bool in = k < K;
            wf[u] = in ? *(const bf16x8_t *)(wp + k0 + u * 32) : zero8();
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                xf[mt][u] = (in && mt * 16 + r < M) ? *(const bf16x8_t *)(x + (size_t)(mt * 16 + r) * a.ldx + k) : zero8();
        }
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], xf[mt][u], acc[mt], 0, 0, 0);
    }
    f32x4_t *red = (f32x4_t *)smem;   // [WAVES][MT][64]
#pragma unroll
    for (int mt = 0; mt < MT; mt++) red[(wave * MT + mt) * kWave + lane] = acc[mt];
    __syncthreads();
    for (int e = threadIdx.x; e < MT * kWave; e += THREADS)
        finish_group<MT, WAVES, PRO, EPI, RT>(a, red, nullptr, e / kWave, e % kWave, n0, N);
}

int device_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

template <int PRO, int EPI>
int launch_resident(SkinnyArgs a, hipStream_t stream) {
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int WAVES = 8;
    const int kpad = (a.K + 127) / 128 * 128;
    // all of K when the rows fit into 136 KiB (one workgroup per CU; two when they fit into 64 KiB), else chunks of 64 KiB
    int kc = kpad;
    if ((size_t)a.M * (kpad + 8) * sizeof(bf16_t) > 136 * 1024) {
        kc = ((int)(64 * 1024 / sizeof(bf16_t) / a.M) - 8) / 128 * 128;
        if (kc < 128) return 1;
    }
    a.kc = kc;
    const size_t stage = ((size_t)a.M * (kc + 8) * sizeof(bf16_t) + 15) / 16 * 16;
    const size_t red = (size_t)WAVES * RT * kWave * sizeof(f32x4_t);
    const size_t smem = stage + red + (size_t)WAVES * 16 * sizeof(float);
    a.ssq_off = (int)(stage + red);
    const int n_out = EPI == EPI_SWIGLU ? a.N / 2 : a.N;
    const int ntiles = (n_out + 15) / 16;
    const int per_cu = smem <= 76 * 1024 ? 2 : 1;
    // every workgroup takes the same number of tiles (or one fewer): 896 tiles on 512 slots run as 448 x 2
    const int slots = device_cus() * per_cu;
    const int rounds = (ntiles + slots - 1) / slots;
    const int grid = (ntiles + rounds - 1) / rounds;
    static bool attribute_set = false;   // more than the default 64 KiB of dynamic LDS has to be asked for once
    if (!attribute_set) {
        const hipError_t e = hipFuncSetAttribute((const void *)skinny_resident_kernel<PRO, EPI>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        FLLM_REQUIRE(e == hipSuccess, "linear_skinny: cannot raise the LDS limit: %s", hipGetErrorString(e));
        attribute_set = true;
    }
    hipLaunchKernelGGL((skinny_resident_kernel<PRO, EPI>), dim3(grid), dim3(WAVES * kWave), smem, stream, a, (int)stage);
    return fllm_check_launch("linear_skinny");
}

template <int MT, int WAVES, int EPI>
int launch_direct(const SkinnyArgs &a, hipStream_t stream) {
    const size_t smem = (size_t)WAVES * MT * kWave * sizeof(f32x4_t);
    hipLaunchKernelGGL((skinny_direct_kernel<MT, WAVES, EPI>), dim3((a.N + 15) / 16), dim3(WAVES * kWave), smem, stream, a);
    return fllm_check_launch("linear_skinny");
}

template <int PRO, int EPI>
int dispatch(const SkinnyArgs &a, hipStream_t stream) {
    const int mt = (a.M + 15) / 16;
    if (mt == 1) return launch_resident<PRO, EPI>(a, stream);
    if constexpr (PRO == PRO_BF16 && (EPI == EPI_STORE || EPI == EPI_STORE_F32 || EPI == EPI_ADD)) {
        const bool wide = (a.N + 15) / 16 < 1024;   // few row tiles: more waves per tile keep enough loads in flight
#define FLLM_GO(MT) return wide ? launch_direct<MT, 16, EPI>(a, stream) : launch_direct<MT, 8, EPI>(a, stream)
        if (mt == 2) { FLLM_GO(2); }
        if (mt == 3) { FLLM_GO(3); }
        FLLM_GO(4);
#undef FLLM_GO
    }
    return 1;   // the fused forms are for up to 16 rows
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// The decode-shaped product of fllm_linear.  0: launched, negative: error, 1: shape declined.
int fllm_linear_bf16_skinny(const void *x, int ldx, const void *w, const float *bias, void *out, int ldo, int M, int N,
                            int K, int out_mode, hipStream_t stream) {
    if (M > 64 || K % 8 != 0 || ldx % 8 != 0 || !aligned16(x) || !aligned16(w)) return 1;
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = ldx;
    a.w = (const bf16_t *)w;
    a.bias = bias;
    a.out = out;
    a.ldo = ldo;
    a.M = M;
    a.N = N;
    a.K = K;
    if (out_mode == 0) return dispatch<PRO_BF16, EPI_STORE>(a, stream);
    if (out_mode == 1) return dispatch<PRO_BF16, EPI_STORE_F32>(a, stream);
    return dispatch<PRO_BF16, EPI_ADD>(a, stream);
}

// The fused forms read the float32 rows once per workgroup: worth it while there are few rows.
extern "C" int fllm_fused_decode_supported(int M, int K) { return (M >= 1 && M <= 16 && K % 8 == 0) ? 1 : 0; }

extern "C" int fllm_norm_linear(const float *x, const float *norm_w, float eps, const void *w, const float *bias, void *out,
                                int M, int N, int K, hipStream_t stream) {
    FLLM_REQUIRE(fllm_fused_decode_supported(M, K), "norm_linear: takes 1..16 rows and K a multiple of 8 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(aligned16(x) && aligned16(w) && aligned16(norm_w), "norm_linear: operands must be 16-byte aligned");
    FLLM_REQUIRE(eps > 0.f, "norm_linear: eps must be positive");
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = K;
    a.norm_w = norm_w;
    a.eps = eps;
    a.w = (const bf16_t *)w;
    a.bias = bias;
    a.out = out;
    a.ldo = N;
    a.M = M;
    a.N = N;
    a.K = K;
    const int rc = dispatch<PRO_NORM_F32, EPI_STORE>(a, stream);
    FLLM_REQUIRE(rc != 1, "norm_linear: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

extern "C" int fllm_norm_gate_up_swiglu(const float *x, const float *norm_w, float eps, const void *w_gate_up,
                                        const float *bias, void *out, int M, int inter, int K, hipStream_t stream) {
    FLLM_REQUIRE(fllm_fused_decode_supported(M, K), "norm_gate_up_swiglu: takes 1..16 rows and K a multiple of 8 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(aligned16(x) && aligned16(w_gate_up) && aligned16(norm_w), "norm_gate_up_swiglu: operands must be 16-byte aligned");
    FLLM_REQUIRE(eps > 0.f && inter > 0, "norm_gate_up_swiglu: bad eps or size");
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = K;
    a.norm_w = norm_w;
    a.eps = eps;
    a.w = (const bf16_t *)w_gate_up;
    a.bias = bias;
    a.out = out;
    a.ldo = inter;
    a.M = M;
    a.N = 2 * inter;
    a.K = K;
    const int rc = dispatch<PRO_NORM_F32, EPI_SWIGLU>(a, stream);
    FLLM_REQUIRE(rc != 1, "norm_gate_up_swiglu: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

extern "C" int fllm_norm_qkv_rope_store(const float *x, const float *norm_w, float eps, const void *w_qkv, const float *bias,
                                        void *q_out, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                                        int table_stride, const float *cos_table, const float *sin_table, int rope_dims,
                                        void *k_pages, void *v_pages, int M, int heads, int kv_heads, int head_dim, int K,
                                        int page_size, int store_kv, hipStream_t stream) {
    FLLM_REQUIRE(fllm_fused_decode_supported(M, K), "norm_qkv_rope_store: takes 1..16 rows and K a multiple of 8 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(aligned16(x) && aligned16(w_qkv) && aligned16(norm_w), "norm_qkv_rope_store: operands must be 16-byte aligned");
    FLLM_REQUIRE(head_dim % 4 == 0 && rope_dims % 2 == 0 && rope_dims <= head_dim && rope_dims >= 0,
                 "norm_qkv_rope_store: head_dim %d must be a multiple of 4 and rope_dims %d even and no larger", head_dim, rope_dims);
    FLLM_REQUIRE(heads > 0 && kv_heads > 0 && page_size > 0 && table_stride > 0 && eps > 0.f, "norm_qkv_rope_store: bad sizes");
    FLLM_REQUIRE(!store_kv || (k_pages && v_pages), "norm_qkv_rope_store: pages missing");
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = K;
    a.norm_w = norm_w;
    a.eps = eps;
    a.w = (const bf16_t *)w_qkv;
    a.bias = bias;
    a.out = q_out;
    a.ldo = heads * head_dim;
    a.M = M;
    a.N = (heads + 2 * kv_heads) * head_dim;
    a.K = K;
    a.row_pos = row_pos;
    a.row_seg = row_seg;
    a.tables = tables;
    a.table_stride = table_stride;
    a.cos_t = cos_table;
    a.sin_t = sin_table;
    a.rope_dims = rope_dims;
    a.k_pages = (bf16_t *)k_pages;
    a.v_pages = (bf16_t *)v_pages;
    a.heads = heads;
    a.kv_heads = kv_heads;
    a.head_dim = head_dim;
    a.page_size = page_size;
    a.store_kv = store_kv;
    const int rc = dispatch<PRO_NORM_F32, EPI_QKV>(a, stream);
    FLLM_REQUIRE(rc != 1, "norm_qkv_rope_store: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}
