// Embedding gather, RMSNorm, SwiGLU and rotary + cache store.  All arithmetic is float32; the
// element type only says how operands are stored.
#include "api.h"
#include "common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

template <typename T>
__global__ void __launch_bounds__(kBlock)
embed_kernel(const int32_t *__restrict__ ids, const T *__restrict__ table, float *__restrict__ out, int width, int vocab,
             float scale) {
    const int r = blockIdx.x;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // ids are validated on the host; never read outside the table
    const T *src = table + (size_t)id * width;
    float *dst = out + (size_t)r * width;
    for (int c = threadIdx.x; c < width; c += kBlock) dst[c] = to_f32<T>(src[c]) * scale;
}

// One workgroup per output row.  The sum of squares is taken in a fixed order (thread t adds
// elements t, t + 256, ...; then lanes, then waves), so a row gives the same bits whatever else
// is in the batch.
template <typename T>
__global__ void __launch_bounds__(kBlock)
rmsnorm_kernel(const float *__restrict__ x, const int32_t *__restrict__ rows, const float *__restrict__ weight,
               T *__restrict__ out, int width, float eps) {
    __shared__ float scratch[kWaves];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    const float *src = x + (size_t)r * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += kBlock) {
        const float v = src[c];
        ss += v * v;
    }
    ss = block_sum<kWaves>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    T *dst = out + (size_t)i * width;
    for (int c = threadIdx.x; c < width; c += kBlock) dst[c] = from_f32<T>(src[c] * (inv * weight[c]));
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
swiglu_kernel(const T *__restrict__ gu, T *__restrict__ out, int rows, int inter) {
    const size_t total = (size_t)rows * inter;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock) {
        const size_t r = i / inter, j = i - r * inter;
        const float g = to_f32<T>(gu[r * 2 * inter + j]);
        const float u = to_f32<T>(gu[r * 2 * inter + inter + j]);
        out[i] = from_f32<T>(g / (1.0f + expf(-g)) * u);
    }
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
rope_kv_store_kernel(T *__restrict__ qkv, const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seg,
                     const int32_t *__restrict__ tables, int table_stride, const float *__restrict__ cos_table,
                     const float *__restrict__ sin_table, T *__restrict__ k_pages, T *__restrict__ v_pages, int heads,
                     int kv_heads, int head_dim, int rope_dims, int pairing, int page_size, int store_kv) {
    const int r = blockIdx.x;
    const int seg = row_seg[r];
    if (seg < 0) return;   // padding row
    const int pos = row_pos[r];
    const int half = rope_dims / 2;
    const float *cs = cos_table + (size_t)pos * half;
    const float *sn = sin_table + (size_t)pos * half;
    T *row = qkv + (size_t)r * (heads + 2 * kv_heads) * head_dim;

    // queries, in place
    for (int i = threadIdx.x; i < heads * half; i += kBlock) {
        const int h = i / half, l = i - h * half;
        const int ia = pairing ? 2 * l : l, ib = pairing ? 2 * l + 1 : l + half;
        T *head = row + (size_t)h * head_dim;
        const float a = to_f32<T>(head[ia]), b = to_f32<T>(head[ib]);
        head[ia] = from_f32<T>(a * cs[l] - b * sn[l]);
        head[ib] = from_f32<T>(b * cs[l] + a * sn[l]);
    }
    if (!store_kv) {
        // a layer that reads another layer's cache still rotates nothing else
        return;
    }
    const int page = tables[(size_t)seg * table_stride + pos / page_size];
    const int off = pos % page_size;
    const T *krow = row + (size_t)heads * head_dim;
    const T *vrow = krow + (size_t)kv_heads * head_dim;
    // keys: rotated lanes, then the lanes rotary leaves alone
    for (int i = threadIdx.x; i < kv_heads * half; i += kBlock) {
        const int h = i / half, l = i - h * half;
        const int ia = pairing ? 2 * l : l, ib = pairing ? 2 * l + 1 : l + half;
        const T *head = krow + (size_t)h * head_dim;
        const float a = to_f32<T>(head[ia]), b = to_f32<T>(head[ib]);
        T *dst = k_pages + (((size_t)page * kv_heads + h) * page_size + off) * head_dim;
        dst[ia] = from_f32<T>(a * cs[l] - b * sn[l]);
        dst[ib] = from_f32<T>(b * cs[l] + a * sn[l]);
    }
    const int rest = head_dim - rope_dims;
    for (int i = threadIdx.x; i < kv_heads * rest; i += kBlock) {
        const int h = i / rest, c = rope_dims + (i - h * rest);
        k_pages[(((size_t)page * kv_heads + h) * page_size + off) * head_dim + c] = krow[(size_t)h * head_dim + c];
    }
    // values, stored transposed inside the page: [head_dim][token]
    for (int i = threadIdx.x; i < kv_heads * head_dim; i += kBlock) {
        const int h = i / head_dim, c = i - h * head_dim;
        v_pages[(((size_t)page * kv_heads + h) * head_dim + c) * page_size + off] = vrow[i];
    }
}

}  // namespace

extern "C" int fllm_embed(const int32_t *ids, const void *table, float *out, int rows, int width, int vocab,
                          int table_dtype, float scale, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && vocab > 0, "embed: bad sizes rows=%d width=%d vocab=%d", rows, width, vocab);
    if (rows == 0) return 0;
    if (table_dtype == FLLM_F32)
        hipLaunchKernelGGL(embed_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, ids, (const float *)table, out, width,
                           vocab, scale);
    else if (table_dtype == FLLM_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, ids, (const bf16_t *)table, out,
                           width, vocab, scale);
    else
        FLLM_REQUIRE(false, "embed: unknown dtype %d", table_dtype);
    return fllm_check_launch("embed");
}

extern "C" int fllm_rmsnorm(const float *x, const int32_t *rows, const float *weight, void *out, int count, int width,
                            float eps, int out_dtype, hipStream_t stream) {
    FLLM_REQUIRE(count >= 0 && width > 0, "rmsnorm: bad sizes count=%d width=%d", count, width);
    FLLM_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive");
    if (count == 0) return 0;
    if (out_dtype == FLLM_F32)
        hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(count), dim3(kBlock), 0, stream, x, rows, weight, (float *)out,
                           width, eps);
    else if (out_dtype == FLLM_BF16)
        hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(count), dim3(kBlock), 0, stream, x, rows, weight, (bf16_t *)out,
                           width, eps);
    else
        FLLM_REQUIRE(false, "rmsnorm: unknown dtype %d", out_dtype);
    return fllm_check_launch("rmsnorm");
}

extern "C" int fllm_swiglu(const void *gate_up, void *out, int rows, int inter, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && inter > 0, "swiglu: bad sizes rows=%d inter=%d", rows, inter);
    if (rows == 0) return 0;
    const size_t total = (size_t)rows * inter;
    const int grid = (int)((total + kBlock - 1) / kBlock < 65535 ? (total + kBlock - 1) / kBlock : 65535);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(swiglu_kernel<float>, dim3(grid), dim3(kBlock), 0, stream, (const float *)gate_up, (float *)out,
                           rows, inter);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3(grid), dim3(kBlock), 0, stream, (const bf16_t *)gate_up,
                           (bf16_t *)out, rows, inter);
    else
        FLLM_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
    return fllm_check_launch("swiglu");
}

extern "C" int fllm_rope_kv_store(void *qkv, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                                  int table_stride, const float *cos_table, const float *sin_table, int table_positions,
                                  void *k_pages, void *v_pages, int num_pages, int rows, int heads, int kv_heads,
                                  int head_dim, int rope_dims, int pairing, int page_size, int dtype, int store_kv,
                                  hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && page_size > 0 && table_stride > 0,
                 "rope_kv_store: bad sizes");
    FLLM_REQUIRE(rope_dims >= 0 && rope_dims <= head_dim && rope_dims % 2 == 0,
                 "rope_kv_store: rope_dims %d must be even and at most head_dim %d", rope_dims, head_dim);
    FLLM_REQUIRE(pairing == 0 || pairing == 1, "rope_kv_store: unknown pairing %d", pairing);
    FLLM_REQUIRE(!store_kv || (k_pages && v_pages && num_pages > 0), "rope_kv_store: pages missing");
    (void)table_positions;
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(rope_kv_store_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, (float *)qkv, row_pos, row_seg,
                           tables, table_stride, cos_table, sin_table, (float *)k_pages, (float *)v_pages, heads, kv_heads,
                           head_dim, rope_dims, pairing, page_size, store_kv);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(rope_kv_store_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, (bf16_t *)qkv, row_pos,
                           row_seg, tables, table_stride, cos_table, sin_table, (bf16_t *)k_pages, (bf16_t *)v_pages, heads,
                           kv_heads, head_dim, rope_dims, pairing, page_size, store_kv);
    else
        FLLM_REQUIRE(false, "rope_kv_store: unknown dtype %d", dtype);
    return fllm_check_launch("rope_kv_store");
}
