// Paged causal attention, plain form: one workgroup per (row, head), float32 arithmetic, online
// softmax over chunks of 256 keys.  Used by the true 32-bit path and by the bfloat16 path for
// shapes the MFMA kernels refuse.  A row's result depends only on its own position, window and
// pages, never on the rest of the batch.
#include "api.h"
#include "common.h"

int fllm_attention_bf16_fast(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                             int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                             int num_segs, void *out, int rows, int heads, int kv_heads, int head_dim, int page_size,
                             int num_pages, float scale, int window, int max_context, int single_from, void *workspace,
                             size_t workspace_bytes, hipStream_t stream);   // attention_mfma.hip; 1: shape declined
size_t fllm_attention_bf16_workspace_bytes(int rows, int heads, int kv_heads, int head_dim, int max_context);

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;
constexpr int kMaxDimPerThread = 2;   // head_dim <= 512

template <typename T>
__global__ void __launch_bounds__(kBlock)
attention_generic_kernel(const T *__restrict__ q, int q_stride, const T *__restrict__ k_pages,
                         const T *__restrict__ v_pages, const int32_t *__restrict__ tables, int table_stride,
                         const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seg, T *__restrict__ out,
                         int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                         const float *__restrict__ head_slopes) {
    extern __shared__ float smem[];
    float *qs = smem;                   // head_dim
    float *sc = smem + head_dim;        // kBlock
    float *scratch = sc + kBlock;       // kWaves
    const int r = blockIdx.x, h = blockIdx.y;
    const int seg = row_seg[r];
    T *dst = out + ((size_t)r * heads + h) * head_dim;
    if (seg < 0) {   // padding row
        for (int c = threadIdx.x; c < head_dim; c += kBlock) dst[c] = from_f32<T>(0.f);
        return;
    }
    const int pos = row_pos[r];
    const int n = pos + 1;
    const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
    const int kvh = h / (heads / kv_heads);
    const int32_t *tbl = tables + (size_t)seg * table_stride;
    const T *qrow = q + (size_t)r * q_stride + (size_t)h * head_dim;
    for (int c = threadIdx.x; c < head_dim; c += kBlock) qs[c] = to_f32<T>(qrow[c]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[kMaxDimPerThread] = {0.f, 0.f};
    for (int c0 = lo; c0 < n; c0 += kBlock) {
        const int key = c0 + threadIdx.x;
        float s = -INFINITY;
        if (key < n) {
            const int page = tbl[key / page_size], off = key % page_size;
            const T *kr = k_pages + key_offset(page, kv_heads, kvh, page_size, head_dim, off, 0);     // chunk c / 8 lies c / 8 * page_size * 8 on
            float dot = 0.f;
            for (int c = 0; c < head_dim; c++) dot = fmaf(qs[c], to_f32<T>(kr[(size_t)(c >> 3) * page_size * 8 + (c & 7)]), dot);
            s = dot * scale;
            if (head_slopes != nullptr) s = fmaf(head_slopes[h], (float)(key - pos), s);   // a bias by distance (<= 0 keys back)
        }
        const float m_new = fmaxf(m, block_max<kWaves>(s, scratch));
        const float alpha = expf(m - m_new);   // first chunk: exp(-inf) = 0
        const float p = key < n ? expf(s - m_new) : 0.f;
        sc[threadIdx.x] = p;
        l = l * alpha + block_sum<kWaves>(p, scratch);   // the barriers inside also publish sc[]
        const int count = n - c0 < kBlock ? n - c0 : kBlock;
#pragma unroll
        for (int t = 0; t < kMaxDimPerThread; t++) {
            const int c = threadIdx.x + t * kBlock;
            if (c >= head_dim) break;
            float a = acc[t] * alpha;
            for (int j = 0; j < count; j++) {
                const int kj = c0 + j;
                const int page = tbl[kj / page_size], off = kj % page_size;
                a = fmaf(sc[j], to_f32<T>(v_pages[(((size_t)page * kv_heads + kvh) * head_dim + c) * page_size + off]), a);
            }
            acc[t] = a;
        }
        m = m_new;
        __syncthreads();   // sc[] is rewritten by the next chunk
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int t = 0; t < kMaxDimPerThread; t++) {
        const int c = threadIdx.x + t * kBlock;
        if (c < head_dim) dst[c] = from_f32<T>(acc[t] * inv);
    }
}

}  // namespace

extern "C" size_t fllm_attention_workspace_bytes(int rows, int heads, int kv_heads, int head_dim, int max_context) {
    return fllm_attention_bf16_workspace_bytes(rows, heads, kv_heads, head_dim, max_context);
}

namespace {
int attention_any(const void *q, int q_stride, const void *k_pages, const void *v_pages,
                  const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                  const int32_t *seg_start, int num_segs, void *out, int rows, int heads, int kv_heads,
                  int head_dim, int page_size, int num_pages, float scale, int window, int dtype,
                  int max_context, int single_from, void *workspace, size_t workspace_bytes, const float *head_slopes,
                  hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && page_size > 0 && table_stride > 0 && num_pages > 0,
                 "attention: bad sizes");
    FLLM_REQUIRE(heads % kv_heads == 0, "attention: %d heads are not a multiple of %d key/value heads", heads, kv_heads);
    FLLM_REQUIRE(head_dim % 8 == 0, "attention: head size %d; keys lie in chunks of 8 values in a page, head sizes come in steps of 8", head_dim);
    FLLM_REQUIRE(num_segs > 0 && seg_start != nullptr, "attention: segment starts are required");
    FLLM_REQUIRE(single_from >= 0 && single_from <= num_segs, "attention: single_from %d is outside 0..%d", single_from, num_segs);
    FLLM_REQUIRE(q_stride >= heads * head_dim, "attention: q_stride %d is shorter than heads*head_dim", q_stride);
    if (rows == 0) return 0;
    if (dtype == FLLM_BF16 && head_slopes == nullptr) {     // the MFMA kernels know no bias: biased scores take the plain kernel
        const int fast = fllm_attention_bf16_fast(q, q_stride, k_pages, v_pages, tables, table_stride, row_pos, row_seg,
                                                  seg_start, num_segs, out, rows, heads, kv_heads, head_dim, page_size,
                                                  num_pages, scale, window, max_context, single_from, workspace,
                                                  workspace_bytes, stream);
        if (fast <= 0) return fast;
    }
    FLLM_REQUIRE(head_dim <= kBlock * kMaxDimPerThread, "attention: head_dim %d is larger than %d", head_dim,
                 kBlock * kMaxDimPerThread);
    FLLM_REQUIRE(heads <= 65535, "attention: too many heads");
    const size_t smem = (size_t)(head_dim + kBlock + kWaves) * sizeof(float);
    const dim3 grid(rows, heads);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(attention_generic_kernel<float>, grid, dim3(kBlock), smem, stream, (const float *)q, q_stride,
                           (const float *)k_pages, (const float *)v_pages, tables, table_stride, row_pos, row_seg,
                           (float *)out, heads, kv_heads, head_dim, page_size, scale, window, head_slopes);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(attention_generic_kernel<bf16_t>, grid, dim3(kBlock), smem, stream, (const bf16_t *)q, q_stride,
                           (const bf16_t *)k_pages, (const bf16_t *)v_pages, tables, table_stride, row_pos, row_seg,
                           (bf16_t *)out, heads, kv_heads, head_dim, page_size, scale, window, head_slopes);
    else
        FLLM_REQUIRE(false, "attention: unknown dtype %d", dtype);
    return fllm_check_launch("attention");
}
}  // namespace

extern "C" int fllm_attention(const void *q, int q_stride, const void *k_pages, const void *v_pages,
                              const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                              const int32_t *seg_start, int num_segs, void *out, int rows, int heads, int kv_heads,
                              int head_dim, int page_size, int num_pages, float scale, int window, int dtype,
                              int max_context, int single_from, void *workspace, size_t workspace_bytes,
                              hipStream_t stream) {
    return attention_any(q, q_stride, k_pages, v_pages, tables, table_stride, row_pos, row_seg, seg_start, num_segs, out, rows,
                         heads, kv_heads, head_dim, page_size, num_pages, scale, window, dtype, max_context, single_from,
                         workspace, workspace_bytes, nullptr, stream);
}

extern "C" int fllm_attention_sloped(const void *q, int q_stride, const void *k_pages, const void *v_pages,
                                     const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                                     const int32_t *seg_start, int num_segs, void *out, int rows, int heads, int kv_heads,
                                     int head_dim, int page_size, int num_pages, float scale, int window, int dtype,
                                     int max_context, const float *head_slopes, hipStream_t stream) {
    FLLM_REQUIRE(head_slopes != nullptr, "attention_sloped: a slope per head is required");
    return attention_any(q, q_stride, k_pages, v_pages, tables, table_stride, row_pos, row_seg, seg_start, num_segs, out, rows,
                         heads, kv_heads, head_dim, page_size, num_pages, scale, window, dtype, max_context, num_segs,
                         nullptr, 0, head_slopes, stream);
}
