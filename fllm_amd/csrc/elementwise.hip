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
// the elements of its groups of four, groups t, t + 256, ...; then lanes, then waves), so a row
// gives the same bits whatever else is in the batch.  With `branch` the kernel first adds it to
// the row (x += branch, in float32, written back): residual add and the next norm in one pass.
// Rows of up to 256 * 4 * VEC values stay in registers between the two uses.
template <typename T, typename B, int VEC>
__global__ void __launch_bounds__(kBlock)
rmsnorm_kernel(float *__restrict__ x, const B *__restrict__ branch, const int32_t *__restrict__ rows,
               const float *__restrict__ weight, T *__restrict__ out, int width, float eps) {
    __shared__ float scratch[kWaves];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    float *src = x + (size_t)r * width;
    const B *br = branch ? branch + (size_t)r * width : nullptr;
    T *dst = out + (size_t)i * width;
    if constexpr (VEC > 0) {   // width is a multiple of 4 and at most 1024 * VEC
        f32x4_t v[VEC > 0 ? VEC : 1];
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            const int c = (threadIdx.x + j * kBlock) * 4;
            if (c < width) {
                v[j] = *(const f32x4_t *)(src + c);
                if (br) {
#pragma unroll
                    for (int e = 0; e < 4; e++) v[j][e] += to_f32<B>(br[c + e]);
                    *(f32x4_t *)(src + c) = v[j];
                }
#pragma unroll
                for (int e = 0; e < 4; e++) ss += v[j][e] * v[j][e];
            }
        }
        ss = block_sum<kWaves>(ss, scratch);
        const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            const int c = (threadIdx.x + j * kBlock) * 4;
            if (c < width) {
                const f32x4_t w = *(const f32x4_t *)(weight + c);
#pragma unroll
                for (int e = 0; e < 4; e++) dst[c + e] = from_f32<T>(v[j][e] * (inv * w[e]));
            }
        }
    } else {
        float ss = 0.f;
        for (int c = threadIdx.x; c < width; c += kBlock) {
            float v = src[c];
            if (br) {
                v += to_f32<B>(br[c]);
                src[c] = v;
            }
            ss += v * v;
        }
        ss = block_sum<kWaves>(ss, scratch);   // its barriers also order the row's writes before the reads below
        const float inv = 1.0f / sqrtf(ss / (float)width + eps);
        for (int c = threadIdx.x; c < width; c += kBlock) dst[c] = from_f32<T>(src[c] * (inv * weight[c]));
    }
}

// What a product that adds into the residual stream leaves for the RMSNorm behind it (fllm_linear_add_normed), made
// from rows that no such product wrote (the first layer's): xn = x * weight in bfloat16 and the row's sum of squares as
// one part, added in the order of rmsnorm_kernel.
__global__ void __launch_bounds__(kBlock)
prepare_norm_kernel(const float *__restrict__ x, const float *__restrict__ weight, bf16_t *__restrict__ xn, float *__restrict__ ssq,
                    int width) {
    __shared__ float scratch[kWaves];
    const int r = blockIdx.x;
    const float *src = x + (size_t)r * width;
    bf16_t *dst = xn + (size_t)r * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += kBlock) {
        const float v = src[c];
        ss += v * v;
        dst[c] = (bf16_t)(v * weight[c]);
    }
    ss = block_sum<kWaves>(ss, scratch);
    if (threadIdx.x == 0) ssq[r] = ss;
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
swiglu_kernel(const T *__restrict__ gu, T *__restrict__ out, int inter) {
    const size_t r = blockIdx.y;
    const T *g = gu + r * 2 * inter, *u = g + inter;
    T *o = out + r * inter;
    constexpr int V = 16 / sizeof(T);   // values per 16-byte access
    typedef __attribute__((ext_vector_type(V))) T vec_t;
    const int c = (blockIdx.x * kBlock + threadIdx.x) * V;
    if (c + V <= inter && inter % V == 0) {
        const vec_t gv = *(const vec_t *)(g + c), uv = *(const vec_t *)(u + c);
        vec_t ov;
#pragma unroll
        for (int e = 0; e < V; e++) {
            const float gf = to_f32<T>(gv[e]);
            ov[e] = from_f32<T>(gf / (1.0f + expf(-gf)) * to_f32<T>(uv[e]));
        }
        *(vec_t *)(o + c) = ov;
    } else {
        for (int e = c; e < c + V && e < inter; e++) {
            const float gf = to_f32<T>(g[e]);
            o[e] = from_f32<T>(gf / (1.0f + expf(-gf)) * to_f32<T>(u[e]));
        }
    }
}

// residual[r, :] += branch[r, :], the sum in float32
template <typename T>
__global__ void __launch_bounds__(kBlock)
add_residual_kernel(float *__restrict__ residual, const T *__restrict__ branch, size_t total) {
    for (size_t i = ((size_t)blockIdx.x * kBlock + threadIdx.x) * 4; i < total; i += (size_t)gridDim.x * kBlock * 4) {
        if (i + 4 <= total) {
            f32x4_t r = *(const f32x4_t *)(residual + i);
#pragma unroll
            for (int j = 0; j < 4; j++) r[j] += to_f32<T>(branch[i + j]);
            *(f32x4_t *)(residual + i) = r;
        } else {
            for (size_t j = i; j < total; j++) residual[j] += to_f32<T>(branch[j]);
        }
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
        k_pages[key_offset(page, kv_heads, h, page_size, head_dim, off, ia)] = from_f32<T>(a * cs[l] - b * sn[l]);
        k_pages[key_offset(page, kv_heads, h, page_size, head_dim, off, ib)] = from_f32<T>(b * cs[l] + a * sn[l]);
    }
    const int rest = head_dim - rope_dims;
    for (int i = threadIdx.x; i < kv_heads * rest; i += kBlock) {
        const int h = i / rest, c = rope_dims + (i - h * rest);
        k_pages[key_offset(page, kv_heads, h, page_size, head_dim, off, c)] = krow[(size_t)h * head_dim + c];
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

namespace {

template <typename T, typename B>
void launch_rmsnorm(float *x, const B *branch, const int32_t *rows, const float *weight, T *out, int count, int width,
                    float eps, hipStream_t stream) {
    const bool vec = width % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)weight & 15) == 0;
#define FLLM_NORM(V) hipLaunchKernelGGL((rmsnorm_kernel<T, B, V>), dim3(count), dim3(kBlock), 0, stream, x, branch, rows, weight, out, width, eps)
    if (vec && width <= 1024) FLLM_NORM(1);
    else if (vec && width <= 2048) FLLM_NORM(2);
    else if (vec && width <= 4096) FLLM_NORM(4);
    else if (vec && width <= 8192) FLLM_NORM(8);
    else FLLM_NORM(0);
#undef FLLM_NORM
}

template <typename B>
int dispatch_rmsnorm(float *x, const B *branch, const int32_t *rows, const float *weight, void *out, int count, int width,
                     float eps, int out_dtype, hipStream_t stream) {
    if (out_dtype == FLLM_F32) launch_rmsnorm<float, B>(x, branch, rows, weight, (float *)out, count, width, eps, stream);
    else if (out_dtype == FLLM_BF16) launch_rmsnorm<bf16_t, B>(x, branch, rows, weight, (bf16_t *)out, count, width, eps, stream);
    else FLLM_REQUIRE(false, "rmsnorm: unknown dtype %d", out_dtype);
    return fllm_check_launch("rmsnorm");
}

}  // namespace

extern "C" int fllm_rmsnorm(const float *x, const int32_t *rows, const float *weight, void *out, int count, int width,
                            float eps, int out_dtype, hipStream_t stream) {
    FLLM_REQUIRE(count >= 0 && width > 0, "rmsnorm: bad sizes count=%d width=%d", count, width);
    FLLM_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive");
    if (count == 0) return 0;
    return dispatch_rmsnorm<float>(const_cast<float *>(x), nullptr, rows, weight, out, count, width, eps, out_dtype, stream);
}

extern "C" int fllm_add_rmsnorm(float *x, const void *branch, int branch_dtype, const float *weight, void *out, int count,
                                int width, float eps, int out_dtype, hipStream_t stream) {
    FLLM_REQUIRE(count >= 0 && width > 0, "add_rmsnorm: bad sizes count=%d width=%d", count, width);
    FLLM_REQUIRE(eps > 0.f && branch != nullptr, "add_rmsnorm: eps must be positive and the branch given");
    if (count == 0) return 0;
    if (branch_dtype == FLLM_F32)
        return dispatch_rmsnorm<float>(x, (const float *)branch, nullptr, weight, out, count, width, eps, out_dtype, stream);
    FLLM_REQUIRE(branch_dtype == FLLM_BF16, "add_rmsnorm: unknown dtype %d", branch_dtype);
    return dispatch_rmsnorm<bf16_t>(x, (const bf16_t *)branch, nullptr, weight, out, count, width, eps, out_dtype, stream);
}

extern "C" int fllm_prepare_norm(const float *x, const float *weight, void *xn, float *ssq, int rows, int width, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && x != nullptr && weight != nullptr && xn != nullptr && ssq != nullptr,
                 "prepare_norm: bad operands rows=%d width=%d", rows, width);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(prepare_norm_kernel, dim3(rows), dim3(kBlock), 0, stream, x, weight, (bf16_t *)xn, ssq, width);
    return fllm_check_launch("prepare_norm");
}

extern "C" int fllm_swiglu(const void *gate_up, void *out, int rows, int inter, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && inter > 0, "swiglu: bad sizes rows=%d inter=%d", rows, inter);
    if (rows == 0) return 0;
    FLLM_REQUIRE(rows <= 65535 * 32, "swiglu: too many rows");
    for (int r0 = 0; r0 < rows; r0 += 65535) {   // grid.y is limited to 65535
        const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
        if (dtype == FLLM_F32) {
            const dim3 grid((inter + kBlock * 4 - 1) / (kBlock * 4), nr);
            hipLaunchKernelGGL(swiglu_kernel<float>, grid, dim3(kBlock), 0, stream, (const float *)gate_up + (size_t)r0 * 2 * inter,
                               (float *)out + (size_t)r0 * inter, inter);
        } else if (dtype == FLLM_BF16) {
            const dim3 grid((inter + kBlock * 8 - 1) / (kBlock * 8), nr);
            hipLaunchKernelGGL(swiglu_kernel<bf16_t>, grid, dim3(kBlock), 0, stream,
                               (const bf16_t *)gate_up + (size_t)r0 * 2 * inter, (bf16_t *)out + (size_t)r0 * inter, inter);
        } else {
            FLLM_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
        }
    }
    return fllm_check_launch("swiglu");
}

extern "C" int fllm_add_residual(float *residual, const void *branch, int rows, int width, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0, "add_residual: bad sizes rows=%d width=%d", rows, width);
    FLLM_REQUIRE(((uintptr_t)residual & 15) == 0, "add_residual: the residual must be 16-byte aligned");
    if (rows == 0) return 0;
    const size_t total = (size_t)rows * width;
    const size_t groups = (total + 4 * kBlock - 1) / (4 * kBlock);
    const int grid = (int)(groups < 16384 ? groups : 16384);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(add_residual_kernel<float>, dim3(grid), dim3(kBlock), 0, stream, residual, (const float *)branch, total);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(add_residual_kernel<bf16_t>, dim3(grid), dim3(kBlock), 0, stream, residual, (const bf16_t *)branch,
                           total);
    else
        FLLM_REQUIRE(false, "add_residual: unknown dtype %d", dtype);
    return fllm_check_launch("add_residual");
}

// bfloat16 rows, pairs (2l, 2l+1), head_dim and rope_dims in steps of 8: every thread takes 8 neighbouring lanes of
// a head (16-byte loads and stores; cosines and sines as two 16-byte loads each).  Prompt portions: four workgroups
// share 8 rows (a read and a write of the same buffer cannot overlap inside a thread, so many short threads beat few
// long ones); where the rows are 8 consecutive tokens of one request that start at a multiple of 8 (a prompt portion), their values go
// into the transposed page as one 16-byte store per head lane instead of eight 2-byte ones.
template <int RB>
__global__ void __launch_bounds__(kBlock)
rope_kv_store_vec_kernel(bf16_t *__restrict__ qkv, const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seg,
                         const int32_t *__restrict__ tables, int table_stride, const float *__restrict__ cos_table,
                         const float *__restrict__ sin_table, bf16_t *__restrict__ k_pages, bf16_t *__restrict__ v_pages,
                         int rows, int heads, int kv_heads, int head_dim, int rope_dims, int page_size, int store_kv) {
    const int r0 = blockIdx.x * RB;
    const int nrows = min(RB, rows - r0);
    const int half = rope_dims / 2;
    const int per_head = head_dim / 8;
    const int rot_heads = store_kv ? heads + kv_heads : heads;
    const size_t row_elems = (size_t)(heads + 2 * kv_heads) * head_dim;
    // position (-1: padding row), page and slot of the workgroup's rows
    __shared__ int s_pos[RB], s_page[RB], s_off[RB], s_run;
    if ((int)threadIdx.x < nrows) {
        const int r = r0 + threadIdx.x;
        const int seg = row_seg[r], pos = row_pos[r];
        s_pos[threadIdx.x] = seg < 0 ? -1 : pos;
        s_page[threadIdx.x] = (store_kv && seg >= 0) ? tables[(size_t)seg * table_stride + pos / page_size] : 0;
        s_off[threadIdx.x] = pos % page_size;
    }
    if (threadIdx.x == 0) {
        const int seg0 = row_seg[r0], pos0 = row_pos[r0];
        bool run = RB == 8 && store_kv && nrows == RB && seg0 >= 0 && (pos0 & (RB - 1)) == 0 && page_size % RB == 0;
        for (int i = 1; i < RB && run; i++) run = row_seg[r0 + i] == seg0 && row_pos[r0 + i] == pos0 + i;
        s_run = run;
    }
    __syncthreads();
    const bool run = s_run != 0;

    // queries and keys: every (row, 16-byte chunk) is a piece of work of its own, so that a thread has several in flight
    const int per_row = rot_heads * per_head;
    const int first = blockIdx.y * kBlock + threadIdx.x, stride = gridDim.y * kBlock;   // the workgroups of a row group share its pieces
    for (int it = first; it < nrows * per_row; it += stride) {
        const int i = RB == 1 ? 0 : it / per_row, t = it - i * per_row;
        const int pos = s_pos[i];
        if (pos < 0) continue;   // padding row
        const int h = t / per_head, c = (t - h * per_head) * 8;
        bf16_t *row = qkv + (size_t)(r0 + i) * row_elems;
        bf16x8_t v = *(const bf16x8_t *)(row + (size_t)h * head_dim + c);
        if (c < rope_dims) {   // rope_dims is a multiple of 8: the chunk is rotated as a whole
            const f32x4_t c4 = *(const f32x4_t *)(cos_table + (size_t)pos * half + c / 2);
            const f32x4_t s4 = *(const f32x4_t *)(sin_table + (size_t)pos * half + c / 2);
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const float a = (float)v[2 * p], b = (float)v[2 * p + 1];
                v[2 * p] = (bf16_t)(a * c4[p] - b * s4[p]);
                v[2 * p + 1] = (bf16_t)(b * c4[p] + a * s4[p]);
            }
        }
        if (h < heads) *(bf16x8_t *)(row + (size_t)h * head_dim + c) = v;
        else *(bf16x8_t *)(k_pages + key_offset(s_page[i], kv_heads, h - heads, page_size, head_dim, s_off[i], c)) = v;
    }
    if (!store_kv) return;
    if (!run) {
        // values, stored transposed inside the page: [head_dim][token]
        const int v_per_row = kv_heads * per_head;
        for (int it = first; it < nrows * v_per_row; it += stride) {
            const int i = RB == 1 ? 0 : it / v_per_row, t = it - i * v_per_row;
            if (s_pos[i] < 0) continue;
            const int h = t / per_head, c = (t - h * per_head) * 8;
            const bf16x8_t v = *(const bf16x8_t *)(qkv + (size_t)(r0 + i) * row_elems + (size_t)(heads + kv_heads + h) * head_dim + c);
            bf16_t *dst = v_pages + (((size_t)s_page[i] * kv_heads + h) * head_dim + c) * page_size + s_off[i];
#pragma unroll
            for (int e = 0; e < 8; e++) dst[(size_t)e * page_size] = v[e];
        }
        return;
    }
    // the values of the 8 tokens, one head lane at a time: 16 contiguous bytes of the transposed page
    const int page = s_page[0], off = s_off[0];
    const bf16_t *vbase = qkv + (size_t)r0 * row_elems + (size_t)(heads + kv_heads) * head_dim;
    for (int t = first; t < kv_heads * head_dim; t += stride) {
        const int h = t / head_dim, c = t - h * head_dim;
        bf16x8_t v;
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = vbase[(size_t)(RB == 8 ? i : 0) * row_elems + t];
        *(bf16x8_t *)(v_pages + (((size_t)page * kv_heads + h) * head_dim + c) * page_size + off) = v;
    }
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
    FLLM_REQUIRE(head_dim % 8 == 0, "rope_kv_store: head size %d; keys lie in chunks of 8 values in a page, head sizes come in steps of 8", head_dim);
    (void)table_positions;
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(rope_kv_store_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, (float *)qkv, row_pos, row_seg,
                           tables, table_stride, cos_table, sin_table, (float *)k_pages, (float *)v_pages, heads, kv_heads,
                           head_dim, rope_dims, pairing, page_size, store_kv);
    else if (dtype == FLLM_BF16 && pairing == 1 && head_dim % 8 == 0 && rope_dims % 8 == 0 && ((uintptr_t)qkv & 15) == 0 &&
             ((uintptr_t)cos_table & 15) == 0 && ((uintptr_t)sin_table & 15) == 0 && (!store_kv || ((((uintptr_t)k_pages | (uintptr_t)v_pages) & 15) == 0)))
    {
        // prompt portions: 8 rows a workgroup, so that runs of 8 tokens store their values 16 bytes at a time; few rows
        // (decode steps): a workgroup a row
        if (rows >= 256)
            hipLaunchKernelGGL(rope_kv_store_vec_kernel<8>, dim3((rows + 7) / 8, 4), dim3(kBlock), 0, stream, (bf16_t *)qkv, row_pos,
                               row_seg, tables, table_stride, cos_table, sin_table, (bf16_t *)k_pages, (bf16_t *)v_pages, rows,
                               heads, kv_heads, head_dim, rope_dims, page_size, store_kv);
        else
            hipLaunchKernelGGL(rope_kv_store_vec_kernel<1>, dim3(rows), dim3(kBlock), 0, stream, (bf16_t *)qkv, row_pos, row_seg,
                               tables, table_stride, cos_table, sin_table, (bf16_t *)k_pages, (bf16_t *)v_pages, rows, heads,
                               kv_heads, head_dim, rope_dims, page_size, store_kv);
    }
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(rope_kv_store_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, (bf16_t *)qkv, row_pos,
                           row_seg, tables, table_stride, cos_table, sin_table, (bf16_t *)k_pages, (bf16_t *)v_pages, heads,
                           kv_heads, head_dim, rope_dims, pairing, page_size, store_kv);
    else
        FLLM_REQUIRE(false, "rope_kv_store: unknown dtype %d", dtype);
    return fllm_check_launch("rope_kv_store");
}

namespace {
__global__ void carry_ids_kernel(int32_t *__restrict__ ids, const int32_t *__restrict__ source, const int32_t *__restrict__ previous,
                                 int rows) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r < rows && source[r] >= 0) ids[r] = previous[source[r]];
}
}  // namespace

extern "C" int fllm_carry_ids(int32_t *ids, const int32_t *source, const int32_t *previous, int rows, int previous_rows,
                              hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && previous_rows >= 0, "carry_ids: bad sizes");
    (void)previous_rows;      // the host has checked every source against it
    if (rows == 0) return 0;
    hipLaunchKernelGGL(carry_ids_kernel, dim3((rows + 255) / 256), dim3(256), 0, stream, ids, source, previous, rows);
    return fllm_check_launch("carry_ids");
}
