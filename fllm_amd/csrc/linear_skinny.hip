// Decode-step matrix products (M <= 64 rows) in bfloat16: y = f(x) w^T with the weight matrix
// streamed exactly once from HBM, and the work around the product folded into the same kernel:
//
//   prologue  BF16      x is bfloat16 [M, K]
//             NORM_F32  x is the float32 residual stream; the operand is x * norm_weight and the row's
//                       rsqrt(mean(x^2) + eps) is applied to the sums afterwards (a row scale commutes
//                       with the product), so RMSNorm costs no pass of its own
//             SCALED    the same norm, prepared by the product before: x * norm_weight arrives as bfloat16
//                       rows, and every row's sum of squares in parts (one a tile of that product's
//                       outputs), which are added in order.  Half the bytes of NORM_F32 and no conversion
//                       (up to 16 rows)
//   epilogue  STORE / STORE_F32 / ADD (add to the float32 residual stream; on request it also leaves what
//                       the SCALED prologue of the next product takes: the new rows times the next norm's
//                       weight in bfloat16, and each tile's share of the rows' sums of squares)
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
#include "plans.h"

namespace {

// 16 bytes of zeros in device memory: what a lane loads when it has nothing of its own to load, so that every lane
// issues every load and no load sits behind a branch.
__device__ uint4 kZeros = {0u, 0u, 0u, 0u};     // not const: in the same address space as the tensors it stands in for

// Partial sums that workgroups hand to each other go through the device workspace in 16-byte pieces that pass by the
// caches of the compute units and of their die on both ways (the sc0 sc1 forms of the buffer instructions: written
// through to memory, read from memory), as device-scope atomics do for single words.  The workspace is one buffer
// for these instructions; offsets are in bytes from its base.
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
constexpr int kThroughCaches = 17;        // cache policy bits sc0 (1) and sc1 (16)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t workspace_buffer(float *base) {
    return __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7fffffff, 0x00020000);      // raw buffer, offsets up to 2 GiB
}
__device__ __forceinline__ void hand_over(__amdgpu_buffer_rsrc_t ws, unsigned int byte_offset, f32x4_t v) {
    u32x4_t bits = {__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])};
    __builtin_amdgcn_raw_buffer_store_b128(bits, ws, byte_offset, 0, kThroughCaches);
}
__device__ __forceinline__ f32x4_t take_over(__amdgpu_buffer_rsrc_t ws, unsigned int byte_offset) {
    const u32x4_t bits = __builtin_amdgcn_raw_buffer_load_b128(ws, byte_offset, 0, kThroughCaches);
    return (f32x4_t){__uint_as_float(bits[0]), __uint_as_float(bits[1]), __uint_as_float(bits[2]), __uint_as_float(bits[3])};
}

constexpr int kWideRows = 128;            // the most rows of the kernel that passes the activations through LDS in chunks
enum { PRO_BF16 = 0, PRO_NORM_F32 = 1, PRO_SCALED = 2 };
enum { EPI_STORE = 0, EPI_STORE_F32 = 1, EPI_ADD = 2, EPI_QKV = 3, EPI_SWIGLU = 4 };

struct SkinnyArgs {
    const void *x;
    int ldx;
    const float *norm_w;
    float eps;
    const bf16_t *w;
    const bf16_t *w_tiles;   // the same matrix tile by tile (fllm_tile_weights), or null
    const float *bias;
    void *out;
    int ldo;
    int M, N, K;
    int S, slice;  // K is cut into S slices of `slice` elements (a multiple of 128); a workgroup stages one slice
    int ssq_off;   // byte offset of the sums of squares in LDS (behind the staging / reduction area)
    float *ws;     // S > 1: partial sums [tile][slice][RT][64 lanes][4], then sums of squares [tile][slice][16]
    float *ws_ssq;
    int *counters; // S > 1: items of a tile counted so far (zero between launches)
    // QKV epilogue
    const int32_t *row_pos, *row_seg, *tables;
    int table_stride;
    const float *cos_t, *sin_t;
    int rope_dims;
    bf16_t *k_pages, *v_pages;
    int heads, kv_heads, head_dim, page_size, store_kv;
    // ADD epilogue, on request (next_x != null): for the norm that reads the sums next
    const float *next_w;   // [N] that norm's weight
    bf16_t *next_x;        // [M, N] (out + sum) * next_w
    float *next_ssq;       // [M, next_tiles] sum of squares of (out + sum) over a tile's outputs
    int next_nt, next_tiles;   // outputs a tile (16 or 8) and tiles a row: set by the launch
    int *next_tiles_out;   // host memory: where the launch leaves next_tiles for the caller
    // SCALED prologue
    const float *ssq_in;   // [M, ssq_count]
    int ssq_count;
#ifdef FLLM_TIMELINE
    unsigned long long *timeline;   // measurement builds only: [workgroup][8] times of the 100 MHz clock
#endif
};

#ifdef FLLM_TIMELINE
#define FLLM_STAMP(a, k)                                                                                   \
    do {                                                                                                   \
        if ((a).timeline != nullptr && threadIdx.x == 0) (a).timeline[blockIdx.x * 8 + (k)] = __builtin_amdgcn_s_memrealtime(); \
    } while (0)
#else
#define FLLM_STAMP(a, k) \
    do {                 \
    } while (0)
#endif

__device__ __forceinline__ bf16x4_t pack4(f32x4_t v) {
    bf16x4_t p;
#pragma unroll
    for (int i = 0; i < 4; i++) p[i] = (bf16_t)v[i];
    return p;
}

__device__ __forceinline__ bf16x8_t zero8() {
    bf16x8_t z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16_t)0.0f;
    return z;
}

// The sums of one output group (row m, columns nb .. nb + 3) over the waves of a workgroup, in wave order.
template <int WAVES, int RT>
__device__ __forceinline__ void sum_waves(const f32x4_t *red, int stride_t, int idx, f32x4_t (&s)[RT]) {
#pragma unroll
    for (int t = 0; t < RT; t++) {
        s[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int wv = 0; wv < WAVES; wv++) s[t] += red[(wv * RT + t) * stride_t + idx];
    }
}

// What an epilogue reads from global memory besides the sums.  The resident kernel asks for it while the
// products of the item are still running, so that the end of an item waits for no load.
struct EpilogueOperands {
    bool have = false;     // resid / cs / sn hold this item's values
    f32x4_t resid;         // EPI_ADD: out[m, nb .. nb + 3]
    f32x4_t next_w;        // EPI_ADD that prepares the next norm: that norm's weight at nb .. nb + 3
    float cs[2], sn[2];    // EPI_QKV: cosine and sine of the two pairs at nb, nb + 2
    int seg = -1, pos = 0, page = 0;   // EPI_QKV: the row's segment, position and page (do not depend on the item)
};

template <int EPI>
__device__ __forceinline__ void load_row_operands(const SkinnyArgs &a, int m, EpilogueOperands &e) {
    if (EPI != EPI_QKV || m >= a.M) return;
    e.seg = a.row_seg[m];
    e.pos = a.row_pos[m];
    if (e.seg >= 0 && a.store_kv) e.page = a.tables[(size_t)e.seg * a.table_stride + e.pos / a.page_size];
}

template <int EPI>
__device__ __forceinline__ void load_item_operands(const SkinnyArgs &a, int m, int nb, int n_out, EpilogueOperands &e) {
    e.have = false;
    if (m >= a.M || nb >= n_out) return;
    if (EPI == EPI_ADD) {
        if (nb + 3 < n_out && (a.ldo & 3) == 0 && ((uintptr_t)a.out & 15) == 0) {
            e.resid = *(const f32x4_t *)((const float *)a.out + (size_t)m * a.ldo + nb);
            if (a.next_x != nullptr) e.next_w = *(const f32x4_t *)(a.next_w + nb);
            e.have = true;
        }
    } else if (EPI == EPI_QKV) {
        const int d = a.head_dim;
        const int hd = nb / d, j = nb - hd * d;
        if (e.seg >= 0 && hd < a.heads + a.kv_heads && j + 3 < a.rope_dims) {
            const float *cs = a.cos_t + (size_t)e.pos * (a.rope_dims / 2) + j / 2, *sn = a.sin_t + (size_t)e.pos * (a.rope_dims / 2) + j / 2;
            e.cs[0] = cs[0], e.cs[1] = cs[1], e.sn[0] = sn[0], e.sn[1] = sn[1];
            e.have = true;
        }
    }
}

// What happens to the finished sums of one output group: row scale of the norm, bias, then the store.
// ss: the row's sum of squares (norm prologue).
template <int PRO, int EPI, int RT>
__device__ __forceinline__ void epilogue(const SkinnyArgs &a, f32x4_t (&s)[RT], float ss, int m, int nb, int n_out,
                                         const EpilogueOperands &e) {
    const int N = a.N, K = a.K;
    if (PRO != PRO_BF16) {
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
    // the four outputs of a lane are neighbours in a row: one store where the row's pitch and the base keep them aligned
    const bool whole = nb + 3 < n_out && (a.ldo & 3) == 0;
    if (EPI == EPI_ADD && (e.have || (whole && ((uintptr_t)a.out & 15) == 0))) {
        f32x4_t *dst = (f32x4_t *)((float *)a.out + (size_t)m * a.ldo + nb);
        const f32x4_t sum = (e.have ? e.resid : *dst) + s[0];
        *dst = sum;
        if (a.next_x != nullptr) {
            // For the norm that reads these rows next: its operand, and this tile's share of the row's sum of squares.
            // The lanes that hold a row's outputs of this tile sit 16 (and 32) lanes apart and are all here.
            const f32x4_t w = e.have ? e.next_w : *(const f32x4_t *)(a.next_w + nb);
            *(bf16x4_t *)(a.next_x + (size_t)m * a.N + nb) = pack4(sum * w);
            float sq = sum[0] * sum[0] + sum[1] * sum[1] + sum[2] * sum[2] + sum[3] * sum[3];
            sq += __shfl_xor(sq, 16, kWave);
            if (a.next_nt == 16) sq += __shfl_xor(sq, 32, kWave);
            if ((threadIdx.x & (kWave - 1)) < 16) a.next_ssq[(size_t)m * a.next_tiles + nb / a.next_nt] = sq;
        }
    } else if (EPI == EPI_STORE && whole && ((uintptr_t)a.out & 7) == 0) {
        *(bf16x4_t *)((bf16_t *)a.out + (size_t)m * a.ldo + nb) = pack4(s[0]);
    } else if (EPI == EPI_STORE_F32 && whole && ((uintptr_t)a.out & 15) == 0) {
        *(f32x4_t *)((float *)a.out + (size_t)m * a.ldo + nb) = s[0];
    } else if (EPI == EPI_STORE || EPI == EPI_STORE_F32 || EPI == EPI_ADD) {
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
        f32x4_t act;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float gt = s[0][i], up = s[RT - 1][i];
            act[i] = gt / (1.0f + expf(-gt)) * up;
        }
        if (whole && ((uintptr_t)a.out & 7) == 0) {
            *(bf16x4_t *)((bf16_t *)a.out + (size_t)m * a.ldo + nb) = pack4(act);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (nb + i < n_out) ((bf16_t *)a.out)[(size_t)m * a.ldo + nb + i] = (bf16_t)act[i];
        }
    } else {   // EPI_QKV: N = (heads + 2 kv_heads) * head_dim, head_dim a multiple of 4, so nb..nb+3 lie in one head
        const int seg = e.seg;
        if (seg < 0) return;
        const int pos = e.pos;
        const int d = a.head_dim;
        const int hd = nb / d, j = nb - hd * d;          // head (q heads, then k heads, then v heads), lane in head
        float v[4] = {s[0][0], s[0][1], s[0][2], s[0][3]};
        if (hd < a.heads + a.kv_heads && j < a.rope_dims) {   // rope_dims is even; j is a multiple of 4
            const float *cs = a.cos_t + (size_t)pos * (a.rope_dims / 2), *sn = a.sin_t + (size_t)pos * (a.rope_dims / 2);
#pragma unroll
            for (int p = 0; p < 2; p++) {
                if (j + 2 * p < a.rope_dims) {
                    const int l2 = (j + 2 * p) / 2;
                    const float c = e.have ? e.cs[p] : cs[l2], sv = e.have ? e.sn[p] : sn[l2];
                    const float x0 = v[2 * p], x1 = v[2 * p + 1];
                    v[2 * p] = x0 * c - x1 * sv;
                    v[2 * p + 1] = x1 * c + x0 * sv;
                }
            }
        }
        const f32x4_t v4 = {v[0], v[1], v[2], v[3]};
        if (hd < a.heads) {
            bf16_t *q = (bf16_t *)a.out + (size_t)m * a.ldo + nb;
            if ((a.ldo & 3) == 0 && ((uintptr_t)a.out & 7) == 0) {
                *(bf16x4_t *)q = pack4(v4);
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++) q[i] = (bf16_t)v[i];
            }
        } else if (a.store_kv) {
            const int page = e.page;
            const int off = pos % a.page_size;
            if (hd < a.heads + a.kv_heads) {
                const int kvh = hd - a.heads;
                bf16_t *kd = a.k_pages + key_offset(page, a.kv_heads, kvh, a.page_size, d, off, j);      // j .. j + 3 lie in one chunk of 8
                if (((uintptr_t)a.k_pages & 7) == 0) {      // head_dim and j are multiples of 4
                    *(bf16x4_t *)kd = pack4(v4);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) kd[i] = (bf16_t)v[i];
                }
            } else {
                const int kvh = hd - a.heads - a.kv_heads;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    a.v_pages[(((size_t)page * a.kv_heads + kvh) * d + j + i) * a.page_size + off] = (bf16_t)v[i];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// up to 16 rows: activations stay in LDS, workgroups walk over the weight row tiles
// ---------------------------------------------------------------------------------------------
// The product is cut into items (weight row tile, K slice).  Workgroup b of the grid owns slice
// b % S and the tiles b / S, b / S + G / S, ...  Its 8 waves split the slice into contiguous ranges;
// every wave stages the activations of its own range in LDS (for the norm prologue: x * norm_weight
// as bfloat16, and its part of every row's sum of squares) and needs nobody else's, so no wave waits
// for another before the end of an item.  The weights go from global memory straight into MFMA A
// operands, two blocks of loads (8 KiB a wave) in flight ahead of the products, across tile borders.
//
// What the 16 A rows of a product are (TM):
//   TM_ROWS16  16 weight rows, one K range                                   (16 outputs a row)
//   TM_DUALK   up to 8 activation rows: 8 weight rows, each with two K ranges (the halves of the wave's
//              range): A row r and B column r take K half r / 8, so D[r][c] is a partial sum where
//              r / 8 == c / 8, and the two are added at the end               (8 outputs a row)
//   TM_GATEUP  8 gate rows and the 8 up rows that belong to them              (8 outputs a row)
// The smaller tiles are what fills the chip evenly: 16-row tiles of the model's projections come to
// 1.5 or 3.5 a compute-unit slot.
//
// At the end of an item the waves' sums meet in LDS; one wave (they take turns) adds them in wave
// order.  With S = 1 it runs the epilogue.  With S > 1 (only when the activations of all of K do not
// fit into LDS) it leaves the item's sums in the workspace and counts the item; the workgroup that
// counts a tile's last item adds the S partial sums in slice order and runs the epilogue, so the
// result does not depend on which workgroup came last.
enum { TM_ROWS16 = 0, TM_DUALK = 1, TM_GATEUP = 2 };

// A load of weights.  Every weight is read once a step, so the loads from the tile-major copies carry the
// non-temporal hint: the lines do not push the activations, which every workgroup reads again, out of the caches, and a
// kernel that only reads gets 7.1 instead of 6.3 TB/s with it.  Only where a load instruction takes whole 128-byte
// lines, though: from the matrix as the checkpoint has it an instruction takes half a line of each of 16 rows and the
// next one the other half, and with the hint the second asks memory again (4,096 x 28,672 at one row: 41.0 us plain,
// 43.0 with the hint, 38.0 with hint and copy; the vocabulary projection 176.8 us plain, 187.8 with the hint).
template <bool STREAMED>
__device__ __forceinline__ bf16x8_t load_weights(const bf16_t *p) {
#ifdef FLLM_WEIGHTS_TEMPORAL
    return *(const bf16x8_t *)p;
#else
    if (STREAMED) return __builtin_nontemporal_load((const bf16x8_t *)p);
    return *(const bf16x8_t *)p;
#endif
}

template <int PRO, int EPI, int TM, int WAVES, bool XD, bool WT = false>
__global__ void __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(4, 4)))   // 16 waves a CU: 128 registers
skinny_resident_kernel(SkinnyArgs a, int red_off) {
    static_assert(!XD || PRO == PRO_BF16, "activations straight from global memory: the bfloat16 prologue only");
    static_assert(!WT || TM != TM_DUALK, "tile-major weights: whole 16-row tiles (or 8 gate and 8 up rows), one slice");
    constexpr int U = 4;                           // k-steps of 32 per block: four 16-byte loads per lane
    constexpr int KB = 32 * U;                     // K elements of one range per block
    constexpr int RB = 4;                          // rows of activations staged at a time (more would spill registers)
    constexpr int NT = TM == TM_ROWS16 ? 16 : 8;   // outputs per row and tile
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    static_assert((EPI == EPI_SWIGLU) == (TM == TM_GATEUP), "gate/up tiles belong to the SwiGLU epilogue");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N, K = a.K, S = a.S;
    FLLM_STAMP(a, 0);
    const int n_out = EPI == EPI_SWIGLU ? N / 2 : N;
    const int ntiles = (n_out + NT - 1) / NT;
    const int pitch = a.slice + 8;
    bf16_t *xs = (bf16_t *)smem;                                  // [M][pitch]
    f32x4_t *red = (f32x4_t *)(smem + red_off);                   // [WAVES][64]
    float *ssq_part = (float *)(smem + a.ssq_off);                // [WAVES][16]

    const int sl = blockIdx.x % S;
    const int tile0 = blockIdx.x / S, tstride = gridDim.x / S;
    const int ks0 = sl * a.slice;
    const int kcn = min(K, ks0 + a.slice) - ks0;                  // a multiple of 8
    const int my_items = tile0 < ntiles ? (ntiles - tile0 + tstride - 1) / tstride : 0;
    // the wave's contiguous part of the slice (relative to ks0), in steps of 64, and its blocks (the same number for every wave)
    const int kwlen = ((kcn + WAVES - 1) / WAVES + 63) / 64 * 64;
    const int kw0 = min(kcn, wave * kwlen), kw1 = min(kcn, kw0 + kwlen);
    const int half = TM == TM_DUALK ? kwlen / 2 : kwlen;          // the K range that one A row covers in an item
    const int nbw = (half + KB - 1) / KB;
    // this lane's A row and B column: weight row in the tile, activation row, and where its K range starts
    const int wrow_in_tile = TM == TM_ROWS16 ? r : (r & 7) + (TM == TM_GATEUP ? (r >> 3) * n_out : 0);
    const int kr0 = kw0 + (TM == TM_DUALK ? (r >> 3) * half : 0) + g * 8;      // relative to ks0
    const int kr1 = TM == TM_DUALK ? min(kw1, kw0 + ((r >> 3) + 1) * half) : kw1;
    const int row_limit = TM == TM_GATEUP ? n_out : N;            // weight rows past it are clamped (never stored)

    // cursor of the loads: (item, block in item) of the next block to ask for
    int l_item = 0, l_j = 0;
    const int xrow_i = TM == TM_DUALK ? (r & 7) : r;
    const bool xvalid = xrow_i < M;
    // XD: the activations are not staged; a block's B operands come from global memory (L2) together with its weights
    struct Block {
        bf16x8_t w[U];
        bf16x8_t x[XD ? U : 1];
    };
    auto issue = [&](Block &buf) {
        if (l_item < my_items) {
            int row = (tile0 + l_item * tstride) * NT + (TM == TM_ROWS16 ? r : (r & 7));
            if (row >= row_limit) row = row_limit - 1;
            if (TM == TM_GATEUP) row += (r >> 3) * n_out;
            const int kb = kr0 + l_j * KB;
            if (WT) {
                // tile-major weights (fllm_tile_weights): the 16 rows x 128 columns of a block lie together in the order
                // the lanes take them, so a load instruction reads 1 KiB in a row instead of 64 bytes of each of 16 rows
                const bf16_t *wp = a.w_tiles + (size_t)(tile0 + l_item * tstride) * 16 * K + (size_t)((kw0 + l_j * KB) / KB) * (16 * KB) + lane * 8;
#pragma unroll
                for (int u = 0; u < U; u++) buf.w[u] = kb + u * 32 < kr1 ? load_weights<true>(wp + u * (16 * 32)) : zero8();
            } else {
                const bf16_t *wp = a.w + (size_t)row * K + ks0 + kb;
#pragma unroll
                for (int u = 0; u < U; u++) buf.w[u] = kb + u * 32 < kr1 ? load_weights<false>(wp + u * 32) : zero8();
            }
            if (XD) {
                const bf16_t *xp = (const bf16_t *)a.x + (size_t)xrow_i * a.ldx + ks0 + kb;
#pragma unroll
                for (int u = 0; u < U; u++) buf.x[XD ? u : 0] = (kb + u * 32 < kr1 && xvalid) ? *(const bf16x8_t *)(xp + u * 32) : zero8();
            }
        }
        if (++l_j == nbw) l_j = 0, l_item++;
    };
    (void)wrow_in_tile;
    // SCALED: the parts of the sums of squares of this wave's rows (rows wave and wave + WAVES) are asked for before
    // anything else and added up after the staging, when they have long arrived: up to 256 parts a row, four a lane
    f32x4_t ssq_pre[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    const bool ssq_quick = PRO == PRO_SCALED && a.ssq_count <= 4 * kWave && (a.ssq_count & 3) == 0 && ((uintptr_t)a.ssq_in & 15) == 0;
    if (PRO == PRO_SCALED && ssq_quick && sl == 0) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int m = wave + k * WAVES;
            if (m < M && lane * 4 < a.ssq_count) ssq_pre[k] = *(const f32x4_t *)(a.ssq_in + (size_t)m * a.ssq_count + lane * 4);
        }
    }
#ifndef FLLM_BLOCKS_IN_FLIGHT
#define FLLM_BLOCKS_IN_FLIGHT 2
#endif
    constexpr int NB = XD ? 2 : FLLM_BLOCKS_IN_FLIGHT;      // blocks of weights a wave has asked for ahead of its products
    Block bl[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) issue(bl[i]);      // in flight while the activations are staged
    // what the epilogue reads besides the sums: the part that belongs to this lane's row now, the part that belongs
    // to an item when the wave whose turn it is to finish the item starts on it
    const int m_out = TM == TM_DUALK ? (r & 7) : r;
    const bool owner = TM == TM_ROWS16 ? true : (g < 2 && (TM == TM_GATEUP || r < 8));
    EpilogueOperands eo;
    load_row_operands<EPI>(a, m_out, eo);
    auto item_operands = [&](int it) {
        if (S == 1 && it < my_items && wave == (it & (WAVES - 1)) && owner)
            load_item_operands<EPI>(a, m_out, (tile0 + it * tstride) * NT + g * 4, n_out, eo);
    };
    item_operands(0);

    // the wave's own columns kw0 .. kw1 of every row
    if (PRO != PRO_BF16 && lane < 16) ssq_part[wave * 16 + lane] = 0.f;
    __builtin_amdgcn_wave_barrier();
    if (PRO == PRO_SCALED && sl == 0 && !ssq_quick) {
        // the rows' sums of squares arrive in parts: wave w adds those of rows w, w + WAVES, ..., lane by lane in
        // index order and then across the lanes, which no other row or wave changes
        for (int m = wave; m < M; m += WAVES) {
            float t = 0.f;
            for (int i = lane; i < a.ssq_count; i += kWave) t += a.ssq_in[(size_t)m * a.ssq_count + i];
            t = wave_sum(t);
            if (lane == 0) ssq_part[wave * 16 + m] = t;
        }
    }
    for (int cw = kw0; cw < (XD ? 0 : kw1); cw += kWave * 8) {   // the same trips for every lane: the sums below are over the wave
        const int c0 = cw + lane * 8;
        const bool in = c0 < kw1;
        if (PRO != PRO_NORM_F32) {
            const bf16_t *x = (const bf16_t *)a.x + ks0 + c0;
            for (int m0 = 0; m0 < M; m0 += 4) {
                bf16x8_t v[4];
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (in && m0 + i < M) v[i] = *(const bf16x8_t *)(x + (size_t)(m0 + i) * a.ldx);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (in && m0 + i < M) *(bf16x8_t *)(xs + (m0 + i) * pitch + c0) = v[i];
            }
        } else {
            const float *x = (const float *)a.x + ks0 + c0;
            f32x4_t w0 = {0.f, 0.f, 0.f, 0.f}, w1 = w0;
            if (in) w0 = *(const f32x4_t *)(a.norm_w + ks0 + c0), w1 = *(const f32x4_t *)(a.norm_w + ks0 + c0 + 4);
            for (int m0 = 0; m0 < M; m0 += RB) {   // the loads of RB rows are in flight together
                f32x4_t xv[RB][2];
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    xv[i][0] = xv[i][1] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                    if (in && m0 + i < M) {
                        xv[i][0] = *(const f32x4_t *)(x + (size_t)(m0 + i) * a.ldx);
                        xv[i][1] = *(const f32x4_t *)(x + (size_t)(m0 + i) * a.ldx + 4);
                    }
                }
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    if (m0 + i >= M) break;
                    bf16x8_t v;
                    float ss = 0.f;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        ss += xv[i][0][e] * xv[i][0][e] + xv[i][1][e] * xv[i][1][e];
                        v[e] = (bf16_t)(xv[i][0][e] * w0[e]);
                        v[4 + e] = (bf16_t)(xv[i][1][e] * w1[e]);
                    }
                    if (in) *(bf16x8_t *)(xs + (m0 + i) * pitch + c0) = v;
                    ss = wave_sum(ss);
                    if (lane == 0) ssq_part[wave * 16 + m0 + i] += ss;
                }
            }
        }
    }
    if (PRO == PRO_SCALED && ssq_quick && sl == 0) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int m = wave + k * WAVES;
            if (m < M) {      // the same for all lanes of the wave
                const float t = wave_sum((ssq_pre[k][0] + ssq_pre[k][1]) + (ssq_pre[k][2] + ssq_pre[k][3]));
                if (lane == 0) ssq_part[wave * 16 + m] = t;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();   // the wave reads what its own lanes wrote: LDS keeps a wave's accesses in order

    // cursor of the products
    int item = 0, j = 0;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    const bf16_t *xrow = xs + xrow_i * pitch + kr0;
    FLLM_STAMP(a, 1);

    auto step = [&](Block &buf) {
        bf16x8_t xf[U];
        const int kb = kr0 + j * KB;
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (XD) xf[u] = buf.x[XD ? u : 0];
            else xf[u] = (kb + u * 32 < kr1 && xvalid) ? *(const bf16x8_t *)(xrow + j * KB + u * 32) : zero8();
        }
#pragma unroll
        for (int u = 0; u < U; u++) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf.w[u], xf[u], acc, 0, 0, 0);
        issue(buf);      // the block two ahead takes this one's registers
#ifdef FLLM_TIMELINE
        if (item == 0 && j == 0) {
            asm volatile("" ::"v"(acc));      // the first block's products have been issued: its loads had arrived
            FLLM_STAMP(a, 2);
        }
#endif
        if (++j < nbw) return;
        // the item is complete: the waves' sums meet in LDS; one wave (they take turns) adds them up and goes on
        // to the epilogue while the others start the next item
        j = 0;
        if (item == my_items - 1) FLLM_STAMP(a, 3);
        red[wave * kWave + lane] = acc;
        acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        __syncthreads();
        const int tile = tile0 + item * tstride;
        const bool finisher = wave == (item & (WAVES - 1));
        // D[row 4 g + i][column r]: for the 8-output tiles the lanes g < 2 (`owner`) hold outputs 4 g + i, and their
        // partners sit 32 lanes on (TM_GATEUP: the up rows) or 32 + 8 lanes on (TM_DUALK: the other K half)
        f32x4_t s[RT];
        if (finisher && owner) {
#pragma unroll
            for (int t = 0; t < RT; t++) s[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int wv = 0; wv < WAVES; wv++) {
                s[0] += red[wv * kWave + lane];
                if (TM == TM_DUALK) s[0] += red[wv * kWave + lane + 40];
                if (TM == TM_GATEUP) s[RT - 1] += red[wv * kWave + lane + 32];
            }
        }
        __syncthreads();      // the sums have been read: the next item may overwrite them
        if (finisher) {
            do {
                const int m = m_out, nb = tile * NT + g * 4;
                float ss = 0.f;
                if (PRO != PRO_BF16) {
#pragma unroll
                    for (int wv = 0; wv < WAVES; wv++) ss += ssq_part[wv * 16 + m];
                }
                if (S > 1) {
                    float *part = a.ws + ((size_t)(tile * S + sl) * RT * kWave + lane) * 4;
                    if (owner && m < M) {
#pragma unroll
                        for (int t = 0; t < RT; t++)
#pragma unroll
                            for (int i = 0; i < 4; i++)
                                __hip_atomic_store(part + t * kWave * 4 + i, s[t][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (PRO != PRO_BF16 && g == 0)
                            __hip_atomic_store(a.ws_ssq + (size_t)(tile * S + sl) * 16 + m, ss, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    // Every access to the workspace goes to the device's point of coherence by itself (agent-scope
                    // atomics), so no cache has to be written back or dropped: it is enough that the wave's partial
                    // sums have arrived there before the item is counted.
                    parts_published();
                    int seen = 0;
                    if (lane == 0) seen = __hip_atomic_fetch_add(a.counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    seen = __shfl(seen, 0, kWave);
                    if (seen != S - 1) break;       // another workgroup finishes this tile
                    parts_visible();
                    if (lane == 0) __hip_atomic_store(a.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
                    if (!owner || m >= M) break;
#pragma unroll
                    for (int t = 0; t < RT; t++) s[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                    ss = 0.f;
                    // four slices at a time: their loads are all asked for before the first is added (in slice order)
                    for (int s0 = 0; s0 < S; s0 += 4) {
                        float pv[4][RT][4], ps[4];
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const bool live = s0 + j < S;
                            const float *src = a.ws + ((size_t)(tile * S + (live ? s0 + j : s0)) * RT * kWave + lane) * 4;
#pragma unroll
                            for (int t = 0; t < RT; t++)
#pragma unroll
                                for (int i = 0; i < 4; i++)
                                    pv[j][t][i] = live ? __hip_atomic_load(src + t * kWave * 4 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
                            ps[j] = (PRO != PRO_BF16 && live)
                                        ? __hip_atomic_load(a.ws_ssq + (size_t)(tile * S + s0 + j) * 16 + m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                        : 0.f;
                        }
#pragma unroll
                        for (int j = 0; j < 4; j++) {
#pragma unroll
                            for (int t = 0; t < RT; t++)
#pragma unroll
                                for (int i = 0; i < 4; i++) s[t][i] += pv[j][t][i];
                            ss += ps[j];
                        }
                    }
                }
                if (!owner || m >= M || nb >= n_out) break;
                if (S > 1) eo.have = false;     // the tile was finished by whoever came last: nothing was asked for ahead
                epilogue<PRO, EPI, RT>(a, s, ss, m, nb, n_out, eo);
            } while (false);
        }
        item++;
        item_operands(item);
    };

    const int total = my_items * nbw;
    for (int q = 0; q < total; q += NB) {
#pragma unroll
        for (int i = 0; i < NB; i++)
            if (i == 0 || q + i < total) step(bl[i]);
    }
    FLLM_STAMP(a, 4);
}

// ---------------------------------------------------------------------------------------------
// 17 to 64 rows: a workgroup of four waves takes four weight row tiles and a K slice
// ---------------------------------------------------------------------------------------------
// Every wave owns one 16-row weight tile (8 gate + 8 up rows for the SwiGLU form) for the whole K
// slice of its workgroup, so no sums cross waves.  The activations of the slice pass through LDS in
// chunks of 256 columns, shared by the four waves, the next chunk on its way from global memory
// while the current one is multiplied (two buffers, one barrier per chunk).  The weights go from
// global memory straight into MFMA A operands, two chunks (16 KiB a wave) in flight ahead of the
// products, across chunk, tile and item borders.  Workgroup b owns slice b % S and the row groups
// b / S, b / S + G / S, ...  With S > 1 a wave leaves its tile's sums in the workspace and counts
// the tile; the wave that counts the last slice adds the S partial sums in slice order and runs
// the epilogue (as in the resident kernel).
// WT: the weights come from their tile-major copy (fllm_tile_weights, fllm_tile_weights_gate_up), K a multiple of 256.
// PRO_SCALED: the rows are what the product before prepared for an RMSNorm (fllm_linear_add_normed); the row's scale,
// from the parts of its sum of squares, multiplies the finished sums.
template <int MT, int EPI, bool WT = false, int WAVES = 4, int PRO = PRO_BF16>
__global__ void __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
skinny_wide_kernel(SkinnyArgs a) {
    static_assert(PRO == PRO_BF16 || PRO == PRO_SCALED, "rows arrive in bfloat16");
    constexpr int THREADS = WAVES * kWave;
    constexpr int KC = 256;                        // columns per chunk
    constexpr int KS = KC / 32;                    // MFMA k-steps per chunk
    constexpr int XP = KC + 8;                     // pitch of an activation row in LDS
    constexpr int ROWS = MT * 16;
    constexpr int XPIECES = ROWS * (KC / 8);       // 16-byte pieces of a chunk of activations
    constexpr int XL = (XPIECES + THREADS - 1) / THREADS;   // loads per thread and chunk
    constexpr int NT = EPI == EPI_SWIGLU ? 8 : 16; // outputs per row and tile
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][ROWS * XP];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N, K = a.K, S = a.S;
    const int n_out = EPI == EPI_SWIGLU ? N / 2 : N;
    const int ntiles = (n_out + NT - 1) / NT;
    const int ngroups = (ntiles + WAVES - 1) / WAVES;
    const int sl = blockIdx.x % S;
    const int rg0 = blockIdx.x / S, rstride = gridDim.x / S;
    const int ks0 = sl * a.slice;
    const int kcn = min(K, ks0 + a.slice) - ks0;                  // columns of this slice, a multiple of 8
    const int nchunks = (kcn + KC - 1) / KC;
    const int my_items = rg0 < ngroups ? (ngroups - rg0 + rstride - 1) / rstride : 0;
    const int total = my_items * nchunks;                         // chunk steps of this workgroup, the same for every wave
    const bf16_t *x = (const bf16_t *)a.x;

    // weights: cursor (item, chunk) of the next chunk to ask for
    int w_item = 0, w_chunk = 0;
    // Every lane issues every load: where it has nothing of its own to load (columns behind the slice, rows behind
    // the last one, items behind the last item) it reads 16 bytes of zeros, or weights that meet zeros on the
    // activation side.  No load sits behind a branch, so a chunk waits for its own loads only and the loads of the
    // chunks behind it stay in flight.
    const bf16_t *zeros = (const bf16_t *)&kZeros;
    auto issue_w = [&](bf16x8_t (&buf)[KS]) {
        const bool live = w_item < my_items;
        const int tile = (rg0 + (live ? w_item : 0) * rstride) * WAVES + wave;
        int row = tile * NT + (EPI == EPI_SWIGLU ? (r & 7) : r);
        if (row >= n_out) row = n_out - 1;    // past the end: computed from a valid row, never stored
        if (EPI == EPI_SWIGLU) row += (r >> 3) * n_out;
        const int kb = w_chunk * KC + g * 8;
        if (WT) {
            // a chunk is two blocks of 128 columns of the tile, each 4 KiB in the order the lanes take it
            const bf16_t *wp = a.w_tiles + (size_t)min(tile, ntiles - 1) * 16 * K + (size_t)((ks0 + w_chunk * KC) >> 7) * 2048 + lane * 8;
#pragma unroll
            for (int u = 0; u < KS; u++) buf[u] = load_weights<true>(live ? wp + (u >> 2) * 2048 + (u & 3) * 512 : zeros);
        } else {
            const bf16_t *wp = a.w + (size_t)row * K + ks0;
#pragma unroll
            for (int u = 0; u < KS; u++) buf[u] = load_weights<false>(live ? wp + min(kb + u * 32, kcn - 8) : zeros);
        }
        if (++w_chunk == nchunks) w_chunk = 0, w_item++;
    };
    // activations: the chunk index within the slice is all that matters (every item walks the same slice)
    bf16x8_t xr[XL];
    auto load_x = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int idx = threadIdx.x + i * THREADS;
            const int m = idx / (KC / 8), c = (idx - m * (KC / 8)) * 8 + chunk * KC;
            xr[i] = *(const bf16x8_t *)((m < M && c < kcn && idx < XPIECES) ? x + (size_t)m * a.ldx + ks0 + c : zeros);
        }
    };
    auto store_x = [&](int buffer) {
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const int idx = threadIdx.x + i * THREADS;
            const int m = idx / (KC / 8), c = (idx - m * (KC / 8)) * 8;
            if (XPIECES % THREADS == 0 || idx < XPIECES) *(bf16x8_t *)(&xs[buffer][m * XP + c]) = xr[i];
        }
    };

    bf16x8_t wa[KS], wb[KS];
    issue_w(wa);
    issue_w(wb);
    __shared__ float ssq_rows[PRO == PRO_SCALED ? ROWS : 1];
    if (PRO == PRO_SCALED) {
        // A row's sum of squares arrives in parts (up to a few hundred).  Four neighbouring threads share a row: each adds
        // a quarter of the parts in index order, all its loads asked for together, and the quarters are added in order:
        // the same sum for a row whatever the batch and the workgroup, and one trip to memory for all rows at once.
        static_assert(THREADS >= 4 * ROWS, "four threads a row");
        const int m = threadIdx.x >> 2, q = threadIdx.x & 3;
        float t = 0.f;
        if (threadIdx.x < 4 * ROWS) {      // whole waves: ROWS is a multiple of 16
            const int per = (a.ssq_count + 3) / 4;
            const int i0 = min(q * per, a.ssq_count), i1 = min(i0 + per, a.ssq_count);
            if (m < M) {
                const float *parts = a.ssq_in + (size_t)m * a.ssq_count;
                if ((per & 3) == 0 && (a.ssq_count & 3) == 0 && ((uintptr_t)a.ssq_in & 15) == 0) {
#pragma unroll 4
                    for (int i = i0; i < i1; i += 4) {
                        const f32x4_t v = *(const f32x4_t *)(parts + i);
                        t += v[0];
                        t += v[1];
                        t += v[2];
                        t += v[3];
                    }
                } else {
                    for (int i = i0; i < i1; i++) t += parts[i];
                }
            }
            const float t1 = __shfl_xor(t, 1, kWave);
            const float pair = (q & 1) ? t1 + t : t + t1;          // quarter 2 k, then quarter 2 k + 1
            const float other = __shfl_xor(pair, 2, kWave);
            const float sum = (q & 2) ? other + pair : pair + other;
            if (q == 0 && m < M) ssq_rows[m] = sum;
        }
    }
    if (total > 0) {
        load_x(0);
        store_x(0);
    }
    __syncthreads();

    f32x4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    int item = 0, chunk = 0;

    auto step = [&](bf16x8_t (&buf)[KS], int q) {
        const int next_chunk = chunk + 1 == nchunks ? 0 : chunk + 1;
        load_x(next_chunk);      // on its way while this chunk is multiplied (once more than needed at the very end)
        const bf16_t *xb = &xs[q & 1][r * XP + g * 8];
#pragma unroll
        for (int u = 0; u < KS; u++) {
            bf16x8_t xf[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) xf[mt] = *(const bf16x8_t *)(xb + mt * 16 * XP + u * 32);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf[u], xf[mt], acc[mt], 0, 0, 0);
        }
        issue_w(buf);      // the chunk two ahead takes this one's registers
        store_x((q + 1) & 1);
        __syncthreads();   // the next chunk is in LDS; everybody has read the one before it
        chunk = next_chunk;
        if (chunk != 0 || item >= my_items) return;      // (a step behind the last item multiplies zeros and ends nothing)
        // the item is complete: this wave's tile has its sums over the slice
        const int tile = (rg0 + item * rstride) * WAVES + wave;
        item++;
        const bool owner = EPI == EPI_SWIGLU ? g < 2 : true;      // 8-output tiles: lanes g < 2 hold gate rows, g >= 2 the up rows
        const int nb = tile * NT + g * 4;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            f32x4_t s[RT];
            s[0] = acc[mt];
            if (EPI == EPI_SWIGLU) {
#pragma unroll
                for (int i = 0; i < 4; i++) s[RT - 1][i] = __shfl(acc[mt][i], (lane + 32) & 63, kWave);
            }
            acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            const int m = mt * 16 + r;
            bool finish = tile < ntiles;
            if (S > 1 && tile < ntiles) {       // wave-uniform: the whole wave takes part in the hand-over
                const __amdgpu_buffer_rsrc_t wsb = workspace_buffer(a.ws);
                const unsigned int part = (unsigned int)(((((size_t)tile * S + sl) * MT + mt) * RT * kWave + lane) * 16);
                if (owner && m < M) {
#pragma unroll
                    for (int t = 0; t < RT; t++) hand_over(wsb, part + t * kWave * 16, s[t]);
                }
                if (mt == MT - 1) {
                    // the pieces pass by the caches on both ways: it is enough that the wave's own have arrived in
                    // memory before the tile is counted
                    parts_published();
                    int seen = 0;
                    if (lane == 0) seen = __hip_atomic_fetch_add(a.counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    seen = __shfl(seen, 0, kWave);
                    if (seen == S - 1) {        // the last slice of this tile: add the parts in slice order
                        parts_visible();
                        if (lane == 0) __hip_atomic_store(a.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                        for (int mt2 = 0; mt2 < MT; mt2++) {
                            const int m2 = mt2 * 16 + r;
                            const bool mine = owner && m2 < M && nb < n_out;
                            f32x4_t t2[RT];
#pragma unroll
                            for (int t = 0; t < RT; t++) t2[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                            // the parts of up to eight slices are asked for together (one trip to memory, not one a
                            // slice) and added in slice order; every lane loads, so that no load sits behind a branch
                            constexpr int GRP = MT > 4 ? 4 : 8;      // (with more row tiles the registers are needed elsewhere)
                            for (int s0 = 0; s0 < S; s0 += GRP) {
                                f32x4_t pv[GRP][RT];
#pragma unroll
                                for (int j = 0; j < GRP; j++) {
                                    const int s2 = s0 + j < S ? s0 + j : s0;
                                    const unsigned int src = (unsigned int)(((((size_t)tile * S + s2) * MT + mt2) * RT * kWave + lane) * 16);
#pragma unroll
                                    for (int t = 0; t < RT; t++) pv[j][t] = take_over(wsb, src + t * kWave * 16);
                                }
#pragma unroll
                                for (int j = 0; j < GRP; j++)
#pragma unroll
                                    for (int t = 0; t < RT; t++)
                                        if (s0 + j < S) t2[t] += pv[j][t];
                            }
                            if (!mine) continue;
                            EpilogueOperands eo;
                            load_row_operands<EPI>(a, m2, eo);
                            epilogue<PRO, EPI, RT>(a, t2, PRO == PRO_SCALED ? ssq_rows[m2] : 0.f, m2, nb, n_out, eo);
                        }
                    }
                }
                finish = false;
            }
            if (finish && owner && m < M && nb < n_out) {
                EpilogueOperands eo;
                load_row_operands<EPI>(a, m, eo);
                epilogue<PRO, EPI, RT>(a, s, PRO == PRO_SCALED ? ssq_rows[m] : 0.f, m, nb, n_out, eo);
            }
        }
    };

    // The two buffers take turns without a condition between them (an odd number of steps gets one more, which
    // multiplies zeros): only then does the compiler see that the loads of one buffer always lie behind those of
    // the other, and lets them stay in flight.
    for (int q = 0; q < total; q += 2) {
        step(wa, q);
        step(wb, q + 1);
    }
}

// ---------------------------------------------------------------------------------------------
// 17 to 64 rows: the activations of a K slice stay in LDS, one workgroup a compute unit walks over row groups
// ---------------------------------------------------------------------------------------------
// With this many rows the activations weigh as much as the weights a workgroup streams past them, so they must not
// be fetched again for every weight tile.  A workgroup of 8 waves stages ONE K slice of all rows in LDS (up to 1,024
// columns of 64 rows: 132 KiB; for the norm prologue x * norm_weight as bfloat16, and the slice's part of every row's
// sum of squares) and keeps it for the whole launch.  It then walks over row groups of 8 weight tiles, one tile a
// wave (16 weight rows, or 8 gate and 8 up rows), each wave over the whole slice: the weights go from global
// memory straight into MFMA A operands, two chunks of 256 columns (16 KiB a wave) in flight ahead of the products;
// the B operands come from LDS.  No wave waits for another after the staging.  Workgroup b owns slice b % S and the
// row groups b / S, b / S + G / S, ...  With S > 1 a wave leaves its tile's sums (and the slice's sums of squares)
// in the workspace and counts the tile; the wave that counts the last slice adds the S parts in slice order and
// runs the epilogue, so the result does not depend on who came last.
template <int PRO, int EPI, int MT>
__global__ void __launch_bounds__(8 * kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
skinny_slab_kernel(SkinnyArgs a, int cells_off) {
    constexpr int WAVES = 8, THREADS = WAVES * kWave;
    constexpr int KC = 256;                        // columns per chunk of weights
    constexpr int KS = KC / 32;                    // MFMA k-steps per chunk
    constexpr int ROWS = MT * 16;
    constexpr int NT = EPI == EPI_SWIGLU ? 8 : 16; // outputs per row and tile
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N, K = a.K, S = a.S;
    const int n_out = EPI == EPI_SWIGLU ? N / 2 : N;
    const int ntiles = (n_out + NT - 1) / NT;
    const int ngroups = (ntiles + WAVES - 1) / WAVES;
    const int sl = blockIdx.x % S;
    const int rg0 = blockIdx.x / S, rstride = gridDim.x / S;
    const int ks0 = sl * a.slice;
    const int kcn = min(K, ks0 + a.slice) - ks0;                  // columns of this slice, a multiple of 8
    const int nchunks = (kcn + KC - 1) / KC;
    const int my_items = rg0 < ngroups ? (ngroups - rg0 + rstride - 1) / rstride : 0;
    const int total = my_items * nchunks;                         // chunk steps of every wave of this workgroup
    const int pitch = a.slice + 8;
    bf16_t *xs = (bf16_t *)smem;                                  // [ROWS][pitch]; columns from kcn on and rows from M on are zero
    float *cells = (float *)(smem + cells_off);                   // norm prologue: [ROWS][slice / 512] sums of squares
    const int cpr = a.slice / 8;                                  // 16-byte pieces of a staged row
    const int cells_per_row = (a.slice + 511) / 512;

    // weights: cursor (item, chunk) of the next chunk to ask for.  Every lane issues every load (zeros where it has
    // nothing of its own), so no load sits behind a branch and the chunks behind the current one stay in flight.
    int w_item = 0, w_chunk = 0;
    // Every wave walks the chunks of its slice in a circle, starting at a chunk of its own: at any moment the waves of
    // the device then read different columns, which lie in different memory channels (all waves at the same columns
    // of rows that are a power of two apart would crowd into a few channels).
    const int phase = (wave + rg0) % nchunks;
    const bf16_t *zeros = (const bf16_t *)&kZeros;
    auto issue_w = [&](bf16x8_t (&buf)[KS]) __attribute__((always_inline)) {
        const bool live = w_item < my_items;
        const int tile = (rg0 + (live ? w_item : 0) * rstride) * WAVES + wave;
        int row = tile * NT + (EPI == EPI_SWIGLU ? (r & 7) : r);
        if (row >= n_out) row = n_out - 1;    // past the end: computed from a valid row, never stored
        if (EPI == EPI_SWIGLU) row += (r >> 3) * n_out;
        const int kb = ((w_chunk + phase) % nchunks) * KC + g * 8;
        const bf16_t *wp = a.w + (size_t)row * K + ks0;
#pragma unroll
        for (int u = 0; u < KS; u++) buf[u] = load_weights<false>(live ? wp + min(kb + u * 32, kcn - 8) : zeros);
        if (++w_chunk == nchunks) w_chunk = 0, w_item++;
    };
    bf16x8_t wa[KS], wb[KS];
    issue_w(wa);      // in flight while the activations are staged
    issue_w(wb);

    // ---- staging: piece idx of the slice is (row idx / cpr, columns (idx % cpr) * 8 ...) ----
    if (PRO == PRO_BF16) {
        const bf16_t *x = (const bf16_t *)a.x;
        constexpr int B = 8;       // loads in flight a thread
        for (int i0 = threadIdx.x; i0 < ROWS * cpr; i0 += B * THREADS) {
            bf16x8_t v[B];
#pragma unroll
            for (int i = 0; i < B; i++) {
                const int idx = i0 + i * THREADS;
                const int m = idx / cpr, c = (idx - m * cpr) * 8;
                v[i] = *(const bf16x8_t *)((idx < ROWS * cpr && m < M && c < kcn) ? x + (size_t)m * a.ldx + ks0 + c : zeros);
            }
#pragma unroll
            for (int i = 0; i < B; i++) {
                const int idx = i0 + i * THREADS;
                const int m = idx / cpr, c = (idx - m * cpr) * 8;
                if (idx < ROWS * cpr) *(bf16x8_t *)(xs + m * pitch + c) = v[i];
            }
        }
    } else {
        // A wave covers 512 consecutive columns of one row at a time (the slice is a multiple of 512 columns), so one
        // cell holds the squares of exactly one wave's trip: every cell is written once, and a row's sum is the sum of
        // its cells in order.
        const float *x = (const float *)a.x;
        constexpr int B = 4;
        for (int i0 = threadIdx.x; i0 < ROWS * cpr; i0 += B * THREADS) {
            f32x4_t xv[B][2], nw[B][2];
#pragma unroll
            for (int i = 0; i < B; i++) {
                const int idx = i0 + i * THREADS;
                const int m = idx / cpr, c = (idx - m * cpr) * 8;
                const bool in = idx < ROWS * cpr && m < M && c < kcn;
                const float *src = in ? x + (size_t)m * a.ldx + ks0 + c : (const float *)zeros;
                const float *wsrc = in ? a.norm_w + ks0 + c : (const float *)zeros;
                xv[i][0] = *(const f32x4_t *)src;
                xv[i][1] = in ? *(const f32x4_t *)(src + 4) : (f32x4_t){0.f, 0.f, 0.f, 0.f};
                nw[i][0] = *(const f32x4_t *)wsrc;
                nw[i][1] = in ? *(const f32x4_t *)(wsrc + 4) : (f32x4_t){0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int i = 0; i < B; i++) {
                const int idx = i0 + i * THREADS;     // the same for all lanes of a wave up to the lane index: no lane leaves the loop early
                const int m = idx / cpr, c = (idx - m * cpr) * 8;
                bf16x8_t v;
                float ss = 0.f;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    ss += xv[i][0][e] * xv[i][0][e] + xv[i][1][e] * xv[i][1][e];
                    v[e] = (bf16_t)(xv[i][0][e] * nw[i][0][e]);
                    v[4 + e] = (bf16_t)(xv[i][1][e] * nw[i][1][e]);
                }
                if (idx < ROWS * cpr) *(bf16x8_t *)(xs + m * pitch + c) = v;
                ss = wave_sum(ss);
                if (lane == 0 && idx < ROWS * cpr) cells[m * cells_per_row + c / 512] = ss;
            }
        }
    }
    __syncthreads();

    f32x4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    int item = 0, chunk = 0;
    const bf16_t *xb = xs + r * pitch + g * 8;

    // ---- what happens to a finished tile ----
    // One slice (S == 1): the wave runs the epilogue.  Several: the wave leaves its sums and its slice's sums of
    // squares in the workspace, counts the tile, and whoever counts last adds the S parts in slice order and runs
    // the epilogue.  None of this may make the wave wait, or the weights stop streaming, so it is spread over three
    // item ends: the parts are sent at the end of their own item; the tile is counted at the end of the item after,
    // behind a release fence (the stores have had an item's time by then); the count is looked at one item later still.
    const bool owner = EPI == EPI_SWIGLU ? g < 2 : true;      // 8-output tiles: lanes g < 2 hold gate rows, g >= 2 the up rows
    const __amdgpu_buffer_rsrc_t wsb = workspace_buffer(a.ws);
    int sent_tile = -1;                     // parts sent, tile not counted yet
    int counted_tile = -1, counted_raw = 0; // tile counted; lane 0 holds what the counter said, not looked at yet

    // the epilogue of one 16-row block of a tile
    auto finish_rows = [&](int tile, int mt, f32x4_t (&s)[RT], float ss) __attribute__((always_inline)) {
        const int nb = tile * NT + g * 4;
        const int m = mt * 16 + r;
        if (!owner || m >= M || nb >= n_out) return;
        EpilogueOperands eo;
        load_row_operands<EPI>(a, m, eo);
        load_item_operands<EPI>(a, m, nb, n_out, eo);
        epilogue<PRO, EPI, RT>(a, s, ss, m, nb, n_out, eo);
    };
    auto look = [&]() __attribute__((always_inline)) {
        if (counted_tile < 0) return;
        const int tile = counted_tile;
        counted_tile = -1;
        if (__shfl(counted_raw, 0, kWave) != S - 1) return;      // another workgroup finishes this tile
        parts_visible();
        if (lane == 0) __hip_atomic_store(a.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        // one block of 16 rows after the other (few registers: this runs in the middle of the stream of weights); the
        // parts of two slices are asked for before the first is added, and they are added in slice order
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const bool mine = owner && mt * 16 + r < M;
            f32x4_t s[RT];
#pragma unroll
            for (int t = 0; t < RT; t++) s[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            float ss = 0.f;
            for (int s0 = 0; s0 < S; s0 += 2) {
                f32x4_t pv[2][RT];
                float ps[2];
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const bool live = s0 + j < S;
                    const size_t at = (size_t)tile * S + (live ? s0 + j : s0);
                    const unsigned int src = (unsigned int)(((at * MT + mt) * RT * kWave + lane) * 16);
#pragma unroll
                    for (int t = 0; t < RT; t++) {
                        const f32x4_t got = take_over(wsb, src + t * kWave * 16);     // every lane loads: no load behind a branch
                        pv[j][t] = (live && mine) ? got : (f32x4_t){0.f, 0.f, 0.f, 0.f};
                    }
                    ps[j] = 0.f;
                    if (PRO == PRO_NORM_F32) {
                        const float got = __hip_atomic_load(a.ws_ssq + at * ROWS + mt * 16 + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        ps[j] = live ? got : 0.f;
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; j++) {
#pragma unroll
                    for (int t = 0; t < RT; t++) s[t] += pv[j][t];
                    ss += ps[j];
                }
            }
            finish_rows(tile, mt, s, ss);
        }
    };
    // The parts were sent at the end of the item before: by now their stores have had an item's time to complete, and
    // the release fence waits for whatever of them has not (loads and stores of a wave may complete out of their order
    // of issue with respect to each other, so counting outstanding operations cannot stand in for it).
    auto count = [&]() __attribute__((always_inline)) {
        if (sent_tile < 0) return;
        parts_published();
        if (lane == 0) counted_raw = __hip_atomic_fetch_add(a.counters + sent_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        counted_tile = sent_tile;
        sent_tile = -1;
    };

    auto step = [&](bf16x8_t (&buf)[KS]) __attribute__((always_inline)) {
        const bf16_t *xc = xb + ((chunk + phase) % nchunks) * KC;
#pragma unroll
        for (int u = 0; u < KS; u++) {
            bf16x8_t xf[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) xf[mt] = *(const bf16x8_t *)(xc + mt * 16 * pitch + u * 32);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf[u], xf[mt], acc[mt], 0, 0, 0);
        }
        issue_w(buf);      // the chunk two ahead takes this one's registers
        if (++chunk < nchunks) return;
        chunk = 0;
        if (item >= my_items) return;      // (a step behind the last item multiplied zeros and ends nothing)
        // the item is complete: this wave's tile has its sums over the slice
        const int tile = (rg0 + item * rstride) * WAVES + wave;
        item++;
        if (S > 1) {
            look();
            count();
        }
        f32x4_t s[MT][RT];
        float ss[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            s[mt][0] = acc[mt];
            if (EPI == EPI_SWIGLU) {
#pragma unroll
                for (int i = 0; i < 4; i++) s[mt][RT - 1][i] = __shfl(acc[mt][i], (lane + 32) & 63, kWave);
            }
            acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            ss[mt] = 0.f;
            if (PRO == PRO_NORM_F32) {
                for (int c = 0; c < cells_per_row; c++) ss[mt] += cells[(mt * 16 + r) * cells_per_row + c];
            }
        }
        if (tile >= ntiles) return;        // wave-uniform: a wave without a tile in the last row group
        if (S == 1) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) finish_rows(tile, mt, s[mt], ss[mt]);
            return;
        }
        // a tile's part of a slice: [mt][t][lane] pieces of 16 bytes; offsets in bytes from the start of the partial sums
        const unsigned int part = (unsigned int)((((size_t)tile * S + sl) * MT * RT * kWave + lane) * 16);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            if (!owner || mt * 16 + r >= M) continue;
#pragma unroll
            for (int t = 0; t < RT; t++) hand_over(wsb, part + (mt * RT + t) * kWave * 16, s[mt][t]);
            if (PRO == PRO_NORM_F32 && g == 0)
                __hip_atomic_store(a.ws_ssq + ((size_t)tile * S + sl) * ROWS + mt * 16 + r, ss[mt], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        sent_tile = tile;
    };

    // The two buffers take turns without a condition between them (an odd number of steps gets one more, which
    // multiplies zeros): only then does the compiler see that the loads of one buffer always lie behind those of
    // the other, and lets them stay in flight.
    for (int q = 0; q < total; q += 2) {
        step(wa);
        step(wb);
    }
    if (S > 1) {       // what the last items left to do
        look();
        count();
        look();
    }
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

// Workspace of the K-sliced products: the device workspace, if the host program has set one.
struct Workspace {
    float *base = nullptr;
    size_t bytes = 0;
};
constexpr size_t kCounterBytes = kWorkspaceCounterBytes;
static_assert(kWorkspaceCounterBytes == fllm_plan::kCounterBytes, "plans.h and common.h agree on the counters");
using fllm_plan::ResidentPlan;

// the plan of a resident launch (plans.h), with the options that are set by hand
ResidentPlan plan_resident(int M, int K, int ntiles, int rt, const Workspace &ws, bool x_direct) {
    return fllm_plan::plan_resident(M, K, ntiles, rt, ws.bytes, ws.base != nullptr, x_direct, fllm_option_linear_slices());
}

#ifdef FLLM_TIMELINE
unsigned long long *g_timeline = nullptr;
#endif

template <int PRO, int EPI, int TM, int WAVES, bool XD = false, bool WT = false>
int launch_resident_plan(SkinnyArgs a, const ResidentPlan &p, int ntiles, const Workspace &ws, hipStream_t stream) {
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
#ifdef FLLM_TIMELINE
    a.timeline = g_timeline;
#endif
    a.S = p.S;
    a.slice = p.slice;
    a.ssq_off = (int)(p.stage + p.red);
    if (a.next_x != nullptr) {
        a.next_nt = TM == TM_ROWS16 ? 16 : 8;
        a.next_tiles = ntiles;
        if (a.next_tiles_out != nullptr) *a.next_tiles_out = ntiles;
    }
    if (p.S > 1) {
        a.counters = (int *)ws.base;
        a.ws = (float *)((unsigned char *)ws.base + kCounterBytes);
        a.ws_ssq = a.ws + fllm_plan::resident_ssq_offset_floats(ntiles, p.S, RT);
    }
    // One workgroup per slot of the chip and slice, tiles dealt out in turn: the first slots of the
    // compute units get one tile more than the second ones when the tiles do not divide evenly.
    const int groups = fllm_plan::resident_groups(p, ntiles, device_cus());
    static bool attribute_set = false;   // more than the default 64 KiB of dynamic LDS has to be asked for once
    if (!attribute_set) {
        const hipError_t e = hipFuncSetAttribute((const void *)skinny_resident_kernel<PRO, EPI, TM, WAVES, XD, WT>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        FLLM_REQUIRE(e == hipSuccess, "linear_skinny: cannot raise the LDS limit: %s", hipGetErrorString(e));
        attribute_set = true;
    }
    hipLaunchKernelGGL((skinny_resident_kernel<PRO, EPI, TM, WAVES, XD, WT>), dim3(groups * p.S), dim3(WAVES * kWave), p.smem, stream,
                       a, (int)p.stage);
    return fllm_check_launch("linear_skinny");
}

// Tile-major weights serve matrices whose eight waves' K ranges are whole blocks of 128 columns.
bool tiles_fit(int N, int K) { return N >= 16 && K >= 1024 && K % 1024 == 0; }

// tiles[T][B][u][lane][8] = w[16 T + lane % 16][128 B + 32 u + 8 (lane / 16) ...]: tile T of 16 rows, block B of 128 columns,
// k-step u of 32, and inside it the 16 bytes of each of the 64 lanes of a wave in lane order; rows past N are zeros
// `half_rows` > 0: w is a gate matrix on top of an up matrix of `half_rows` rows each, and tile T is rows 8 T .. 8 T + 7 of
// the one followed by the same rows of the other, as the SwiGLU epilogue wants them
__global__ void __launch_bounds__(256) tile_weights_kernel(const bf16_t *__restrict__ w, bf16_t *__restrict__ tiles, int N, int K, size_t pieces,
                                                           int half_rows) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const int blocks = K / 128;
    for (size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x; v < pieces; v += stride) {
        const int lane = (int)(v & 63), u = (int)((v >> 6) & 3);
        const size_t tb = v >> 8;
        const int B = (int)(tb % blocks);
        const size_t T = tb / blocks;
        const int r = lane & 15;
        size_t n = T * 16 + r;
        bool there = n < (size_t)N;
        if (half_rows > 0) {
            const size_t o = T * 8 + (r & 7);
            there = o < (size_t)half_rows;
            n = o + (size_t)(r >> 3) * half_rows;
        }
        const int k = B * 128 + u * 32 + (lane >> 4) * 8;
        *(bf16x8_t *)(tiles + v * 8) = there ? *(const bf16x8_t *)(w + n * K + k) : zero8();
    }
}

// Whether a staged launch (activations in LDS) may stream the tile-major copy: one slice, and every wave's K range whole
// blocks of 128 columns
bool staged_tiles_fit(const SkinnyArgs &a, const ResidentPlan &p, int n_out) {
    return a.w_tiles != nullptr && p.S == 1 && tiles_fit(n_out, a.K) && a.K % (p.waves * 128) == 0;
}

template <int PRO, int EPI>
int launch_resident(const SkinnyArgs &a, hipStream_t stream) {
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    Workspace ws;
    {
        void *base = nullptr;
        size_t bytes = 0;
        if (fllm_device_workspace(&base, &bytes)) ws.base = (float *)base, ws.bytes = bytes;
    }
    const int n_out = EPI == EPI_SWIGLU ? a.N / 2 : a.N;
    const int tiles16 = (n_out + 15) / 16, tiles8 = (n_out + 7) / 8;
    if constexpr (EPI == EPI_SWIGLU) {
        const ResidentPlan p = plan_resident(a.M, a.K, tiles8, RT, ws, false);
        if (p.S == 0) return 1;
        if (fllm_option_resident_tiles() && staged_tiles_fit(a, p, n_out)) {    // the copy of fllm_tile_weights_gate_up
            if (p.waves == 8) return launch_resident_plan<PRO, EPI, TM_GATEUP, 8, false, true>(a, p, tiles8, ws, stream);
            return launch_resident_plan<PRO, EPI, TM_GATEUP, 16, false, true>(a, p, tiles8, ws, stream);
        }
        if (p.waves == 8) return launch_resident_plan<PRO, EPI, TM_GATEUP, 8>(a, p, tiles8, ws, stream);
        return launch_resident_plan<PRO, EPI, TM_GATEUP, 16>(a, p, tiles8, ws, stream);
    } else {
        // bfloat16 activations are read where they lie when a workgroup sees few tiles (it reads each of them once
        // per tile: no dearer than staging for a tile or two, and nothing waits for the staging); with many tiles a
        // workgroup, and for the norm prologue, they are staged in LDS
        const bool x_direct = PRO == PRO_BF16 && fllm_option_x_direct() && a.ldx % 8 == 0 && tiles16 <= 4 * device_cus();
        ResidentPlan p = plan_resident(a.M, a.K, tiles16, RT, ws, x_direct);
        if (p.S == 0) return 1;
        // 8-row tiles (two K halves a product) when the rows allow it and the 16-row tiles come to between half a
        // tile and two tiles per slot, unevenly: 384 tiles on 512 slots run as long as 512 would.  Also when the 16-row
        // tiles fill no more than half of the compute units (narrow models): twice the workgroups, each with half the
        // weights (128 tiles of 2,048 x 8,192: 12.7 -> 9.4 us at one row; 192 tiles gain nothing, 7.7 -> 8.1 us, and at
        // 256 tiles it is the other way round, 26.9 -> 32.3 us)
        const int slots = device_cus() * p.per_cu;
        const bool uneven = 2 * tiles16 > slots && tiles16 < 2 * slots && tiles16 % slots != 0;
        const bool dual = a.M <= 8 && p.S == 1 && fllm_option_dual_k() && (uneven || 2 * tiles16 <= device_cus());
        if constexpr (PRO == PRO_BF16) {
            if constexpr (EPI == EPI_ADD) {     // the output and down projections: their tile-major copy, where there is one
                if (x_direct && !dual && a.w_tiles != nullptr && tiles_fit(a.N, a.K))
                    return launch_resident_plan<PRO, EPI, TM_ROWS16, 8, true, true>(a, p, tiles16, ws, stream);
            }
            if (x_direct) {
                if (dual) return launch_resident_plan<PRO, EPI, TM_DUALK, 8, true>(a, p, tiles8, ws, stream);
                return launch_resident_plan<PRO, EPI, TM_ROWS16, 8, true>(a, p, tiles16, ws, stream);
            }
        }
        if constexpr ((EPI == EPI_QKV && PRO == PRO_SCALED) || (EPI == EPI_STORE_F32 && PRO == PRO_BF16)) {
            // q/k/v behind a prepared norm and the vocabulary projection: whole 16-row tiles from the tile-major copy,
            // where there is one, rather than the matrix (in 8-row tiles where those fill the device better).  Reading
            // the activations straight from global memory as the output projection does is slower for q/k/v
            // (4,096 x 6,144 at 1, 8, 16 rows: 14.0, 15.4, 18.3 us against 12.4, 15.0, 18.1 staged).
            if (!x_direct && fllm_option_resident_tiles() && staged_tiles_fit(a, p, a.N)) {
                if (p.waves == 8) return launch_resident_plan<PRO, EPI, TM_ROWS16, 8, false, true>(a, p, tiles16, ws, stream);
                return launch_resident_plan<PRO, EPI, TM_ROWS16, 16, false, true>(a, p, tiles16, ws, stream);
            }
        }
        if (dual) {
            if (p.waves == 8) return launch_resident_plan<PRO, EPI, TM_DUALK, 8>(a, p, tiles8, ws, stream);
            return launch_resident_plan<PRO, EPI, TM_DUALK, 16>(a, p, tiles8, ws, stream);
        }
        if (p.waves == 8) return launch_resident_plan<PRO, EPI, TM_ROWS16, 8>(a, p, tiles16, ws, stream);
        return launch_resident_plan<PRO, EPI, TM_ROWS16, 16>(a, p, tiles16, ws, stream);
    }
}

template <int MT, int EPI, bool WT, int WAVES, int PRO>
int launch_wide_kernel(const SkinnyArgs &a, int grid, hipStream_t stream) {
    hipLaunchKernelGGL((skinny_wide_kernel<MT, EPI, WT, WAVES, PRO>), dim3(grid), dim3(WAVES * kWave), 0, stream, a);
    return fllm_check_launch("linear_wide");
}

// 1: the shape is not served (the scaled prologue and the q/k/v epilogue only with the tile-major copy)
template <int MT, int EPI, int PRO = PRO_BF16>
int launch_wide(SkinnyArgs a, hipStream_t stream) {
    constexpr int NT = EPI == EPI_SWIGLU ? 8 : 16;
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    const int n_out = EPI == EPI_SWIGLU ? a.N / 2 : a.N;
    const int ntiles = (n_out + NT - 1) / NT;
    void *base = nullptr;
    size_t bytes = 0;
    const bool have_ws = fllm_device_workspace(&base, &bytes);
    // workgroups of seven or eight waves only with the weights' tile-major copy (they were measured with it)
    const bool tiled = a.w_tiles != nullptr && a.K % 256 == 0;
    if (MT > 4 && !tiled) return 1;
    // more than 64 rows: eight waves share the chunk of activations, which then fills LDS (and the prologue of a
    // prepared norm has four threads a row)
    const fllm_plan::ChunkPlan p =
        MT > 4 ? fllm_plan::plan_chunks(a.K, ntiles, MT, RT, bytes, have_ws, device_cus(), fllm_option_linear_slices(), 8)
        : tiled ? fllm_plan::plan_chunks_balanced(a.K, ntiles, MT, RT, bytes, have_ws, device_cus(), fllm_option_linear_slices(),
                                                  fllm_option_wide_waves())
                : fllm_plan::plan_chunks(a.K, ntiles, MT, RT, bytes, have_ws, device_cus(), fllm_option_linear_slices(), 4);
    a.S = p.S;
    a.slice = p.slice;
    if (p.S > 1) {
        a.counters = (int *)base;
        a.ws = (float *)((unsigned char *)base + kWorkspaceCounterBytes);
    }
    if (a.next_x != nullptr) {
        a.next_nt = NT;
        a.next_tiles = ntiles;
        *a.next_tiles_out = ntiles;
    }
    constexpr bool kTiledOnly = PRO != PRO_BF16 || EPI == EPI_QKV;
    constexpr bool kHasTiles = EPI == EPI_ADD || EPI == EPI_SWIGLU || EPI == EPI_QKV || EPI == EPI_STORE_F32;     // the matrices that get copies
    if constexpr (MT > 4) {
        return launch_wide_kernel<MT, EPI, true, 8, PRO>(a, p.grid, stream);
    } else {
        if constexpr (kHasTiles) {
            if (tiled) {
                if (p.waves == 7) return launch_wide_kernel<MT, EPI, true, 7, PRO>(a, p.grid, stream);
                if (p.waves == 8) return launch_wide_kernel<MT, EPI, true, 8, PRO>(a, p.grid, stream);
                return launch_wide_kernel<MT, EPI, true, 4, PRO>(a, p.grid, stream);
            }
        }
        if constexpr (kTiledOnly) return 1;
        else return launch_wide_kernel<MT, EPI, false, 4, PRO_BF16>(a, p.grid, stream);
    }
}

using fllm_plan::SlabPlan;

template <int PRO, int EPI, int MT>
int launch_slab(SkinnyArgs a, hipStream_t stream) {
    constexpr int NT = EPI == EPI_SWIGLU ? 8 : 16;
    constexpr int RT = EPI == EPI_SWIGLU ? 2 : 1;
    const int n_out = EPI == EPI_SWIGLU ? a.N / 2 : a.N;
    const int ntiles = (n_out + NT - 1) / NT;
    void *base = nullptr;
    size_t bytes = 0;
    const bool have_ws = fllm_device_workspace(&base, &bytes);
    const SlabPlan p = fllm_plan::plan_slab(a.M, ntiles, a.K, MT, RT, PRO == PRO_NORM_F32, NT, bytes, have_ws, device_cus(),
                                            fllm_option_linear_slices());
    if (p.S == 0) return 1;
    a.S = p.S;
    a.slice = p.slice;
    if (p.S > 1) {
        a.counters = (int *)base;
        a.ws = (float *)((unsigned char *)base + kWorkspaceCounterBytes);
        a.ws_ssq = a.ws + fllm_plan::slab_ssq_offset_floats(ntiles, p.S, MT, RT);
    }
    static bool attribute_set = false;   // more than the default 64 KiB of dynamic LDS has to be asked for once
    if (!attribute_set) {
        const hipError_t e = hipFuncSetAttribute((const void *)skinny_slab_kernel<PRO, EPI, MT>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        FLLM_REQUIRE(e == hipSuccess, "linear_skinny: cannot raise the LDS limit: %s", hipGetErrorString(e));
        attribute_set = true;
    }
    hipLaunchKernelGGL((skinny_slab_kernel<PRO, EPI, MT>), dim3(p.grid), dim3(8 * kWave), p.smem, stream, a, (int)p.cells_off);
    return fllm_check_launch("linear_slab");
}

template <int PRO, int EPI>
int dispatch_slab(const SkinnyArgs &a, hipStream_t stream) {
    const int mt = (a.M + 15) / 16;
    if (mt == 2) return launch_slab<PRO, EPI, 2>(a, stream);
    if (mt == 3) return launch_slab<PRO, EPI, 3>(a, stream);
    return launch_slab<PRO, EPI, 4>(a, stream);
}

template <int EPI, int PRO = PRO_BF16>
int dispatch_wide(const SkinnyArgs &a, hipStream_t stream) {
    const int mt = (a.M + 15) / 16;
    if (mt == 2) return launch_wide<2, EPI, PRO>(a, stream);
    if (mt == 3) return launch_wide<3, EPI, PRO>(a, stream);
    if (mt == 4) return launch_wide<4, EPI, PRO>(a, stream);
    // 65 to 128 rows: five to eight row tiles, from the tile-major copies only, for the feed-forward's two products (the
    // GEMM library's down projection of this many rows leaves half of the device idle; its other products are as fast)
    if constexpr (PRO == PRO_BF16 && (EPI == EPI_ADD || EPI == EPI_SWIGLU)) {
        if (mt == 5) return launch_wide<5, EPI, PRO>(a, stream);
        if (mt == 6) return launch_wide<6, EPI, PRO>(a, stream);
        if (mt == 7) return launch_wide<7, EPI, PRO>(a, stream);
        if (mt == 8) return launch_wide<8, EPI, PRO>(a, stream);
    }
    return 1;
}

template <int PRO, int EPI>
int dispatch(const SkinnyArgs &a, hipStream_t stream) {
    const int mt = (a.M + 15) / 16;
    if (mt == 1) return launch_resident<PRO, EPI>(a, stream);
    // Two kernels serve 17 to 64 rows.  The slab kernel (a K slice of the activations resident in LDS, partial sums
    // handed over between workgroups) wins where a matrix has few rows, so that row groups alone would not fill the
    // device (output and down projections: 20 against 32 us and 42 against 51 us at 64 rows of the 8B sizes), and it has
    // the forms with a norm prologue and the q/k/v epilogue.  The chunk kernel wins on matrices of many rows (gate/up:
    // 58 against 69 us), where slices only cost.  "linear.slab" 0 / 2 force one of them where both can serve.
    constexpr bool kChunkCan = PRO == PRO_BF16 && (EPI == EPI_STORE || EPI == EPI_STORE_F32 || EPI == EPI_ADD || EPI == EPI_SWIGLU);
    const int n_out = EPI == EPI_SWIGLU ? a.N / 2 : a.N;
    const int pick = fllm_option_slab();
    const bool slab_first = !kChunkCan || pick == 2 || (pick == 1 && n_out <= 8192);
    if (slab_first) {
        const int rc = dispatch_slab<PRO, EPI>(a, stream);
        if (rc != 1) return rc;
    }
    if constexpr (kChunkCan) return dispatch_wide<EPI>(a, stream);
    return 1;   // the forms with a norm prologue and the q/k/v epilogue need the slab kernel from 17 rows on
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// The decode-shaped product of fllm_linear.  0: launched, negative: error, 1: shape declined.
int fllm_linear_bf16_skinny(const void *x, int ldx, const void *w, const float *bias, void *out, int ldo, int M, int N,
                            int K, int out_mode, hipStream_t stream, const void *w_tiles) {
    if (M > 64 || K % 8 != 0 || ldx % 8 != 0 || !aligned16(x) || !aligned16(w)) return 1;
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = ldx;
    a.w = (const bf16_t *)w;
    a.w_tiles = M <= 16 && out_mode == 1 ? (const bf16_t *)w_tiles : nullptr;     // the form that streams it
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
extern "C" int fllm_fused_decode_supported(int M, int K) {
    return (M >= 1 && M <= 64 && K % 8 == 0 && K >= 8 && K <= 65536) ? 1 : 0;
}

extern "C" int fllm_norm_linear(const float *x, const float *norm_w, float eps, const void *w, const float *bias, void *out,
                                int M, int N, int K, hipStream_t stream) {
    FLLM_REQUIRE(fllm_fused_decode_supported(M, K), "norm_linear: takes 1..64 rows and K a multiple of 8 (M=%d K=%d)", M, K);
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
    FLLM_REQUIRE(fllm_fused_decode_supported(M, K), "norm_gate_up_swiglu: takes 1..64 rows and K a multiple of 8 (M=%d K=%d)", M, K);
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

extern "C" int fllm_gate_up_swiglu(const void *x, int ldx, const void *w_gate_up, const float *bias, void *out, int M,
                                   int inter, int K, hipStream_t stream) {
    FLLM_REQUIRE(M >= 1 && M <= 64 && K % 8 == 0 && K >= 8 && ldx % 8 == 0 && inter > 0,
                 "gate_up_swiglu: takes 1..64 rows and K, ldx in steps of 8 (M=%d K=%d ldx=%d)", M, K, ldx);
    FLLM_REQUIRE(aligned16(x) && aligned16(w_gate_up), "gate_up_swiglu: operands must be 16-byte aligned");
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = ldx;
    a.w = (const bf16_t *)w_gate_up;
    a.bias = bias;
    a.out = out;
    a.ldo = inter;
    a.M = M;
    a.N = 2 * inter;
    a.K = K;
    const int rc = dispatch<PRO_BF16, EPI_SWIGLU>(a, stream);
    FLLM_REQUIRE(rc != 1, "gate_up_swiglu: shape M=%d K=%d does not fit", M, K);
    return rc;
}

namespace {
// the arguments of the q/k/v forms, whatever their prologue
SkinnyArgs qkv_args(const void *x, float eps, const void *w_qkv, const float *bias, void *q_out, const int32_t *row_pos,
                    const int32_t *row_seg, const int32_t *tables, int table_stride, const float *cos_table,
                    const float *sin_table, int rope_dims, void *k_pages, void *v_pages, int M, int heads, int kv_heads,
                    int head_dim, int K, int page_size, int store_kv) {
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = K;
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
    return a;
}
}  // namespace

extern "C" int fllm_norm_qkv_rope_store(const float *x, const float *norm_w, float eps, const void *w_qkv, const float *bias,
                                        void *q_out, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                                        int table_stride, const float *cos_table, const float *sin_table, int rope_dims,
                                        void *k_pages, void *v_pages, int M, int heads, int kv_heads, int head_dim, int K,
                                        int page_size, int store_kv, hipStream_t stream) {
    FLLM_REQUIRE(fllm_fused_decode_supported(M, K), "norm_qkv_rope_store: takes 1..64 rows and K a multiple of 8 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(aligned16(x) && aligned16(w_qkv) && aligned16(norm_w), "norm_qkv_rope_store: operands must be 16-byte aligned");
    FLLM_REQUIRE(head_dim % 8 == 0 && rope_dims % 2 == 0 && rope_dims <= head_dim && rope_dims >= 0,
                 "norm_qkv_rope_store: head_dim %d must be a multiple of 8 and rope_dims %d even and no larger", head_dim, rope_dims);
    FLLM_REQUIRE(heads > 0 && kv_heads > 0 && page_size > 0 && table_stride > 0 && eps > 0.f, "norm_qkv_rope_store: bad sizes");
    FLLM_REQUIRE(!store_kv || (k_pages && v_pages), "norm_qkv_rope_store: pages missing");
    SkinnyArgs a = qkv_args(x, eps, w_qkv, bias, q_out, row_pos, row_seg, tables, table_stride, cos_table, sin_table, rope_dims,
                            k_pages, v_pages, M, heads, kv_heads, head_dim, K, page_size, store_kv);
    a.norm_w = norm_w;
    const int rc = dispatch<PRO_NORM_F32, EPI_QKV>(a, stream);
    FLLM_REQUIRE(rc != 1, "norm_qkv_rope_store: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

// ---------------------------------------------------------------------------------------------
// A norm prepared by the product before it (up to 16 rows)
// ---------------------------------------------------------------------------------------------
// out += x w^T as fllm_linear does with a float32 `out`, and for the RMSNorm that reads `out` next: next_x = out *
// next_w as bfloat16 [M, N], and next_ssq [M, *tiles_out] the sums of squares of out over the outputs of each tile
// (room for M * N / 8 floats).  *tiles_out (host memory) says how many parts a row has.
extern "C" int fllm_weight_tiles_supported(int N, int K) { return tiles_fit(N, K) ? 1 : 0; }

extern "C" size_t fllm_weight_tiles_elements(int N, int K) { return (size_t)((N + 15) / 16) * 16 * (size_t)K; }

extern "C" int fllm_tile_weights(const void *w, void *tiles, int N, int K, hipStream_t stream) {
    FLLM_REQUIRE(tiles_fit(N, K), "tile_weights: takes matrices of at least 16 rows whose width is a multiple of 1,024 (N=%d K=%d)", N, K);
    FLLM_REQUIRE(w != nullptr && tiles != nullptr && aligned16(w) && aligned16(tiles), "tile_weights: operands must be there and 16-byte aligned");
    const size_t pieces = fllm_weight_tiles_elements(N, K) / 8;
    const size_t want = (pieces + 255) / 256;
    hipLaunchKernelGGL(tile_weights_kernel, dim3((unsigned int)(want < 65536 ? want : 65536)), dim3(256), 0, stream, (const bf16_t *)w,
                       (bf16_t *)tiles, N, K, pieces, 0);
    return fllm_check_launch("tile_weights");
}

extern "C" size_t fllm_weight_tiles_elements_gate_up(int inter, int K) { return (size_t)((inter + 7) / 8) * 16 * (size_t)K; }

// The copy for the gate/up product with its SwiGLU epilogue: w is [2 inter][K], gate rows first.
extern "C" int fllm_tile_weights_gate_up(const void *w, void *tiles, int inter, int K, hipStream_t stream) {
    FLLM_REQUIRE(tiles_fit(2 * inter, K), "tile_weights_gate_up: takes matrices whose width is a multiple of 1,024 (inter=%d K=%d)", inter, K);
    FLLM_REQUIRE(w != nullptr && tiles != nullptr && aligned16(w) && aligned16(tiles), "tile_weights_gate_up: operands must be there and 16-byte aligned");
    const size_t pieces = fllm_weight_tiles_elements_gate_up(inter, K) / 8;
    const size_t want = (pieces + 255) / 256;
    hipLaunchKernelGGL(tile_weights_kernel, dim3((unsigned int)(want < 65536 ? want : 65536)), dim3(256), 0, stream, (const bf16_t *)w,
                       (bf16_t *)tiles, 2 * inter, K, pieces, inter);
    return fllm_check_launch("tile_weights_gate_up");
}

// fllm_gate_up_swiglu for 17..64 rows with the weights' tile-major copy (fllm_tile_weights_gate_up; may be null)
extern "C" int fllm_gate_up_swiglu_tiled(const void *x, int ldx, const void *w_gate_up, const void *w_tiles, const float *bias, void *out,
                                         int M, int inter, int K, hipStream_t stream) {
    FLLM_REQUIRE(M >= 17 && M <= kWideRows && K % 8 == 0 && K >= 8 && ldx % 8 == 0 && inter > 0,
                 "gate_up_swiglu_tiled: takes 17..128 rows and K, ldx in steps of 8 (M=%d K=%d ldx=%d)", M, K, ldx);
    FLLM_REQUIRE(M <= 64 || (w_tiles != nullptr && K % 256 == 0), "gate_up_swiglu_tiled: beyond 64 rows it takes the tile-major copy and K in steps of 256 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(aligned16(x) && aligned16(w_gate_up) && (w_tiles == nullptr || aligned16(w_tiles)),
                 "gate_up_swiglu_tiled: operands must be 16-byte aligned");
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = ldx;
    a.w = (const bf16_t *)w_gate_up;
    a.w_tiles = (const bf16_t *)w_tiles;
    a.bias = bias;
    a.out = out;
    a.ldo = inter;
    a.M = M;
    a.N = 2 * inter;
    a.K = K;
    return dispatch_wide<EPI_SWIGLU>(a, stream);
}

// out += x w^T (+ bias) for 1..16 bfloat16 rows and a float32 `out`, as fllm_linear in mode 2; `w_tiles` (may be null):
// the tile-major copy of w, which the kernel streams instead where the launch it chooses can.
extern "C" int fllm_linear_add_tiled(const void *x, int ldx, const void *w, const void *w_tiles, const float *bias, float *out, int ldo,
                                     int M, int N, int K, hipStream_t stream) {
    FLLM_REQUIRE(M >= 1 && M <= kWideRows && K % 8 == 0 && K >= 8 && ldx % 8 == 0 && ldx >= K && ldo >= N,
                 "linear_add_tiled: takes 1..128 rows, K and ldx in steps of 8 (M=%d N=%d K=%d ldx=%d ldo=%d)", M, N, K, ldx, ldo);
    FLLM_REQUIRE(M <= 64 || (w_tiles != nullptr && K % 256 == 0), "linear_add_tiled: beyond 64 rows it takes the tile-major copy and K in steps of 256 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(aligned16(x) && aligned16(w) && out != nullptr && (w_tiles == nullptr || aligned16(w_tiles)),
                 "linear_add_tiled: operands must be there and 16-byte aligned");
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = ldx;
    a.w = (const bf16_t *)w;
    a.w_tiles = (const bf16_t *)w_tiles;
    a.bias = bias;
    a.out = out;
    a.ldo = ldo;
    a.M = M;
    a.N = N;
    a.K = K;
    const int rc = M <= 16 ? launch_resident<PRO_BF16, EPI_ADD>(a, stream) : dispatch_wide<EPI_ADD>(a, stream);
    FLLM_REQUIRE(rc != 1, "linear_add_tiled: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

// out = x w^T (+ bias) for 1..64 bfloat16 rows and a float32 `out` (the vocabulary projection of a decode step), as
// fllm_linear in mode 1, from the tile-major copy of w where the launch it chooses can stream it.
extern "C" int fllm_linear_f32_tiled(const void *x, int ldx, const void *w, const void *w_tiles, const float *bias, float *out, int ldo,
                                     int M, int N, int K, hipStream_t stream) {
    FLLM_REQUIRE(M >= 1 && M <= 64 && K % 8 == 0 && K >= 8 && ldx % 8 == 0 && ldx >= K && ldo >= N,
                 "linear_f32_tiled: takes 1..64 rows, K and ldx in steps of 8 (M=%d N=%d K=%d ldx=%d ldo=%d)", M, N, K, ldx, ldo);
    FLLM_REQUIRE(aligned16(x) && aligned16(w) && out != nullptr && (w_tiles == nullptr || aligned16(w_tiles)),
                 "linear_f32_tiled: operands must be there and 16-byte aligned");
    if (M > 16) {
        SkinnyArgs a = {};
        a.x = x;
        a.ldx = ldx;
        a.w = (const bf16_t *)w;
        a.w_tiles = (const bf16_t *)w_tiles;
        a.bias = bias;
        a.out = out;
        a.ldo = ldo;
        a.M = M;
        a.N = N;
        a.K = K;
        return dispatch_wide<EPI_STORE_F32>(a, stream);
    }
    const int rc = fllm_linear_bf16_skinny(x, ldx, w, bias, out, ldo, M, N, K, 1, stream, w_tiles);
    FLLM_REQUIRE(rc != 1, "linear_f32_tiled: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

extern "C" int fllm_linear_add_normed(const void *x, int ldx, const void *w, const float *bias, float *out, int M, int N, int K,
                                      const float *next_w, void *next_x, float *next_ssq, int *tiles_out, const void *w_tiles,
                                      hipStream_t stream) {
    FLLM_REQUIRE(M >= 1 && M <= kWideRows && K % 8 == 0 && K >= 8 && ldx % 8 == 0 && N >= 16 && N % 16 == 0,
                 "linear_add_normed: takes 1..128 rows, K and ldx in steps of 8 and N in steps of 16 (M=%d N=%d K=%d ldx=%d)", M, N, K, ldx);
    FLLM_REQUIRE(M <= 64 || (w_tiles != nullptr && K % 256 == 0), "linear_add_normed: beyond 64 rows it takes the tile-major copy and K in steps of 256 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(aligned16(x) && aligned16(w) && aligned16(out) && aligned16(next_w) && next_x != nullptr && next_ssq != nullptr &&
                     ((uintptr_t)next_x & 7) == 0 && tiles_out != nullptr && (w_tiles == nullptr || aligned16(w_tiles)),
                 "linear_add_normed: operands must be there and 16-byte aligned");
    SkinnyArgs a = {};
    a.x = x;
    a.ldx = ldx;
    a.w = (const bf16_t *)w;
    a.w_tiles = (const bf16_t *)w_tiles;
    a.bias = bias;
    a.out = out;
    a.ldo = N;
    a.M = M;
    a.N = N;
    a.K = K;
    a.next_w = next_w;
    a.next_x = (bf16_t *)next_x;
    a.next_ssq = next_ssq;
    a.next_tiles_out = tiles_out;
    const int rc = M <= 16 ? launch_resident<PRO_BF16, EPI_ADD>(a, stream) : dispatch_wide<EPI_ADD>(a, stream);
    FLLM_REQUIRE(rc != 1, "linear_add_normed: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

// The forms with a norm prologue, from what fllm_linear_add_normed left: xn [M, K] bfloat16, ssq [M, ssq_count].
// From 17 rows on they need the weights' tile-major copy (`w_tiles`, of fllm_tile_weights_gate_up and fllm_tile_weights) and
// K in steps of 256.
extern "C" int fllm_scaled_gate_up_swiglu(const void *xn, const float *ssq, int ssq_count, float eps, const void *w_gate_up,
                                          const float *bias, void *out, int M, int inter, int K, const void *w_tiles,
                                          hipStream_t stream) {
    FLLM_REQUIRE(M >= 1 && M <= 64 && K % 8 == 0 && K >= 8 && inter > 0 && ssq_count > 0 && eps > 0.f,
                 "scaled_gate_up_swiglu: takes 1..64 rows and K a multiple of 8 (M=%d K=%d parts=%d)", M, K, ssq_count);
    FLLM_REQUIRE(aligned16(xn) && aligned16(w_gate_up) && ssq != nullptr && (w_tiles == nullptr || aligned16(w_tiles)),
                 "scaled_gate_up_swiglu: operands must be 16-byte aligned");
    FLLM_REQUIRE(M <= 16 || (w_tiles != nullptr && K % 256 == 0),
                 "scaled_gate_up_swiglu: from 17 rows on it takes the tile-major copy and K in steps of 256 (M=%d K=%d)", M, K);
    SkinnyArgs a = {};
    a.x = xn;
    a.ldx = K;
    a.eps = eps;
    a.ssq_in = ssq;
    a.ssq_count = ssq_count;
    a.w = (const bf16_t *)w_gate_up;
    a.bias = bias;
    a.out = out;
    a.ldo = inter;
    a.M = M;
    a.N = 2 * inter;
    a.K = K;
    a.w_tiles = (const bf16_t *)w_tiles;
    if (M > 16) return dispatch_wide<EPI_SWIGLU, PRO_SCALED>(a, stream);
    const int rc = launch_resident<PRO_SCALED, EPI_SWIGLU>(a, stream);
    FLLM_REQUIRE(rc != 1, "scaled_gate_up_swiglu: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

extern "C" int fllm_scaled_qkv_rope_store(const void *xn, const float *ssq, int ssq_count, float eps, const void *w_qkv,
                                          const float *bias, void *q_out, const int32_t *row_pos, const int32_t *row_seg,
                                          const int32_t *tables, int table_stride, const float *cos_table, const float *sin_table,
                                          int rope_dims, void *k_pages, void *v_pages, int M, int heads, int kv_heads, int head_dim,
                                          int K, int page_size, int store_kv, const void *w_tiles, hipStream_t stream) {
    FLLM_REQUIRE(M >= 1 && M <= 64 && K % 8 == 0 && K >= 8 && ssq_count > 0,
                 "scaled_qkv_rope_store: takes 1..64 rows and K a multiple of 8 (M=%d K=%d parts=%d)", M, K, ssq_count);
    FLLM_REQUIRE(aligned16(xn) && aligned16(w_qkv) && ssq != nullptr && (w_tiles == nullptr || aligned16(w_tiles)),
                 "scaled_qkv_rope_store: operands must be 16-byte aligned");
    FLLM_REQUIRE(M <= 16 || (w_tiles != nullptr && K % 256 == 0),
                 "scaled_qkv_rope_store: from 17 rows on it takes the tile-major copy and K in steps of 256 (M=%d K=%d)", M, K);
    FLLM_REQUIRE(head_dim % 8 == 0 && rope_dims % 2 == 0 && rope_dims <= head_dim && rope_dims >= 0,
                 "scaled_qkv_rope_store: head_dim %d must be a multiple of 8 and rope_dims %d even and no larger", head_dim, rope_dims);
    FLLM_REQUIRE(heads > 0 && kv_heads > 0 && page_size > 0 && table_stride > 0 && eps > 0.f, "scaled_qkv_rope_store: bad sizes");
    FLLM_REQUIRE(!store_kv || (k_pages && v_pages), "scaled_qkv_rope_store: pages missing");
    SkinnyArgs a = qkv_args(xn, eps, w_qkv, bias, q_out, row_pos, row_seg, tables, table_stride, cos_table, sin_table, rope_dims,
                            k_pages, v_pages, M, heads, kv_heads, head_dim, K, page_size, store_kv);
    a.ssq_in = ssq;
    a.ssq_count = ssq_count;
    a.w_tiles = (const bf16_t *)w_tiles;
    if (M > 16) return dispatch_wide<EPI_QKV, PRO_SCALED>(a, stream);
    const int rc = launch_resident<PRO_SCALED, EPI_QKV>(a, stream);
    FLLM_REQUIRE(rc != 1, "scaled_qkv_rope_store: shape M=%d K=%d does not fit the staging area", M, K);
    return rc;
}

#ifdef FLLM_TIMELINE
// measurement builds only: device memory for [workgroups][8] clock readings of the next resident launches (null: off)
extern "C" void fllm_set_timeline(unsigned long long *buffer) { g_timeline = buffer; }
#endif
