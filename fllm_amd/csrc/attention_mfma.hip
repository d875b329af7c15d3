// Paged causal attention in bfloat16 on the MFMA units of gfx950: scores, softmax statistics
// and output accumulate in float32.
//
// Both kernels compute the TRANSPOSED products, so that a lane keeps one query row throughout:
//   S^T[key][q] = K[key][:] . Q[q][:]          (A = K fragment, B = Q fragment)
//   O^T[d][q]  += V^T[d][key] * P^T[key][q]     (A = V^T fragment, B = P^T fragment)
// With v_mfma_f32_16x16x32_bf16 the result tile D[m = 4*(l/16) + i][n = l%16] leaves lane l with
// four keys of query l%16; the A rows of two consecutive S^T tiles are assigned to keys so that
// these are the keys 8*(l/16) .. 8*(l/16)+7 of a 32-key block, which is exactly the B operand
// layout of the second product: probabilities go from the first MFMA to the second without
// leaving registers, and the running maximum and sum of a query row live in its lanes.
// Values are stored transposed inside a page ([head_dim][token]) so that V^T fragments are
// contiguous 16-byte loads.
//
//   tile kernel    portions of prompts: a workgroup takes up to 64 (token, head-of-group) rows of
//                  one segment and one key/value head; keys and values go through LDS in tiles of 64.
//   tile32 kernel  head sizes 64 and 128: 128 rows per workgroup on 32x32x16 products, the next tile on its way
//                  while the current one is multiplied (described at the kernel); faster than the tile kernel
//                  for portions of any length.  Few rows over long contexts: several workgroups share a row
//                  tile's keys and the one that arrives last adds their parts up.
//   decode kernel  one row per segment: a workgroup takes (row, key/value head, context split), its
//                  sixteen waves stride over 32-key blocks loading K and V^T straight into MFMA
//                  operands; long contexts of small batches are split and merged by a second kernel.
#include <algorithm>
#include "api.h"
#include "common.h"
#include "plans.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr float kLog2e = 1.4426950408889634f;

struct AttnArgs {
    const bf16_t *q;
    int q_stride;
    const bf16_t *kp;
    const bf16_t *vp;
    const int32_t *tables;
    int table_stride;
    const int32_t *row_pos;
    const int32_t *row_seg;
    const int32_t *seg_start;
    int num_segs;
    bf16_t *out;
    int rows, heads, kv_heads, page_size;
    int ps_shift;   // page_size = 1 << ps_shift
    float scale_log2;
    int window;
    float *ws_ml;   // [rows, heads, splits, 2]
    float *ws_o;    // [rows, heads, splits, D]
    int splits, keys_per_split;
    int *counters;  // one per (row, key/value head, query tile), zero between launches: the last split to arrive merges; null: a merge kernel does
    // Prompt portions (tile32 kernel): a row tile with more than part_tiles key tiles is shared by several workgroups
    // (blockIdx.y), each with a stretch of its key tiles; 0: never.  Their partial results meet in `parts_ws`
    // ([row tile][key/value head][part][kPartFloats]) and are counted in `counters` ([row tile][key/value head]).
    int part_tiles;
    float *parts_ws;
};

__device__ __forceinline__ bf16x8_t zero8() {
    bf16x8_t z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16_t)0.0f;
    return z;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// floats that one part of a shared row tile leaves for the merge (tile32 kernel): head_dim / 2 outputs, a maximum
// and a sum for each of its lanes
__host__ __device__ constexpr size_t kPartFloats(int head_dim, int threads) { return fllm_plan::part_floats(head_dim, threads); }

// Online-softmax update of one query row held across the four lane groups of a wave.
// s: NS score tiles (already scaled and masked with -inf); returns the P^T operands.
template <int NS>
__device__ __forceinline__ void softmax_step(f32x4_t (&s)[NS], float &m_run, float &l_run, float &alpha) {
    float tmax = -INFINITY;
#pragma unroll
    for (int t = 0; t < NS; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) tmax = fmaxf(tmax, s[t][i]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m_run, tmax);
    alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(m_run - m_new);
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < NS; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float p = (s[t][i] == -INFINITY) ? 0.f : fast_exp2(s[t][i] - m_new);
            s[t][i] = p;
            psum += p;
        }
    psum += __shfl_xor(psum, 16, kWave);
    psum += __shfl_xor(psum, 32, kWave);
    l_run = l_run * alpha + psum;
    m_run = m_new;
}

__device__ __forceinline__ bf16x8_t pack_p(const f32x4_t &lo, const f32x4_t &hi) {
    bf16x8_t p;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        p[i] = (bf16_t)lo[i];
        p[4 + i] = (bf16_t)hi[i];
    }
    return p;
}

// ---------------------------------------------------------------------------------------------
// tile kernel
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ void __launch_bounds__(kThreads)
attn_tile_kernel(AttnArgs p) {
    constexpr int KT = 64;          // keys per tile
    constexpr int KP = D + 8;       // pitch of a key row in LDS
    constexpr int VP = KT + 8;      // pitch of a value row (one head_dim lane, KT keys) in LDS
    constexpr int KD = D / 32, DT = D / 16;
    __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KP];
    __shared__ __attribute__((aligned(16))) bf16_t Vs[D * VP];
    __shared__ int s_tile[2];
    const int G = p.heads / p.kv_heads;
    const int TQ = 64 / G;          // tokens per tile
    if (threadIdx.x == 0) {
        int b = blockIdx.x, seg = -1, t0 = 0;
        for (int s = 0; s < p.num_segs; s++) {
            const int n = p.seg_start[s + 1] - p.seg_start[s];
            const int nt = (n + TQ - 1) / TQ;
            if (b < nt) {
                seg = s;
                t0 = b;
                break;
            }
            b -= nt;
        }
        s_tile[0] = seg;
        s_tile[1] = t0;
    }
    __syncthreads();
    const int seg = s_tile[0];
    if (seg < 0) return;
    const int row0 = p.seg_start[seg] + s_tile[1] * TQ;
    const int ntok = min(TQ, p.seg_start[seg + 1] - row0);
    const int pos0 = p.row_pos[row0];
    const int kvh = blockIdx.y;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int rr = wave * 16 + c;
    const int tq = rr / G, hg = rr - tq * G;
    const bool rvalid = tq < ntok;
    const int prow = rvalid ? pos0 + tq : -1;
    const int head = kvh * G + hg;
    const int lo_r = (p.window > 0 && prow - p.window + 1 > 0) ? prow - p.window + 1 : 0;
    const int ps = p.page_size, psh = p.ps_shift, pmask = ps - 1, nkv = p.kv_heads;

    bf16x8_t qf[KD];
#pragma unroll
    for (int kk = 0; kk < KD; kk++)
        qf[kk] = rvalid ? *(const bf16x8_t *)(p.q + (size_t)(row0 + tq) * p.q_stride + (size_t)head * D + kk * 32 + g * 8)
                        : zero8();

    const int p_last = pos0 + ntok - 1;
    const int lo_tile = (p.window > 0 && pos0 - p.window + 1 > 0) ? pos0 - p.window + 1 : 0;
    const int kbegin = (lo_tile / KT) * KT;
    const int32_t *tbl = p.tables + (size_t)seg * p.table_stride;
    const int cps = psh - 3;   // log2 of the 16-byte chunks per value row of a page
    constexpr int LD = D == 32 ? 5 : D == 64 ? 6 : 7;   // log2(D)

    f32x4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) o[dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    for (int k0 = kbegin; k0 <= p_last; k0 += KT) {
        __syncthreads();   // the previous tile has been read
        for (int ch = threadIdx.x; ch < KT * D / 8; ch += kThreads) {
            // the chunks in the order in which they lie in a page: token fastest, then the key's chunks, then the tile's pages
            const int wsh = psh < 6 ? psh : 6;           // log2 of the tokens of a page that lie in this tile (KT is 64)
            const int key = ((ch >> (wsh + LD - 3)) << wsh) | (ch & ((1 << wsh) - 1)), dc = (ch >> wsh) & (D / 8 - 1);
            const int kabs = k0 + key;
            bf16x8_t v = zero8();
            if (kabs >= lo_tile && kabs <= p_last) {
                const int page = tbl[kabs >> psh], off = kabs & pmask;
                v = *(const bf16x8_t *)(p.kp + key_offset(page, nkv, kvh, ps, D, off, dc * 8));
            }
            *(bf16x8_t *)(Ks + key * KP + dc * 8) = v;
        }
        for (int ch = threadIdx.x; ch < D * KT / 8; ch += kThreads) {
            const int pg = ch >> (LD + cps), rem = ch & ((D << cps) - 1);
            const int d = rem >> cps, hc = rem & ((1 << cps) - 1);
            const int koff = (pg << psh) + hc * 8;
            const int kabs = k0 + koff;
            bf16x8_t v = zero8();
            if (kabs + 7 >= lo_tile && kabs <= p_last) {
                const int page = tbl[kabs >> psh];
                v = *(const bf16x8_t *)(p.vp + (((size_t)page * nkv + kvh) * D + d) * ps + hc * 8);
                if (kabs + 7 > p_last) {   // slots past the last token hold whatever an earlier request left
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (kabs + e > p_last) v[e] = (bf16_t)0.0f;
                }
            }
            *(bf16x8_t *)(Vs + d * VP + koff) = v;
        }
        __syncthreads();

        f32x4_t s[4];
#pragma unroll
        for (int st = 0; st < 4; st++) {
            s[st] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            const int kb = st >> 1, j = st & 1;
            const int key_local = kb * 32 + (c >> 2) * 8 + j * 4 + (c & 3);   // A row c of this tile
#pragma unroll
            for (int kk = 0; kk < KD; kk++) {
                const bf16x8_t a = *(const bf16x8_t *)(Ks + key_local * KP + kk * 32 + g * 8);
                s[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[kk], s[st], 0, 0, 0);
            }
        }
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const int kb = st >> 1, j = st & 1;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = k0 + kb * 32 + g * 8 + j * 4 + i;
                const bool vis = key <= prow && key >= lo_r;   // prow = -1 for rows outside the segment
                s[st][i] = vis ? s[st][i] * p.scale_log2 : -INFINITY;
            }
        }
        float alpha;
        softmax_step<4>(s, m_run, l_run, alpha);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) o[dt] *= alpha;
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            const bf16x8_t pf = pack_p(s[kb * 2], s[kb * 2 + 1]);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                const bf16x8_t a = *(const bf16x8_t *)(Vs + (dt * 16 + c) * VP + kb * 32 + g * 8);
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf, o[dt], 0, 0, 0);
            }
        }
    }
    if (rvalid) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        bf16_t *dst = p.out + ((size_t)(row0 + tq) * p.heads + head) * D + g * 4;
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            bf16x4_t v;
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = (bf16_t)(o[dt][i] * inv);
            *(bf16x4_t *)(dst + dt * 16) = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// tile kernel on 32x32x16 products: 128 or 256 (token, head-of-group) rows per workgroup
// ---------------------------------------------------------------------------------------------
// v_mfma_f32_32x32x16_bf16: A lane l holds A[m = l%32][k = 8*(l/32) .. +7], B lane l holds
// B[k = 8*(l/32) .. +7][n = l%32], D lane l holds D[m = 8*(i/4) + 4*(l/32) + i%4][n = l%32], i = 0..15.
// A wave owns 32 query rows (n).  The A rows of a 32-key block of S^T are assigned to keys so that
// the sixteen sums of a lane, taken eight at a time, are the keys 16 s + 8 (l/32) .. + 7: the B
// operand of the P V product for that half block, with no exchange between lanes:
//   A row a = 16 s + 8 b + 4 h + i  <->  key 16 s + 8 h + 4 b + i      (s, b, h in {0, 1}, i in 0..3)
// Each K and V fragment read from LDS feeds 32 query rows instead of 16, the next tile is on its way
// from global memory into registers while the current one is multiplied, the scale is folded into
// the exponent (one fused multiply-add per score), tiles wholly below the diagonal skip the mask,
// and the outputs are rescaled only when a row's maximum moved.
// WAVES: 4 (128 rows a workgroup, two workgroups a compute unit) or 8 (256 rows, one workgroup a compute unit: a key or
// value fetched from L2 serves twice the rows; 128 rows over 16,384 keys ask L2 for 6.9 TB/s, which is about what it
// hands to the compute units).
template <int D, int WAVES>
__global__ void __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
attn_tile32_kernel(AttnArgs p) {
    constexpr int THREADS = WAVES * kWave;
    constexpr int KT = 64;          // keys per tile
    constexpr int KP = D + 8;       // pitch of a key row in LDS
    constexpr int VP = KT + 8;      // pitch of a value row (one head_dim lane, KT keys) in LDS
    constexpr int DS = D / 16, DB = D / 32;
    constexpr int CH = KT * D / 8 / THREADS;   // 16-byte chunks per thread and tile (K and V each)
    constexpr int LD = D == 64 ? 6 : 7;         // log2(D)
    static_assert(CH >= 1 && (D == 64 || D == 128), "this tiling takes head_dim 64 or 128");
    __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KP];
    __shared__ __attribute__((aligned(16))) bf16_t Vs[D * VP];
    __shared__ int s_tile[2];
    const int G = p.heads / p.kv_heads;
    const int TQ = WAVES * 32 / G;  // tokens per tile
    // blockIdx.x = (row tile, key/value head), the head fastest: workgroups start in the order of their row tiles,
    // longest contexts first, whatever their head, and with 8 heads each of the 8 dies sees the keys of one head only
    const int group = blockIdx.x;
    if (threadIdx.x == 0) {
        int b = group / p.kv_heads, seg = -1, t0 = 0;
        for (int s = 0; s < p.num_segs; s++) {
            const int n = p.seg_start[s + 1] - p.seg_start[s];
            const int nt = (n + TQ - 1) / TQ;
            if (b < nt) {
                seg = s;
                t0 = nt - 1 - b;    // the tiles with the longest contexts start first
                break;
            }
            b -= nt;
        }
        s_tile[0] = seg;
        s_tile[1] = t0;
    }
    __syncthreads();
    const int seg = s_tile[0];
    if (seg < 0) return;
    const int row0 = p.seg_start[seg] + s_tile[1] * TQ;
    const int ntok = min(TQ, p.seg_start[seg + 1] - row0);
    const int pos0 = p.row_pos[row0];
    const int kvh = group % p.kv_heads;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int q = lane & 31, h = lane >> 5;
    const int rr = wave * 32 + q;
    const int tq = rr / G, hg = rr - tq * G;
    const bool rvalid = tq < ntok;
    const int prow = rvalid ? pos0 + tq : -1;
    const int head = kvh * G + hg;
    const int lo_r = (p.window > 0 && prow - p.window + 1 > 0) ? prow - p.window + 1 : 0;
    const int ps = p.page_size, psh = p.ps_shift, pmask = ps - 1, nkv = p.kv_heads;
    const int cps = psh - 3;        // log2 of the 16-byte chunks per value row of a page

    bf16x8_t qf[DS];
#pragma unroll
    for (int ds = 0; ds < DS; ds++)
        qf[ds] = rvalid ? *(const bf16x8_t *)(p.q + (size_t)(row0 + tq) * p.q_stride + (size_t)head * D + ds * 16 + h * 8)
                        : zero8();

    const int p_last = pos0 + ntok - 1;
    const int lo_tile = (p.window > 0 && pos0 - p.window + 1 > 0) ? pos0 - p.window + 1 : 0;
    // from this key on every row of the workgroup sees every key up to pos0 (no window edge inside)
    const int lo_all = (p.window > 0 && p_last - p.window + 1 > 0) ? p_last - p.window + 1 : 0;
    int kbegin = (lo_tile / KT) * KT;
    // Long contexts of few rows: the key tiles of this row tile are dealt out to `parts` workgroups in equal
    // stretches; a workgroup beyond that number has nothing to do.
    int parts = 1, k_stop = p_last;    // k_stop: the last key of this workgroup's stretch
    if (p.part_tiles > 0) {
        const int nkt = (p_last - kbegin) / KT + 1;
        parts = min((nkt + p.part_tiles - 1) / p.part_tiles, (int)gridDim.y);
        const int part = blockIdx.y;
        if (part >= parts) return;
        const int base = nkt / parts, rem = nkt - base * parts;
        const int first_tile = part * base + min(part, rem), count = base + (part < rem ? 1 : 0);
        kbegin += first_tile * KT;
        k_stop = min(p_last, kbegin + count * KT - 1);
    }
    const int32_t *tbl = p.tables + (size_t)seg * p.table_stride;

    // What of a chunk's address does not change from tile to tile (tiles start at multiples of 64 >= page size)
    int k_key[CH], v_koff[CH], k_in_page[CH], v_in_page[CH], k_lds[CH], v_lds[CH];
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int ch = threadIdx.x + c * THREADS;
        // the chunks in the order in which they lie in a page (token fastest, then the key's chunks, then the tile's pages):
        // a load instruction of a wave reads 1 KiB in a row where a page holds 16 tokens or more
        const int wsh = psh < 6 ? psh : 6;               // log2 of the tokens of a page that lie in this tile (KT is 64)
        const int key = ((ch >> (wsh + LD - 3)) << wsh) | (ch & ((1 << wsh) - 1)), dc = (ch >> wsh) & (D / 8 - 1);
        k_key[c] = key;
        k_in_page[c] = (int)key_offset(0, nkv, kvh, ps, D, key & pmask, dc * 8);
        // A key's row in LDS: bits 2 and 3 of the key swapped, which is where the products read it (row q of a 32-key
        // block is key 16 (q / 16) + 8 (q / 4 % 2) + 4 (q / 8 % 2) + q % 4, see the table above, and that map is this swap): the 8 lanes of a 128-byte LDS access then read 8
        // consecutive rows, 16 bytes further along the banks each, instead of hitting every bank twice.
        k_lds[c] = ((key & ~12) | ((key & 4) << 1) | ((key & 8) >> 1)) * KP + dc * 8;
        const int pg = ch >> (LD + cps), rem = ch & ((D << cps) - 1);
        const int d = rem >> cps, hc = rem & ((1 << cps) - 1);
        v_koff[c] = (pg << psh) + hc * 8;
        v_in_page[c] = (kvh * D + d) * ps + hc * 8;
        v_lds[c] = d * VP + v_koff[c];
    }
    const unsigned page_elems = (unsigned)nkv * ps * D;   // the host has checked that it fits

    bf16x8_t kreg[CH], vreg[CH];
    // A tile's loads depend on its page numbers: those are asked for one tile earlier than the tile's keys and
    // values, which are asked for one tile before they are multiplied, so neither wait lies on the path.
    // Tiles with no edge of the context inside (all but the first of a window and the last one or two) take the
    // branch without a condition per lane: the address arithmetic of a tile is a few instructions a chunk.
    int pgk[CH], pgv[CH];
    auto pages = [&](int k0) {   // page numbers of tile k0 .. k0 + 63 (0 where the tile has no token)
        if (k0 > k_stop) return;
        if (k0 >= lo_tile && k0 + KT - 1 <= p_last) {
            const int32_t *t = tbl + (k0 >> psh);
#pragma unroll
            for (int c = 0; c < CH; c++) {
                pgk[c] = t[k_key[c] >> psh];
                pgv[c] = t[v_koff[c] >> psh];
            }
            return;
        }
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int kabs = k0 + k_key[c], vabs = k0 + v_koff[c];
            pgk[c] = (kabs >= lo_tile && kabs <= p_last) ? tbl[kabs >> psh] : 0;
            pgv[c] = (vabs + 7 >= lo_tile && vabs <= p_last) ? tbl[vabs >> psh] : 0;
        }
    };
    auto fetch = [&](int k0) {   // tile k0 .. k0 + 63 from the pages into registers; pages(k0) has run
        if (k0 >= lo_tile && k0 + KT - 1 <= p_last) {
#pragma unroll
            for (int c = 0; c < CH; c++) {
                kreg[c] = *(const bf16x8_t *)(p.kp + ((size_t)(unsigned)pgk[c] * page_elems + (unsigned)k_in_page[c]));
                vreg[c] = *(const bf16x8_t *)(p.vp + ((size_t)(unsigned)pgv[c] * page_elems + (unsigned)v_in_page[c]));
            }
            return;
        }
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int kabs = k0 + k_key[c];
            bf16x8_t v = zero8();
            if (kabs >= lo_tile && kabs <= p_last)
                v = *(const bf16x8_t *)(p.kp + ((size_t)(unsigned)pgk[c] * page_elems + (unsigned)k_in_page[c]));
            kreg[c] = v;
            const int vabs = k0 + v_koff[c];
            v = zero8();
            if (vabs + 7 >= lo_tile && vabs <= p_last) {
                v = *(const bf16x8_t *)(p.vp + ((size_t)(unsigned)pgv[c] * page_elems + (unsigned)v_in_page[c]));
                if (vabs + 7 > p_last) {   // slots past the last token hold whatever an earlier request left
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (vabs + e > p_last) v[e] = (bf16_t)0.0f;
                }
            }
            vreg[c] = v;
        }
    };

    f32x16_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;   // the running maximum is kept in raw units (before the scale)
    const float sc = p.scale_log2;
    const float tau = 8.0f / sc;

    pages(kbegin);
    fetch(kbegin);
    pages(kbegin + KT);
    for (int k0 = kbegin; k0 <= k_stop; k0 += KT) {
        __syncthreads();   // the previous tile has been read
#pragma unroll
        for (int c = 0; c < CH; c++) {
            *(bf16x8_t *)(Ks + k_lds[c]) = kreg[c];
            *(bf16x8_t *)(Vs + v_lds[c]) = vreg[c];
        }
        __syncthreads();
        if (k0 + KT <= k_stop) {   // in flight while this tile is multiplied
            fetch(k0 + KT);
            pages(k0 + 2 * KT);
        }

        f32x16_t s[2];
#pragma unroll
        for (int rb = 0; rb < 2; rb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) s[rb][i] = 0.f;
            const bf16_t *krow = Ks + (rb * 32 + q) * KP + h * 8;
#pragma unroll
            for (int ds = 0; ds < DS; ds++)
                s[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t *)(krow + ds * 16), qf[ds], s[rb], 0, 0, 0);
        }
        // Tiles wholly below the diagonal and above every window edge need no mask (the same for all rows here).
        // Key k0 + c + 8 h of the others is visible if lo_r <= key <= prow: the constant c is compared with limits
        // that hold everything else.
        if (!(k0 + KT - 1 <= pos0 && k0 >= lo_all)) {
            asm volatile("" ::: "memory");   // a branch of its own: folded into selects it would run for every tile
            const int hi_lim = prow - k0 - 8 * h, lo_lim = lo_r - k0 - 8 * h;   // prow = -1 for rows outside the segment
#pragma unroll
            for (int rb = 0; rb < 2; rb++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int c = rb * 32 + 16 * (i >> 3) + (i & 7);
                    if (!(c <= hi_lim && c >= lo_lim)) s[rb][i] = -INFINITY;
                }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[rb][i]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
        // The reference point of the exponents follows the maximum only when that has grown by more than 2^8 in the
        // exponent's units: until then the probabilities are at most 256 times their final size, which float32 sums and
        // bfloat16 operands hold as well, and the outputs need no rescaling (with it at every new maximum, short
        // contexts rescaled in most tiles).
        const float m_new = tmax > m_run + tau ? tmax : m_run;
        const float mc = m_new == -INFINITY ? 0.f : m_new * sc;   // nothing seen yet: exp2(-inf - 0) = 0 below
        const float alpha = m_run == -INFINITY ? 0.f : fast_exp2(m_run * sc - mc);
        float psum = 0.f;
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float pv = fast_exp2(fmaf(s[rb][i], sc, -mc));   // masked: exp2(-inf) = 0
                s[rb][i] = pv;
                psum += pv;
            }
        psum += __shfl_xor(psum, 32, kWave);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__any(alpha != 1.0f)) {   // once the maximum has settled the outputs need no rescaling
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[db][i] *= alpha;
        }
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                bf16x8_t pf;
#pragma unroll
                for (int e = 0; e < 8; e++) pf[e] = (bf16_t)s[rb][8 * s2 + e];
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    const bf16x8_t a = *(const bf16x8_t *)(Vs + (db * 32 + q) * VP + rb * 32 + 16 * s2 + 8 * h);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf, o[db], 0, 0, 0);
                }
            }
    }
    if (parts > 1) {
        // Every part leaves its maximum, sum and unnormalized outputs at the device's point of coherence, each lane
        // its own values (the parts share the assignment of rows to lanes); the part that arrives last adds them up
        // in the order of the parts, so the result does not depend on which one that is.
        __shared__ int s_seen;
        float *slot = p.parts_ws + (size_t)group * gridDim.y * kPartFloats(D, THREADS);
        float *mine = slot + (size_t)blockIdx.y * kPartFloats(D, THREADS);
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++)
                __hip_atomic_store(mine + (db * 16 + i) * THREADS + threadIdx.x, o[db][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + DB * 16 * THREADS + threadIdx.x, m_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + (DB * 16 + 1) * THREADS + threadIdx.x, l_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        parts_published();      // the part has arrived before it is counted
        __syncthreads();
        int *counter = p.counters + group;
        if (threadIdx.x == 0) s_seen = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (s_seen != parts - 1) return;
        parts_visible();
        if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        float m_all = -INFINITY;
        for (int i0 = 0; i0 < parts; i0 += 8) {       // eight loads in flight at a time
            float mp[8];
#pragma unroll
            for (int i = 0; i < 8; i++)
                mp[i] = i0 + i < parts ? __hip_atomic_load(slot + (size_t)(i0 + i) * kPartFloats(D, THREADS) + DB * 16 * THREADS + threadIdx.x,
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                       : -INFINITY;
#pragma unroll
            for (int i = 0; i < 8; i++) m_all = fmaxf(m_all, mp[i]);
        }
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[db][i] = 0.f;
        l_run = 0.f;
        for (int i = 0; i < parts; i++) {
            const float *from = slot + (size_t)i * kPartFloats(D, THREADS);
            const float mi = __hip_atomic_load(from + DB * 16 * THREADS + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float f = mi == -INFINITY ? 0.f : fast_exp2((mi - m_all) * sc);
            l_run = fmaf(__hip_atomic_load(from + (DB * 16 + 1) * THREADS + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT),
                         f, l_run);
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int j = 0; j < 16; j++)
                    o[db][j] = fmaf(__hip_atomic_load(from + (db * 16 + j) * THREADS + threadIdx.x, __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT), f, o[db][j]);
        }
    }
    if (rvalid) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        bf16_t *dst = p.out + ((size_t)(row0 + tq) * p.heads + head) * D + 4 * h;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                bf16x4_t v;
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = (bf16_t)(o[db][4 * j + i] * inv);
                *(bf16x4_t *)(dst + db * 32 + 8 * j) = v;
            }
    }
}

// ---------------------------------------------------------------------------------------------
// decode kernel
// ---------------------------------------------------------------------------------------------
// A decode step reads the keys and values of a request once, so these loads carry the non-temporal hint (a step of
// the 8B sizes at batch 8: 4.75 -> 4.62 ms at contexts of 8,192, 8.88 -> 8.34 ms at 32,768; 6.20 -> 6.02 ms at batch 64).
#ifdef FLLM_CACHE_TEMPORAL
#define FLLM_CACHE_LOAD(ptr) (*(ptr))
#else
#define FLLM_CACHE_LOAD(ptr) __builtin_nontemporal_load(ptr)
#endif
template <int D, int WAVES>
__global__ void __launch_bounds__(WAVES * kWave)
attn_decode_kernel(AttnArgs p, int qtiles) {
    constexpr int KD = D / 32, DT = D / 16;
    constexpr int OP = D + 1;
    extern __shared__ float dsm[];   // sm_m[WAVES][16], sm_l[WAVES][16], sm_o[WAVES][gq][OP]
    const int row = blockIdx.x;
    const int qtile = blockIdx.y % qtiles, kvh = blockIdx.y / qtiles;
    const int split = blockIdx.z;
    const int G = p.heads / p.kv_heads;
    const int gq = min(G - qtile * 16, 16);   // query heads of this workgroup
    float *sm_m = dsm, *sm_l = dsm + WAVES * 16, *sm_o = dsm + 2 * WAVES * 16;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int hg = qtile * 16 + c;
    const int seg = p.row_seg[row];
    const bool qvalid = hg < G && seg >= 0;
    const int head = kvh * G + (hg < G ? hg : 0);
    const int n = seg >= 0 ? p.row_pos[row] + 1 : 0;
    const int lo = (p.window > 0 && n - p.window > 0) ? n - p.window : 0;
    const int ps = p.page_size, psh = p.ps_shift, pmask = ps - 1, nkv = p.kv_heads;
    const int first = (lo / 32) * 32;
    const int begin = first + split * p.keys_per_split;
    const int end = min(begin + p.keys_per_split, n);
    // the splits that hold keys of this row; the others have nothing to add and leave at once
    const int live_splits = p.counters ? max(1, (n - first + p.keys_per_split - 1) / p.keys_per_split) : p.splits;
    if (p.counters && split >= live_splits) return;
    const int32_t *tbl = p.tables + (size_t)(seg >= 0 ? seg : 0) * p.table_stride;

    bf16x8_t qf[KD];
#pragma unroll
    for (int kk = 0; kk < KD; kk++)
        qf[kk] = qvalid ? *(const bf16x8_t *)(p.q + (size_t)row * p.q_stride + (size_t)head * D + kk * 32 + g * 8) : zero8();

    f32x4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) o[dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // A block is 32 keys: two score tiles of 16.  Row c of tile j is key kb + 16 j + c, so that a load of the tile's keys
    // (chunks 4 kk + g of 16 neighbouring tokens) is 1 KiB in a row where a page holds 16 tokens or more.  Lane (c, g) then
    // holds the scores of keys kb + 16 j + 4 g + i, i = 0..3, and takes exactly those eight keys' values as its operand
    // of the second product: two runs of four neighbouring tokens of V^T, 8 bytes each.
    // The page numbers of a block are asked for one block ahead, so that a block waits for one memory latency
    // (its keys and values), not for two in a row.
    auto block_pages = [&](int kb, int (&kpage)[2], int (&vpage)[2]) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int key = kb + 16 * j + c, vkey = kb + 16 * j + 4 * g;
            kpage[j] = (kb < end && key < n && key >= lo) ? tbl[key >> psh] : 0;
            vpage[j] = (kb < end && vkey < n && vkey + 4 > lo) ? tbl[vkey >> psh] : 0;
        }
    };
    int kpage_next[2], vpage_next[2];
    block_pages(begin + wave * 32, kpage_next, vpage_next);
    for (int kb = begin + wave * 32; kb < end; kb += WAVES * 32) {
        int kpage[2], vpage[2];
#pragma unroll
        for (int j = 0; j < 2; j++) kpage[j] = kpage_next[j], vpage[j] = vpage_next[j];
        block_pages(kb + WAVES * 32, kpage_next, vpage_next);
        // All loads of the block are issued before the first product: one memory latency per block.
        bf16x8_t kf[2][KD];
        bf16x4_t vf[2][DT];
        bool vtail[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int key = kb + 16 * j + c;
            const bool valid = key >= lo && key < n;
            const bf16_t *kr = p.kp + key_offset(kpage[j], nkv, kvh, ps, D, key & pmask, g * 8);
#pragma unroll
            for (int kk = 0; kk < KD; kk++) kf[j][kk] = valid ? FLLM_CACHE_LOAD((const bf16x8_t *)(kr + (size_t)kk * 4 * ps * 8)) : zero8();
            const int vkey = kb + 16 * j + 4 * g;
            const bool vload = vkey < n && vkey + 4 > lo;
            vtail[j] = vload && vkey + 4 > n;
            const bf16_t *vr = p.vp + (((size_t)vpage[j] * nkv + kvh) * D + c) * ps + (vkey & pmask);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) vf[j][dt] = vload ? FLLM_CACHE_LOAD((const bf16x4_t *)(vr + (size_t)dt * 16 * ps)) : (bf16x4_t){(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
        }

        f32x4_t s[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            s[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KD; kk++) s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j][kk], qf[kk], s[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = kb + 16 * j + 4 * g + i;
                const bool vis = key >= lo && key < n;
                s[j][i] = vis ? s[j][i] * p.scale_log2 : -INFINITY;
            }
        float alpha;
        softmax_step<2>(s, m_run, l_run, alpha);
        const bf16x8_t pf = pack_p(s[0], s[1]);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            bf16x8_t a;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    // slots past the last token hold whatever an earlier request left
                    const bool past = vtail[j] && kb + 16 * j + 4 * g + e >= n;
                    a[4 * j + e] = past ? (bf16_t)0.0f : vf[j][dt][e];
                }
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf, o[dt] * alpha, 0, 0, 0);
        }
    }
    // the waves saw different keys: merge their statistics and outputs
    if (g == 0) {
        sm_m[wave * 16 + c] = m_run;
        sm_l[wave * 16 + c] = l_run;
    }
    if (c < gq) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int i = 0; i < 4; i++) sm_o[(wave * gq + c) * OP + dt * 16 + g * 4 + i] = o[dt][i];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < gq * D; idx += WAVES * kWave) {
        const int qi = idx / D, d = idx - qi * D;
        const int h = qtile * 16 + qi;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; w++) m = fmaxf(m, sm_m[w * 16 + qi]);
        float l = 0.f, acc = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            const float f = sm_m[w * 16 + qi] == -INFINITY ? 0.f : fast_exp2(sm_m[w * 16 + qi] - m);
            l += sm_l[w * 16 + qi] * f;
            acc += sm_o[(w * gq + qi) * OP + d] * f;
        }
        const size_t hrow = (size_t)row * p.heads + kvh * G + h;
        if (live_splits == 1) {
            p.out[hrow * D + d] = (bf16_t)(l > 0.f ? acc / l : 0.f);
        } else if (p.counters) {   // read by another workgroup of this launch: straight to the device's point of coherence
            __hip_atomic_store(p.ws_o + (hrow * p.splits + split) * D + d, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (d == 0) {
                __hip_atomic_store(p.ws_ml + (hrow * p.splits + split) * 2, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(p.ws_ml + (hrow * p.splits + split) * 2 + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        } else {
            p.ws_o[(hrow * p.splits + split) * D + d] = acc;
            if (d == 0) {
                p.ws_ml[(hrow * p.splits + split) * 2] = m;
                p.ws_ml[(hrow * p.splits + split) * 2 + 1] = l;
            }
        }
    }
    if (!p.counters || live_splits == 1) return;
    // The split that arrives last adds the parts up, in the order of the splits: the result does not depend on
    // which one that is.  Its partial sums have arrived before it is counted.
    __shared__ int s_seen;
    parts_published();
    __syncthreads();
    int *counter = p.counters + ((size_t)row * p.kv_heads + kvh) * qtiles + qtile;
    if (threadIdx.x == 0) s_seen = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_seen != live_splits - 1) return;
    parts_visible();
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
    // The parts are read eight at a time, all loads of a group asked for before the first is used.  The first group's
    // values are kept: up to eight parts (the usual case) cost one round trip to memory, not one for the largest
    // maximum and another for the sums.
    constexpr int GRP = 8;
    for (int idx = threadIdx.x; idx < gq * D; idx += WAVES * kWave) {
        const int qi = idx / D, d = idx - qi * D;
        const size_t hrow = (size_t)row * p.heads + kvh * G + qtile * 16 + qi;
        const float *ml = p.ws_ml + hrow * p.splits * 2;
        const float *po = p.ws_o + hrow * p.splits * D + d;
        auto load_group = [&](int s0, float (&ms)[GRP], float (&ls)[GRP], float (&os)[GRP]) {
#pragma unroll
            for (int i = 0; i < GRP; i++) {
                const bool live = s0 + i < live_splits;
                ms[i] = live ? __hip_atomic_load(ml + (s0 + i) * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : -INFINITY;
                ls[i] = live ? __hip_atomic_load(ml + (s0 + i) * 2 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
                os[i] = live ? __hip_atomic_load(po + (size_t)(s0 + i) * D, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
            }
        };
        float l = 0.f, acc = 0.f;
        auto add_group = [&](float m, const float (&ms)[GRP], const float (&ls)[GRP], const float (&os)[GRP]) {
#pragma unroll
            for (int i = 0; i < GRP; i++) {       // in the order of the parts
                const float f = ms[i] == -INFINITY ? 0.f : fast_exp2(ms[i] - m);
                l += ls[i] * f;
                acc += os[i] * f;
            }
        };
        float ms0[GRP], ls0[GRP], os0[GRP];
        load_group(0, ms0, ls0, os0);
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < GRP; i++) m = fmaxf(m, ms0[i]);
        for (int s0 = GRP; s0 < live_splits; s0 += GRP) {
            float ms[GRP];
#pragma unroll
            for (int i = 0; i < GRP; i++)
                ms[i] = s0 + i < live_splits ? __hip_atomic_load(ml + (s0 + i) * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : -INFINITY;
#pragma unroll
            for (int i = 0; i < GRP; i++) m = fmaxf(m, ms[i]);
        }
        add_group(m, ms0, ls0, os0);
        for (int s0 = GRP; s0 < live_splits; s0 += GRP) {
            float ms[GRP], ls[GRP], os[GRP];
            load_group(s0, ms, ls, os);
            add_group(m, ms, ls, os);
        }
        p.out[hrow * D + d] = (bf16_t)(l > 0.f ? acc / l : 0.f);
    }
}

template <int D>
__global__ void __launch_bounds__(kWave)
attn_merge_kernel(const float *__restrict__ ws_ml, const float *__restrict__ ws_o, bf16_t *__restrict__ out, int heads,
                  int splits) {
    const size_t hrow = (size_t)blockIdx.x * heads + blockIdx.y;
    float m = -INFINITY;
    for (int s = 0; s < splits; s++) m = fmaxf(m, ws_ml[(hrow * splits + s) * 2]);
    float l = 0.f;
    for (int s = 0; s < splits; s++) {
        const float ms = ws_ml[(hrow * splits + s) * 2];
        l += ws_ml[(hrow * splits + s) * 2 + 1] * (ms == -INFINITY ? 0.f : fast_exp2(ms - m));
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int d = threadIdx.x; d < D; d += kWave) {
        float acc = 0.f;
        for (int s = 0; s < splits; s++) {
            const float ms = ws_ml[(hrow * splits + s) * 2];
            acc += ws_o[(hrow * splits + s) * D + d] * (ms == -INFINITY ? 0.f : fast_exp2(ms - m));
        }
        out[hrow * D + d] = (bf16_t)(acc * inv);
    }
}

using fllm_plan::decode_split_plan;      // how a decode step is split over the context (plans.h)

bool fast_shape(int heads, int kv_heads, int head_dim, int page_size) {
    if (head_dim != 32 && head_dim != 64 && head_dim != 128) return false;
    if (page_size != 8 && page_size != 16 && page_size != 32 && page_size != 64) return false;
    if (heads / kv_heads > 64) return false;
    if (kv_heads > 4096) return false;   // offsets inside a page are kept in 32 bits
    return true;
}

int device_slots() {   // workgroups of the tile32 kernel that the device holds at a time: two a compute unit
    static int slots = 0;
    if (slots == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        int cus = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
        slots = 2 * (cus > 0 ? cus : 256);
    }
    return slots;
}

// How the tile32 kernel shares the key tiles of a row tile among workgroups (plans.h), with the device's slots and
// the option that is set by hand.
int prefill_part_plan(int tiles, int kv_heads, int rows, int max_context, int window, size_t room, int slots, int *max_parts) {
    return fllm_plan::prefill_part_plan(tiles, kv_heads, rows, max_context, window, room, slots, fllm_option_prefill_parts(),
                                        max_parts);
}

// Prompt portions on the 32x32x16 products: WAVES * 32 rows a workgroup.
template <int D, int WAVES>
int launch_tile32(const AttnArgs &a, int max_context, hipStream_t stream) {
    const int G = a.heads / a.kv_heads;
    const int TQ = WAVES * 32 / G;
    const int tiles = (a.rows + TQ - 1) / TQ + a.num_segs;   // upper bound; surplus workgroups leave at once
    AttnArgs p = a;
    int max_parts = 1;
    void *dev_ws = nullptr;
    size_t dev_ws_bytes = 0;
    if (fllm_option_prefill_parts() && fllm_device_workspace(&dev_ws, &dev_ws_bytes) && dev_ws_bytes > kWorkspaceCounterBytes) {
        p.part_tiles = prefill_part_plan(tiles, a.kv_heads, a.rows, max_context, a.window,
                                         (dev_ws_bytes - kWorkspaceCounterBytes) / (kPartFloats(D, WAVES * kWave) * sizeof(float)),
                                         device_slots() * 4 / WAVES, &max_parts);
        p.counters = (int *)dev_ws;
        p.parts_ws = (float *)((unsigned char *)dev_ws + kWorkspaceCounterBytes);
    }
    FLLM_REQUIRE(tiles >= 1 && (long)tiles * a.kv_heads <= 0x7fffffffL && max_parts <= 65535, "attention: grid too large");
    hipLaunchKernelGGL((attn_tile32_kernel<(D >= 64 ? D : 64), WAVES>), dim3(tiles * a.kv_heads, max_parts), dim3(WAVES * kWave), 0, stream, p);
    return fllm_check_launch("attention_tile32");
}

template <int D>
int launch(const AttnArgs &a, int uniform_rows, int max_context, void *workspace, size_t workspace_bytes,
           hipStream_t stream) {
    const int G = a.heads / a.kv_heads;
    if (uniform_rows) {
        const int qtiles = (G + 15) / 16;
        AttnArgs p = a;
        constexpr int WAVES = D >= 128 ? 8 : 16;   // wide heads: fewer waves, so that the operands of a block fit the registers
        void *dev_ws = nullptr;
        size_t dev_ws_bytes = 0;
        const bool fused = fllm_device_workspace(&dev_ws, &dev_ws_bytes) &&
                           (size_t)a.rows * a.kv_heads * qtiles * sizeof(int) <= kWorkspaceCounterBytes && fllm_option_fused_merge();
        decode_split_plan(a.rows, a.kv_heads, qtiles, max_context, WAVES * 32, fused, &p.splits, &p.keys_per_split);
        p.counters = fused && p.splits > 1 ? (int *)dev_ws : nullptr;
        if (p.splits > 1) {
            const size_t need = fllm_plan::decode_workspace_need(a.rows, a.heads, D, p.splits);
            FLLM_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                         "attention: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
            p.ws_ml = (float *)workspace;
            p.ws_o = p.ws_ml + (size_t)a.rows * a.heads * p.splits * 2;
        }
        FLLM_REQUIRE(a.kv_heads * qtiles <= 65535 && p.splits <= 65535, "attention: grid too large");
        const int gq = G < 16 ? G : 16;
        const size_t smem = fllm_plan::decode_lds_bytes(D, G);
        static_assert(WAVES == (D >= 128 ? 8 : 16), "the plan's wave count is the kernel's");
        static bool attribute_set = false;   // more than the default 64 KiB of dynamic LDS has to be asked for once
        if (!attribute_set) {
            const hipError_t e = hipFuncSetAttribute((const void *)attn_decode_kernel<D, WAVES>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 159 * 1024);   // a few static bytes come on top
            FLLM_REQUIRE(e == hipSuccess, "attention: cannot raise the LDS limit: %s", hipGetErrorString(e));
            attribute_set = true;
        }
        hipLaunchKernelGGL((attn_decode_kernel<D, WAVES>), dim3(a.rows, a.kv_heads * qtiles, p.splits), dim3(WAVES * kWave),
                           smem, stream, p, qtiles);
        if (p.splits > 1 && !p.counters)
            hipLaunchKernelGGL(attn_merge_kernel<D>, dim3(a.rows, a.heads), dim3(kWave), 0, stream, p.ws_ml, p.ws_o, a.out,
                               a.heads, p.splits);
        return fllm_check_launch("attention_decode");
    }
    if (D >= 64 && G <= 64 && fllm_option_tile32()) {   // 128 or 256 rows per workgroup on 32x32x16 products
        // 256 rows where they leave no compute unit without a workgroup and the contexts are long: twice the rows for
        // every key fetched from L2 (inside a model: 3 % at contexts of 2,048 to 16,384 keys, nothing or a loss below)
        const int wide = fllm_option_tile32_rows();
        const bool rows256 = wide == 256 || (wide == 0 && max_context > 4096 &&
                                             (long)((a.rows + 256 / G - 1) / (256 / G)) * a.kv_heads >= device_slots() / 2);
        return rows256 ? launch_tile32<D, 8>(a, max_context, stream) : launch_tile32<D, 4>(a, max_context, stream);
    }
    const int TQ = 64 / G;
    const int tiles = (a.rows + TQ - 1) / TQ + a.num_segs;   // upper bound; surplus workgroups leave at once
    hipLaunchKernelGGL(attn_tile_kernel<D>, dim3(tiles, a.kv_heads), dim3(kThreads), 0, stream, a);
    return fllm_check_launch("attention_tile");
}

}  // namespace

size_t fllm_attention_bf16_workspace_bytes(int rows, int heads, int kv_heads, int head_dim, int max_context) {
    if (rows <= 0 || heads <= 0 || kv_heads <= 0) return 0;
    const int qtiles = (heads / kv_heads + 15) / 16;
    int splits, per;
    // the larger of the two plans (with and without the device workspace): which one runs is decided at the launch
    size_t most = 0;
    for (int fused = 0; fused < 2; fused++) {
        decode_split_plan(rows, kv_heads, qtiles, max_context, (head_dim >= 128 ? 8 : 16) * 32, fused != 0, &splits, &per);
        most = std::max(most, fllm_plan::decode_workspace_need(rows, heads, head_dim, splits));
    }
    return most;
}

// 0: launched, negative: error, 1: shape declined (the caller uses the plain kernel)
int fllm_attention_bf16_fast(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                             int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                             int num_segs, void *out, int rows, int heads, int kv_heads, int head_dim, int page_size,
                             int num_pages, float scale, int window, int max_context, int single_from, void *workspace,
                             size_t workspace_bytes, hipStream_t stream) {
    if (!fllm_fast_kernels_enabled()) return 1;
    (void)num_pages;
    if (!fast_shape(heads, kv_heads, head_dim, page_size)) return 1;
    if (q_stride % 8 != 0 || ((uintptr_t)q & 15) != 0) return 1;
    const int singles = num_segs - single_from;       // segments of one row each, at the end of the batch
    if (single_from == 0 && rows != num_segs) return 1;
    if (singles > rows) return 1;
    AttnArgs a;
    a.q = (const bf16_t *)q;
    a.q_stride = q_stride;
    a.kp = (const bf16_t *)k_pages;
    a.vp = (const bf16_t *)v_pages;
    a.tables = tables;
    a.table_stride = table_stride;
    a.row_pos = row_pos;
    a.row_seg = row_seg;
    a.seg_start = seg_start;
    a.num_segs = num_segs;
    a.out = (bf16_t *)out;
    a.rows = rows;
    a.heads = heads;
    a.kv_heads = kv_heads;
    a.page_size = page_size;
    a.ps_shift = page_size == 8 ? 3 : page_size == 16 ? 4 : page_size == 32 ? 5 : 6;
    a.scale_log2 = scale * kLog2e;
    a.window = window;
    a.ws_ml = nullptr;
    a.ws_o = nullptr;
    a.splits = 1;
    a.keys_per_split = 0;
    a.counters = nullptr;
    a.part_tiles = 0;
    a.parts_ws = nullptr;
    auto run = [&](const AttnArgs &part, int uniform) {
        if (head_dim == 32) return launch<32>(part, uniform, max_context, workspace, workspace_bytes, stream);
        if (head_dim == 64) return launch<64>(part, uniform, max_context, workspace, workspace_bytes, stream);
        return launch<128>(part, uniform, max_context, workspace, workspace_bytes, stream);
    };
    if (single_from == 0 || singles == 0) return run(a, single_from == 0);
    // Portions of prompts beside single tokens: the portions go to the tile kernel, the single rows behind them to
    // the decode kernel, which splits long contexts over workgroups (one row of a long context is a poor tile).
    const int first = rows - singles;
    AttnArgs portions = a;
    portions.rows = first;
    portions.num_segs = single_from;
    const int rc = run(portions, 0);
    if (rc != 0) return rc;
    AttnArgs single = a;
    single.q = a.q + (size_t)first * q_stride;
    single.row_pos = row_pos + first;
    single.row_seg = row_seg + first;
    single.seg_start = seg_start + single_from;
    single.num_segs = singles;
    single.out = a.out + (size_t)first * heads * head_dim;
    single.rows = singles;
    return run(single, 1);
}
