// Sampling on the device: one workgroup per row of logits (greedy rows of a wide vocabulary: several).
//
// Greedy rows take the first index of the largest finite value.  Other rows follow the
// reference's device sampler (rust/engine/cuda/sampling.cu:1-13, :253-352): temperature, top-k
// (ties at the threshold are kept), top-p (smallest set of largest values whose mass reaches
// top_p, ties kept), then a Gumbel-max draw: argmax of (logit - max) / T - ln(-ln u_i) over the
// survivors, u_i from Philox-4x32-10 keyed by the request's seed with counter
// (token id, 0, draw_lo, draw_hi) (rust/engine/src/sampling.rs:155-179).  The result depends on
// (seed, draw, logits) only: not on the batch, the row or the launch.
#include "api.h"
#include "common.h"

namespace {

constexpr int kBlock = 1024;
constexpr int kWaves = kBlock / kWave;

struct Shared {
    double dred[kWaves];
    float fred[kWaves];
    int ired[kWaves];
    unsigned hist[256];
    uint32_t prefix;
    int remaining;
};

__device__ __forceinline__ void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int i = 0; i < 10; i++) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c[0]), lo0 = 0xD2511F53u * c[0];
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c[2]), lo1 = 0xCD9E8D57u * c[2];
        const uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
        c[0] = n0; c[1] = lo1; c[2] = n2; c[3] = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

// a number in the open interval (0, 1)
__device__ __forceinline__ float philox_uniform(uint64_t seed, uint64_t draw, uint32_t index) {
    uint32_t c[4] = {index, 0u, (uint32_t)draw, (uint32_t)(draw >> 32)};
    philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
    return ((float)(c[0] >> 8) + 0.5f) / 16777216.0f;
}

// order-preserving map of floats to unsigned integers (larger float, larger key)
__device__ __forceinline__ uint32_t f2key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ double block_sum_d(double v, Shared &sh) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) sh.dred[threadIdx.x / kWave] = v;
    __syncthreads();
    double total = 0.0;
#pragma unroll
    for (int i = 0; i < kWaves; i++) total += sh.dred[i];
    __syncthreads();
    return total;
}

__device__ __forceinline__ float block_max_f(float v, Shared &sh) {
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) sh.fred[threadIdx.x / kWave] = v;
    __syncthreads();
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < kWaves; i++) m = fmaxf(m, sh.fred[i]);
    __syncthreads();
    return m;
}

// largest value, lowest index on ties; index INT_MAX when nothing qualified
__device__ __forceinline__ int block_argmax(float v, int idx, Shared &sh) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, kWave);
        const int oi = __shfl_xor(idx, o, kWave);
        if (ov > v || (ov == v && oi < idx)) {
            v = ov;
            idx = oi;
        }
    }
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) {
        sh.fred[threadIdx.x / kWave] = v;
        sh.ired[threadIdx.x / kWave] = idx;
    }
    __syncthreads();
    float best = sh.fred[0];
    int besti = sh.ired[0];
#pragma unroll
    for (int i = 1; i < kWaves; i++) {
        if (sh.fred[i] > best || (sh.fred[i] == best && sh.ired[i] < besti)) {
            best = sh.fred[i];
            besti = sh.ired[i];
        }
    }
    __syncthreads();
    return besti;
}

__device__ __forceinline__ float sanitize(float v) { return isfinite(v) ? v : -INFINITY; }

__device__ int row_argmax(const float *w, int vocab, Shared &sh) {
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += kBlock) {
        const float v = w[i];
        if (isfinite(v) && v > best) {   // indices rise, so the first maximum stays
            best = v;
            besti = i;
        }
    }
    return block_argmax(best, besti, sh);
}

__global__ void __launch_bounds__(kBlock)
argmax_kernel(const float *__restrict__ logits, int32_t *__restrict__ out, int vocab) {
    __shared__ Shared sh;
    const int idx = row_argmax(logits + (size_t)blockIdx.x * vocab, vocab, sh);
    if (threadIdx.x == 0) out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
}

// The same over `parts` workgroups a row: each takes a stretch of the vocabulary and leaves its best (value,
// index) in `partial`; the one that arrives last (counted in counters[row], zero before and after) picks the
// largest value, on ties the lowest index, so the answer does not depend on who that is.
__global__ void __launch_bounds__(kBlock)
argmax_split_kernel(const float *__restrict__ logits, int32_t *__restrict__ out, int vocab, int parts, int per_part,
                    float *partial_v, int *partial_i, int *counters) {
    __shared__ Shared sh;
    __shared__ int s_seen;
    const int row = blockIdx.x, part = blockIdx.y;
    const int lo = part * per_part, hi = min(vocab, lo + per_part);
    const float *w = logits + (size_t)row * vocab;
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += kBlock) {
        const float v = w[i];
        if (isfinite(v) && v > best) {
            best = v;
            besti = i;
        }
    }
    besti = block_argmax(best, besti, sh);
    if (threadIdx.x == 0) {
        const float bv = besti == 0x7fffffff ? -INFINITY : w[besti];
        __hip_atomic_store(partial_v + (size_t)row * parts + part, bv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(partial_i + (size_t)row * parts + part, besti, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);      // the part has arrived before it is counted
        s_seen = __hip_atomic_fetch_add(counters + row, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (s_seen != parts - 1) return;
    if (threadIdx.x == 0) __hip_atomic_store(counters + row, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float v = -INFINITY;
    int idx = 0x7fffffff;
    if ((int)threadIdx.x < parts) {
        v = __hip_atomic_load(partial_v + (size_t)row * parts + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        idx = __hip_atomic_load(partial_i + (size_t)row * parts + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    idx = block_argmax(v, idx, sh);
    if (threadIdx.x == 0) out[row] = idx == 0x7fffffff ? 0 : idx;
}

// ---------------------------------------------------------------------------------------------
// temperature / top-k / top-p / Gumbel-max
// ---------------------------------------------------------------------------------------------
// The thresholds of top-k and top-p lie among the few largest logits.  One pass over the vocabulary
// fills a histogram over the distance from the largest logit, in steps of 1/64 up to 64 (token
// counts for top-k, probability mass in 40-bit fixed point for top-p: integer sums, so the order of
// the additions does not matter); the bin in which the threshold falls is read off it, the tokens
// up to that bin are gathered into a list (in an order that depends on the data only), and the
// exact thresholds (radix select, bisection over the keys with sums in double precision) and the
// draw then run over the list.  A threshold further than 64 below the maximum puts every token on
// the list.
constexpr int kBins = 4096;
constexpr float kBinsPerUnit = 64.0f;

// bin of a finite logit v <= m; kBins: further from the maximum than the histogram reaches
__device__ __forceinline__ int bin_of(float v, float m) {
    const float d = (m - v) * kBinsPerUnit;
    return d < (float)kBins ? (int)d : kBins;
}

// exclusive prefix sum over the threads of the workgroup, and the total
__device__ __forceinline__ int block_exclusive_scan(int v, Shared &sh, int *total) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int inc = v;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int n = __shfl_up(inc, o, kWave);
        if (lane >= o) inc += n;
    }
    __syncthreads();
    if (lane == kWave - 1) sh.ired[wave] = inc;
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int i = 0; i < kWaves; i++) {
        if (i < wave) before += sh.ired[i];
        all += sh.ired[i];
    }
    __syncthreads();
    *total = all;
    return before + inc - v;
}

// The lowest bin b with sum(hist[0..b]) >= target, kBins when the whole histogram falls short; done by the first
// wave, every lane over 64 bins; the same value in every thread.
__device__ int find_bin(const unsigned long long *hist, unsigned long long target, Shared &sh) {
    __syncthreads();
    if (threadIdx.x < kWave) {
        const int lane = threadIdx.x;
        constexpr int PER = kBins / kWave;
        unsigned long long own = 0;
        for (int i = 0; i < PER; i++) own += hist[lane * PER + i];
        unsigned long long below = 0;      // sum of the lanes before this one
        for (int o = 1; o < kWave; o++) {
            const unsigned long long other = __shfl(own, (lane - o) & (kWave - 1), kWave);
            if (lane - o >= 0) below += other;
        }
        int found = kBins;
        if (below < target && below + own >= target) {      // the crossing lies in this lane's bins: one lane, if any
            unsigned long long cum = below;
            for (int i = 0; i < PER; i++) {
                cum += hist[lane * PER + i];
                if (cum >= target) {
                    found = lane * PER + i;
                    break;
                }
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) found = min(found, __shfl_xor(found, o, kWave));
        if (lane == 0) sh.remaining = found;
    }
    __syncthreads();
    const int bin = sh.remaining;
    __syncthreads();
    return bin;
}

// key of the k-th largest value among get(0 .. n-1): radix select, 4 passes of 8 bits
template <typename Get>
__device__ uint32_t kth_largest_key_of(Get get, int n, int k, Shared &sh) {
    if (threadIdx.x == 0) {
        sh.prefix = 0;
        sh.remaining = k;
    }
    __syncthreads();
    for (int pass = 0; pass < 4; pass++) {
        const int shift = 24 - 8 * pass;
        for (int i = threadIdx.x; i < 256; i += kBlock) sh.hist[i] = 0;
        __syncthreads();
        const uint32_t prefix = sh.prefix;
        for (int i = threadIdx.x; i < n; i += kBlock) {
            const uint32_t key = f2key(get(i));
            const bool match = pass == 0 || (key >> (shift + 8)) == (prefix >> (shift + 8));
            if (match) atomicAdd(&sh.hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int acc = 0;
            const int rem = sh.remaining;
            uint32_t bin = 0;
            for (int b = 255; b >= 0; b--) {
                if (acc + (int)sh.hist[b] >= rem) {
                    bin = (uint32_t)b;
                    break;
                }
                acc += (int)sh.hist[b];
            }
            sh.prefix = prefix | (bin << shift);
            sh.remaining = rem - acc;
        }
        __syncthreads();
    }
    return sh.prefix;
}

// `work` gives every row `vocab` 32-bit words of its own (the list of token ids); it must not overlap the logits.
__global__ void __launch_bounds__(kBlock)
sample_kernel(const float *__restrict__ logits, float *__restrict__ work, const FllmSampleRow *__restrict__ params,
              int32_t *__restrict__ out, int vocab) {
    __shared__ Shared sh;
    __shared__ unsigned long long bins[kBins];
    const int row = blockIdx.x;
    const FllmSampleRow p = params[row];
    const float *src = logits + (size_t)row * vocab;
    if (p.temperature <= 1e-5f) {
        const int idx = row_argmax(src, vocab, sh);
        if (threadIdx.x == 0) out[row] = idx == 0x7fffffff ? 0 : idx;
        return;
    }
    int *list = (int *)(work + (size_t)row * vocab);
    float m = -INFINITY;
    for (int i = threadIdx.x; i < vocab; i += kBlock) m = fmaxf(m, sanitize(src[i]));
    m = block_max_f(m, sh);
    if (!(m > -INFINITY)) {
        if (threadIdx.x == 0) out[row] = 0;   // no finite logit: the reference's argmax gives index 0 as well
        return;
    }
    const float inv_t = (float)(1.0 / (double)p.temperature);
    const bool use_k = p.top_k > 0 && p.top_k < vocab;
    const bool use_p = p.top_p > 0.f && p.top_p < 1.f;
    int count = vocab;                       // tokens the draw looks at: all of them, or the list
    uint32_t threshold = 0;                  // key below which a listed token is out
    if (use_k || use_p) {
        for (int i = threadIdx.x; i < kBins; i += kBlock) bins[i] = 0;
        __syncthreads();
        double total = 0.0;                  // mass of all finite logits (top-p without top-k)
        unsigned long long reach = 0;        // what this thread put into the histogram, in its units (top-p)
        for (int i = threadIdx.x; i < vocab; i += kBlock) {
            const float v = sanitize(src[i]);
            if (!(v > -INFINITY)) continue;
            const int b = bin_of(v, m);
            if (use_k) {
                if (b < kBins) atomicAdd(&bins[b], 1ull);
            } else {
                const float e = expf((v - m) * inv_t);
                total += (double)e;
                const unsigned long long fixed = (unsigned long long)((double)e * 1099511627776.0);
                reach += fixed;
                if (b < kBins && fixed != 0) atomicAdd(&bins[b], fixed);
            }
        }
        int last_bin;
        if (use_k) {
            last_bin = find_bin(bins, (unsigned long long)p.top_k, sh);
        } else {
            total = block_sum_d(total, sh);
            // the sum of every thread's share, far tokens included: integers, the same in any order
            const double all = block_sum_d((double)reach, sh);
            last_bin = find_bin(bins, (unsigned long long)((double)p.top_p * all), sh);
            if (last_bin < kBins) last_bin++;   // a bin to spare: the histogram's sums are rounded, the exact ones decide
        }
        // gather the tokens up to that bin: thread t's tokens in the order it meets them, behind those of the threads before it
        int mine = 0;
        for (int i = threadIdx.x; i < vocab; i += kBlock) {
            const float v = sanitize(src[i]);
            mine += (v > -INFINITY && bin_of(v, m) <= last_bin) ? 1 : 0;
        }
        int at = block_exclusive_scan(mine, sh, &count);
        for (int i = threadIdx.x; i < vocab; i += kBlock) {
            const float v = sanitize(src[i]);
            if (v > -INFINITY && bin_of(v, m) <= last_bin) list[at++] = i;
        }
        __syncthreads();
        auto listed = [&](int i) { return sanitize(src[list[i]]); };
        if (use_k) {
            threshold = kth_largest_key_of(listed, count, min(p.top_k, count), sh);
            if (use_p) {                      // the mass of what top-k left
                total = 0.0;
                for (int i = threadIdx.x; i < count; i += kBlock) {
                    const float v = listed(i);
                    if (f2key(v) >= threshold) total += (double)expf((v - m) * inv_t);
                }
                total = block_sum_d(total, sh);
            }
        }
        if (use_p) {
            const double target = (double)p.top_p * total;
            // largest key t such that the mass of {key >= t} still reaches the target
            uint32_t lo = threshold, hi = 0xFFFFFFFFu;
            while (lo < hi) {
                const uint32_t mid = lo + ((hi - lo) >> 1) + 1;
                double part = 0.0;
                for (int i = threadIdx.x; i < count; i += kBlock) {
                    const float v = listed(i);
                    if (f2key(v) >= mid) part += (double)expf((v - m) * inv_t);
                }
                if (block_sum_d(part, sh) >= target) lo = mid;
                else hi = mid - 1;
            }
            threshold = lo;
        }
    }
    float best = -INFINITY;
    int besti = 0x7fffffff;
    const bool whole = !(use_k || use_p);
    for (int i = threadIdx.x; i < count; i += kBlock) {
        const int id = whole ? i : list[i];
        const float v = sanitize(src[id]);
        if (!(v > -INFINITY) || f2key(v) < threshold) continue;
        const float u = philox_uniform(p.seed, p.draw, (uint32_t)id);
        const float score = (v - m) * inv_t - logf(-logf(u));
        if (score > best || (score == best && id < besti)) {
            best = score;
            besti = id;
        }
    }
    const int idx = block_argmax(best, besti, sh);
    if (threadIdx.x == 0) out[row] = idx == 0x7fffffff ? 0 : idx;
}

}  // namespace

extern "C" int fllm_argmax(const float *logits, int32_t *out, int rows, int vocab, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    // few rows of a wide vocabulary: several workgroups a row, if the device workspace is there for them to meet in
    void *ws = nullptr;
    size_t ws_bytes = 0;
    int parts = (vocab + 8191) / 8192;
    if (parts > 64) parts = 64;
    if (parts * rows > 2048) parts = 2048 / rows;
    if (parts > 1 && fllm_device_workspace(&ws, &ws_bytes) && (size_t)rows * sizeof(int) <= kWorkspaceCounterBytes &&
        kWorkspaceCounterBytes + (size_t)rows * parts * 8 <= ws_bytes) {
        const int per_part = (vocab + parts - 1) / parts;
        float *pv = (float *)((unsigned char *)ws + kWorkspaceCounterBytes);
        int *pi = (int *)(pv + (size_t)rows * parts);
        hipLaunchKernelGGL(argmax_split_kernel, dim3(rows, parts), dim3(kBlock), 0, stream, logits, out, vocab, parts, per_part,
                           pv, pi, (int *)ws);
        return fllm_check_launch("argmax");
    }
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(kBlock), 0, stream, logits, out, vocab);
    return fllm_check_launch("argmax");
}

// ---------------------------------------------------------------------------------------------
// The split argmax for callers that cannot allocate and hand over no workspace.
// ---------------------------------------------------------------------------------------------
// Partial results and arrival counters live in a file-scope device array.  Every GPU holds a copy of its own at an
// address of its own, which the host learns once per device through hipGetSymbolAddress; host code uses that
// address only, never the array's name.  Layout: kStaticRows counters (int), then kStaticRows * kStaticParts
// values (float), then as many indices (int).
constexpr int kStaticRows = 256;         // most rows a call takes
constexpr int kStaticParts = 64;         // most workgroups a row
constexpr size_t kStaticBytes = (size_t)kStaticRows * 4 + (size_t)kStaticRows * kStaticParts * 8;     // 132,096 bytes
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

constexpr int kMaxDevices = 16;
static void *g_static_scratch[kMaxDevices];     // per device: the address of its copy of `scratch`

// the address of the current device's copy, looked up at the first call on that device
static int static_scratch_of_current_device(unsigned char **base) {
    int dev = -1;
    FLLM_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "argmax_static: no current device below %d",
                 kMaxDevices);
    void *ptr = __atomic_load_n(&g_static_scratch[dev], __ATOMIC_ACQUIRE);
    if (ptr == nullptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        FLLM_REQUIRE(e == hipSuccess && ptr != nullptr, "argmax_static: the device's scratch array was not found: %s",
                     hipGetErrorString(e));
        __atomic_store_n(&g_static_scratch[dev], ptr, __ATOMIC_RELEASE);     // threads that race here store the same address
    }
    *base = (unsigned char *)ptr;
    return 0;
}

__global__ void clear_ints_kernel(int *p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

extern "C" int fllm_argmax_static(const float *logits, int32_t *out, int rows, int vocab, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && vocab > 0, "argmax_static: bad sizes rows=%d vocab=%d", rows, vocab);
    FLLM_REQUIRE(rows <= kStaticRows, "argmax_static: %d rows, the static scratch array is made for at most %d (use fllm_argmax)",
                 rows, kStaticRows);
    if (rows == 0) return 0;
    FLLM_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: logits and out are required");
    unsigned char *base = nullptr;
    if (static_scratch_of_current_device(&base) != 0) return -1;
    int parts = (vocab + 8191) / 8192;          // the plan of fllm_argmax
    if (parts > kStaticParts) parts = kStaticParts;
    if (parts * rows > 2048) parts = 2048 / rows;
    if (parts < 1) parts = 1;
    const int per_part = (vocab + parts - 1) / parts;
    int *counters = (int *)base;
    float *pv = (float *)(base + (size_t)kStaticRows * 4);
    int *pi = (int *)(pv + (size_t)kStaticRows * kStaticParts);
    // the array keeps what the call before left (a call that was cut short may have left counts): the counters start at zero
    hipLaunchKernelGGL(clear_ints_kernel, dim3((rows + 255) / 256), dim3(256), 0, stream, counters, rows);
    hipLaunchKernelGGL(argmax_split_kernel, dim3(rows, parts), dim3(kBlock), 0, stream, logits, out, vocab, parts, per_part, pv, pi,
                       counters);
    return fllm_check_launch("argmax_static");
}

extern "C" int fllm_sample(const float *logits, float *work, const FllmSampleRow *params, int32_t *out, int rows,
                           int vocab, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    FLLM_REQUIRE(work != nullptr && params != nullptr, "sample: work and params are required");
    if (rows == 0) return 0;
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kBlock), 0, stream, logits, work, params, out, vocab);
    return fllm_check_launch("sample");
}
