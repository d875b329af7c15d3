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

// A candidate for "the largest value, at the lowest index among equals".  kNone marks "nothing qualified".
constexpr int kNone = 0x7fffffff;
struct Pick {
    float value;
    int index;
};
__device__ __forceinline__ Pick better_of(Pick a, Pick b) {
    const bool take_b = b.value > a.value || (b.value == a.value && b.index < a.index);
    return take_b ? b : a;
}

// What the reductions of a workgroup pass through LDS: one cell a wave.
struct Cells {
    Pick picks[kWaves];
    double sums[kWaves];
    int counts[kWaves];
    int word;            // a value one thread hands to all
    uint32_t key;
    unsigned long long before;
    unsigned long long units[kWaves];
};

__device__ __forceinline__ Pick wave_best(Pick p) {
#pragma unroll
    for (int hop = kWave / 2; hop >= 1; hop /= 2) {
        Pick other;
        other.value = __shfl_xor(p.value, hop, kWave);
        other.index = __shfl_xor(p.index, hop, kWave);
        p = better_of(p, other);
    }
    return p;
}
__device__ __forceinline__ int wave_count(int v) {
#pragma unroll
    for (int hop = kWave / 2; hop >= 1; hop /= 2) v += __shfl_xor(v, hop, kWave);
    return v;
}
__device__ __forceinline__ double wave_mass(double v) {
#pragma unroll
    for (int hop = kWave / 2; hop >= 1; hop /= 2) v += __shfl_xor(v, hop, kWave);
    return v;
}

// The best pick of the workgroup, the same in every thread: every wave leaves its best in its cell and all threads
// fold the cells in wave order.
__device__ __forceinline__ Pick block_best(Pick p, Cells &cells) {
    p = wave_best(p);
    const int wave = threadIdx.x / kWave;
    __syncthreads();                               // the cells are free again
    if (threadIdx.x % kWave == 0) cells.picks[wave] = p;
    __syncthreads();
    Pick all = cells.picks[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) all = better_of(all, cells.picks[w]);
    return all;
}
__device__ __forceinline__ float block_largest(float v, Cells &cells) {
    Pick p = {v, 0};
    return block_best(p, cells).value;
}

// finite values stay, everything else can never be chosen
__device__ __forceinline__ float usable(float v) { return fabsf(v) < INFINITY ? v : -INFINITY; }

// the best pick among w[lo .. hi): a thread meets its indices in rising order, so the first of equal values stays
__device__ __forceinline__ Pick best_in_range(const float *w, int lo, int hi) {
    Pick mine = {-INFINITY, kNone};
    for (int i = lo + (int)threadIdx.x; i < hi; i += kBlock) {
        const float v = w[i];
        if (fabsf(v) < INFINITY && v > mine.value) {
            mine.value = v;
            mine.index = i;
        }
    }
    return mine;
}
__device__ __forceinline__ int32_t token_of(Pick p) { return p.index == kNone ? 0 : p.index; }

__global__ void __launch_bounds__(kBlock)
argmax_kernel(const float *__restrict__ logits, int32_t *__restrict__ out, int vocab) {
    __shared__ Cells cells;
    const Pick best = block_best(best_in_range(logits + (size_t)blockIdx.x * vocab, 0, vocab), cells);
    if (threadIdx.x == 0) out[blockIdx.x] = token_of(best);
}

// The same over `parts` workgroups a row: each takes a stretch of the vocabulary and leaves its best (value,
// index) in `partial`; the one that arrives last (counted in counters[row], zero before and after) picks the
// largest value, on ties the lowest index, so the answer does not depend on who that is.
// A part's workgroup leaves its best and is counted; true in the workgroup that was counted last, which then holds
// the best of all parts in `all` (the largest value, on ties the lowest index, whoever it is) and has put the row's
// counter back to zero.  parts <= kBlock.
__device__ __forceinline__ bool meet_and_merge(Pick best, int row, int part, int parts, float *partial_v, int *partial_i,
                                               int *counters, Cells &cells, Pick *all) {
    if (threadIdx.x == 0) {
        __hip_atomic_store(partial_v + (size_t)row * parts + part, best.value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(partial_i + (size_t)row * parts + part, best.index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        parts_published();      // the part has arrived before it is counted
        cells.word = __hip_atomic_fetch_add(counters + row, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (cells.word != parts - 1) return false;
    parts_visible();
    if (threadIdx.x == 0) __hip_atomic_store(counters + row, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    Pick mine = {-INFINITY, kNone};
    if ((int)threadIdx.x < parts) {
        mine.value = __hip_atomic_load(partial_v + (size_t)row * parts + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        mine.index = __hip_atomic_load(partial_i + (size_t)row * parts + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    *all = block_best(mine, cells);
    return true;
}

__global__ void __launch_bounds__(kBlock)
argmax_split_kernel(const float *__restrict__ logits, int32_t *__restrict__ out, int vocab, int parts, int per_part,
                    float *partial_v, int *partial_i, int *counters) {
    __shared__ Cells cells;
    const int row = blockIdx.x, part = blockIdx.y;
    const int lo = part * per_part, hi = min(vocab, lo + per_part);
    const Pick best = block_best(best_in_range(logits + (size_t)row * vocab, lo, hi), cells);
    Pick all;
    if (meet_and_merge(best, row, part, parts, partial_v, partial_i, counters, cells, &all) && threadIdx.x == 0)
        out[row] = token_of(all);
}

// ---------------------------------------------------------------------------------------------
// Random numbers: Philox-4x32 with ten rounds (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3"), the
// generator the reference keys its draws with (rust/engine/src/sampling.rs:155-183).  A round multiplies two
// counter words by fixed odd constants and mixes the halves of the products with the other words and the key; the
// key moves on by the golden-ratio and sqrt(3) - 1 constants.
// ---------------------------------------------------------------------------------------------
// The uniform number of (seed, draw, token): the counter is (token, 0, draw), the key is the seed; the top 24 bits of
// the first output word, centred in their cell, so that the number lies strictly between 0 and 1.
__device__ __forceinline__ float uniform_of(uint64_t seed, uint64_t draw, uint32_t token) {
    Philox g = {token, 0u, (uint32_t)draw, (uint32_t)(draw >> 32)};
    g.ten_rounds((uint32_t)seed, (uint32_t)(seed >> 32));
    return ((float)(g.c0 >> 8) + 0.5f) * (1.0f / 16777216.0f);
}

// Floats as unsigned integers in the same order: the sign bit is set on positive numbers, all bits are turned
// over on negative ones.
__device__ __forceinline__ uint32_t ordered_key(float f) {
    const uint32_t bits = __float_as_uint(f);
    return bits ^ ((uint32_t)((int32_t)bits >> 31) | 0x80000000u);
}

// ---------------------------------------------------------------------------------------------
// temperature / top-k / top-p / Gumbel-max
// ---------------------------------------------------------------------------------------------
// The thresholds of top-k and top-p lie among the few largest logits.  One pass over the vocabulary
// fills a histogram over the distance from the largest logit, in steps of 1/64 up to 64 (token
// counts for top-k, probability mass in 40-bit fixed point for top-p: integer sums, so the order of
// the additions does not matter); the bin in which the threshold falls is read off it, the tokens
// up to that bin are gathered into a list (in an order that depends on the data only), and the
// exact thresholds and the draw then run over the list.  A threshold further than 64 below the maximum puts every
// token on the list.
//
// A threshold is a key t (ordered_key of a logit): the tokens with keys >= t stay.  Both thresholds are the largest
// t for which a sum over {key >= t} still reaches a target (k tokens; top_p of the mass), and such a t is built
// bit by bit from the top: a bit stays set if the sum with it set still reaches the target.  A list of up to
// kStaged candidates is copied into LDS (logit and weight exp((v - max) / T)) and ONE wave runs the 32 + 32 trials
// over it with shuffles and no barrier; a longer list (a flat distribution with top-p close to 1) takes three
// histograms over the bits of the keys instead, with weights in units of 2^-40 (`key_by_histograms`).
constexpr int kBins = 4096;
constexpr float kBinsPerUnit = 64.0f;
constexpr int kStaged = 4096;            // candidates that fit into the LDS the histogram no longer needs

// bin of a finite logit v <= m; kBins: further from the maximum than the histogram reaches
__device__ __forceinline__ int bin_of(float v, float m) {
    const float d = (m - v) * kBinsPerUnit;
    return d < (float)kBins ? (int)d : kBins;
}

// exclusive prefix sum over the threads of the workgroup, and the total
__device__ __forceinline__ int block_exclusive_scan(int v, Cells &cells, int *total) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int inc = v;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int n = __shfl_up(inc, o, kWave);
        if (lane >= o) inc += n;
    }
    __syncthreads();
    if (lane == kWave - 1) cells.counts[wave] = inc;
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int i = 0; i < kWaves; i++) {
        if (i < wave) before += cells.counts[i];
        all += cells.counts[i];
    }
    __syncthreads();
    *total = all;
    return before + inc - v;
}

// The lowest bin b with sum(hist[0..b]) >= target, kBins when the whole histogram falls short (or target is 0); the
// same value in every thread.  Every thread of the workgroup adds up kBins / kBlock neighbouring bins, the sums
// before each thread come from a scan across the lanes and the waves (integers: any order of adding), and the one
// thread in whose bins the running sum crosses the target says where.  `before`: the sum of the bins before that one.
__device__ int find_bin(const unsigned long long *hist, unsigned long long target, Cells &cells,
                        unsigned long long *before = nullptr) {
    constexpr int PER = kBins / kBlock;
    static_assert(PER * kBlock == kBins, "every thread has the same number of bins");
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    __syncthreads();
    unsigned long long own[PER], sum = 0;
#pragma unroll
    for (int i = 0; i < PER; i++) {
        own[i] = hist[threadIdx.x * PER + i];
        sum += own[i];
    }
    unsigned long long upto = sum;         // this thread's bins and those of the lanes before it
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const unsigned long long other = __shfl_up(upto, o, kWave);
        if (lane >= o) upto += other;
    }
    if (lane == kWave - 1) cells.units[wave] = upto;
    if (threadIdx.x == 0) cells.word = kBins, cells.before = 0;
    __syncthreads();
    unsigned long long below = upto - sum;
#pragma unroll
    for (int w = 0; w < kWaves; w++)
        if (w < wave) below += cells.units[w];
    if (below < target && below + sum >= target) {       // one thread, if any
        unsigned long long cum = below;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            if (cum + own[i] >= target) {
                cells.word = threadIdx.x * PER + i;
                cells.before = cum;
                break;
            }
            cum += own[i];
        }
    }
    __syncthreads();
    const int bin = cells.word;
    if (before != nullptr) *before = cells.before;
    __syncthreads();
    return bin;
}

// Who walks a list of candidates: the first wave alone (sums by shuffles, no barrier; the other waves wait at the
// next barrier) or the whole workgroup (sums through LDS).  Sums are the same in every thread that takes part.
struct OneWave {
    static constexpr int kStride = kWave;
    __device__ static int sum(int v, Cells &) { return wave_count(v); }
    __device__ static double sum(double v, Cells &) { return wave_mass(v); }
};
struct WholeBlock {
    static constexpr int kStride = kBlock;
    __device__ static int sum(int v, Cells &cells) {
        v = wave_count(v);
        __syncthreads();
        if (threadIdx.x % kWave == 0) cells.counts[threadIdx.x / kWave] = v;
        __syncthreads();
        int all = 0;
#pragma unroll
        for (int w = 0; w < kWaves; w++) all += cells.counts[w];
        return all;
    }
    __device__ static double sum(double v, Cells &cells) {
        v = wave_mass(v);
        __syncthreads();
        if (threadIdx.x % kWave == 0) cells.sums[threadIdx.x / kWave] = v;
        __syncthreads();
        double all = 0.0;
#pragma unroll
        for (int w = 0; w < kWaves; w++) all += cells.sums[w];      // in wave order: the same in every thread
        return all;
    }
};

// The largest key t such that at least k of the n candidates have keys >= t (the key of the k-th largest), built
// from the top bit down.  1 <= k <= n.
template <typename Who, typename KeyAt>
__device__ uint32_t key_of_kth_largest(KeyAt key_at, int n, int k, Cells &cells) {
    uint32_t t = 0;
    for (int bit = 31; bit >= 0; bit--) {
        const uint32_t trial = t | (1u << bit);
        int mine = 0;
        for (int i = threadIdx.x; i < n; i += Who::kStride) mine += key_at(i) >= trial ? 1 : 0;
        if (Who::sum(mine, cells) >= k) t = trial;
    }
    return t;
}

// Sum of the weights of the candidates with keys >= t.
template <typename Who, typename KeyAt, typename WeightAt>
__device__ double mass_from(KeyAt key_at, WeightAt weight_at, int n, uint32_t t, Cells &cells) {
    double mine = 0.0;
    for (int i = threadIdx.x; i < n; i += Who::kStride)
        if (key_at(i) >= t) mine += (double)weight_at(i);
    return Who::sum(mine, cells);
}

// The largest key t >= floor such that the weights of the candidates with keys >= t add up to `target` or more
// (floor itself if no larger key does).
template <typename Who, typename KeyAt, typename WeightAt>
__device__ uint32_t key_of_mass(KeyAt key_at, WeightAt weight_at, int n, uint32_t floor, double target, Cells &cells) {
    uint32_t t = 0;
    for (int bit = 31; bit >= 0; bit--) {
        const uint32_t trial = t | (1u << bit);
        // below the floor the answer is known: everything from the floor up counts, and that reaches the target
        if (trial <= floor || mass_from<Who>(key_at, weight_at, n, trial, cells) >= target) t = trial;
    }
    return t > floor ? t : floor;
}

// A candidate's weight in units of 2^-40: integers, whose sums do not depend on the order of the additions.
__device__ __forceinline__ unsigned long long units_of(float weight) {
    return (unsigned long long)((double)weight * 1099511627776.0);
}

// the sum of `v` over the workgroup, the same in every thread
__device__ __forceinline__ unsigned long long block_units(unsigned long long v, Cells &cells) {
#pragma unroll
    for (int hop = kWave / 2; hop >= 1; hop /= 2) v += __shfl_xor(v, hop, kWave);
    __syncthreads();
    if (threadIdx.x % kWave == 0) cells.units[threadIdx.x / kWave] = v;
    __syncthreads();
    unsigned long long all = 0;
#pragma unroll
    for (int w = 0; w < kWaves; w++) all += cells.units[w];
    return all;
}

// Long lists (more candidates than fit into LDS): the largest key t >= floor such that the candidates with keys in
// [t, ...) that are not below `floor` weigh `target` or more (MASS: in units of 2^-40; otherwise every candidate
// weighs 1), found with three histograms over the key's bits, 12, 12 and 8 from the top, instead of 32 walks over
// the list: each histogram covers the keys that share the bits found so far, its bin 0 holds the largest of them,
// and the bin at which the running sum reaches what is still missing gives the next bits.  `floor` if no larger
// key reaches the target.  `hist`: kBins cells of LDS.
template <bool MASS, typename KeyAt, typename WeightAt>
__device__ uint32_t key_by_histograms(KeyAt key_at, WeightAt weight_at, int n, uint32_t floor, unsigned long long target,
                                      unsigned long long *hist, Cells &cells) {
    uint32_t prefix = 0;
    int known = 0;                          // bits of the answer found so far, from the top
    unsigned long long above = 0;           // weight of the candidates whose keys lie above every key that begins with `prefix`
    for (int round = 0; round < 3; round++) {
        const int bits = round < 2 ? 12 : 8;
        const int shift = 32 - known - bits;
        const uint32_t mask = (1u << bits) - 1;
        for (int i = threadIdx.x; i < kBins; i += kBlock) hist[i] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < n; i += kBlock) {
            const uint32_t key = key_at(i);
            if (key == 0 || key < floor || (known > 0 && (key >> (32 - known)) != prefix)) continue;     // key 0: not a candidate
            const unsigned long long w = MASS ? units_of(weight_at(i)) : 1ull;
            if (w != 0) atomicAdd(&hist[mask - ((key >> shift) & mask)], w);
        }
        unsigned long long before = 0;
        const int bin = find_bin(hist, target - above, cells, &before);
        if (bin > (int)mask) return floor;   // everything from the floor up falls short of the target (rounding): keep it all
        above += before;
        prefix = (prefix << bits) | (mask - (uint32_t)bin);
        known += bits;
    }
    return prefix > floor ? prefix : floor;
}

// Both thresholds over one list.  `total` comes in as the mass of all finite logits and is replaced by the mass of
// what top-k keeps when top-k is on.
// min-p (`min_p` > 0) stands between the two: a candidate that weighs less than min_p (times the largest weight, which
// is 1) counts for nothing in top-p; the caller leaves such candidates out of the draw itself.
template <typename Who, typename KeyAt, typename WeightAt>
__device__ uint32_t thresholds(KeyAt key_at, WeightAt weight_at, int n, int top_k, bool use_k, bool use_p, float top_p,
                               float min_p, double total, Cells &cells) {
    uint32_t t = 0;
    if (use_k) t = key_of_kth_largest<Who>(key_at, n, min(top_k, n), cells);
    if (use_p) {
        auto heavy_key_at = [&](int i) { return weight_at(i) >= min_p ? key_at(i) : 0u; };     // min_p 0: every candidate
        if (use_k || min_p > 0.f) total = mass_from<Who>(heavy_key_at, weight_at, n, t > 1u ? t : 1u, cells);     // key 0: left out
        t = key_of_mass<Who>(heavy_key_at, weight_at, n, t, (double)top_p * total, cells);
    }
    return t;
}

// The same thresholds for a short list, by one wave (all 64 lanes must call): up to 4 * kWave candidates.  Instead of
// building each threshold bit by bit, with a sum across the lanes a bit, every lane ranks the candidates it holds
// (lane, lane + 64, ...) against all others: how many keys are no smaller than its own, and how much they weigh,
// added in index order.  The k-th largest key is the largest one that at least k keys are no smaller than; the top-p
// threshold the largest one from which on the weights reach the target.  Two sums across the lanes in all.
constexpr int kShortList = 4 * kWave;
__device__ __forceinline__ uint32_t wave_largest_key(uint32_t v) {
#pragma unroll
    for (int hop = kWave / 2; hop >= 1; hop /= 2) {
        const uint32_t other = (uint32_t)__shfl_xor((int)v, hop, kWave);
        v = other > v ? other : v;
    }
    return v;
}
template <typename KeyAt, typename WeightAt>
__device__ uint32_t thresholds_of_short_list(KeyAt key_at, WeightAt weight_at, int n, int top_k, bool use_k, bool use_p, float top_p,
                                             float min_p, double total) {
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t key[4];
    float weight[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int i = lane + e * kWave;
        key[e] = i < n ? key_at(i) : 0u;
        weight[e] = i < n ? weight_at(i) : 0.f;
    }
    uint32_t t = 0;
    if (use_k) {
        const int k = min(top_k, n);
        int no_smaller[4] = {0, 0, 0, 0};
        for (int j = 0; j < n; j++) {
            const uint32_t other = key_at(j);
#pragma unroll
            for (int e = 0; e < 4; e++) no_smaller[e] += other >= key[e] ? 1 : 0;
        }
        uint32_t mine = 0;
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (lane + e * kWave < n && no_smaller[e] >= k && key[e] > mine) mine = key[e];
        t = wave_largest_key(mine);
    }
    if (use_p) {
        // min-p: a candidate that weighs less than min_p counts for nothing here (key 0)
        uint32_t heavy[4];
#pragma unroll
        for (int e = 0; e < 4; e++) heavy[e] = weight[e] >= min_p ? key[e] : 0u;
        const uint32_t from = t > 1u ? t : 1u;
        double from_own[4] = {0.0, 0.0, 0.0, 0.0}, kept = 0.0;
        for (int j = 0; j < n; j++) {
            const float w = weight_at(j);
            const uint32_t other = w >= min_p ? key_at(j) : 0u;
            if (other >= from) kept += (double)w;
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (other >= heavy[e]) from_own[e] += (double)w;
        }
        if (use_k || min_p > 0.f) total = kept;          // top-p looks at what top-k and min-p left
        const double target = (double)top_p * total;
        uint32_t mine = 0;
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (heavy[e] != 0u && from_own[e] >= target && heavy[e] > mine) mine = heavy[e];
        const uint32_t reached = wave_largest_key(mine);
        t = reached > t ? reached : t;
    }
    return t;
}

// The threshold of a list too long for LDS, by the whole workgroup: top-k over `key_at` (key 0: not a candidate), then
// top-p over `heavy_key_at`, which is key_at with 0 for a candidate that min-p drops.  `all_units`: with top-p alone, the
// mass of every finite logit in units of 2^-40, listed or not.  `bins`: kBins cells of LDS.
template <typename KeyAt, typename WeightAt, typename HeavyKeyAt>
__device__ uint32_t threshold_of_long_list(KeyAt key_at, WeightAt weight_at, HeavyKeyAt heavy_key_at, int count, int top_k, bool use_k,
                                           bool use_p, bool use_m, float top_p, unsigned long long all_units, unsigned long long *bins,
                                           Cells &cells) {
    uint32_t t = 0;
    unsigned long long whole = all_units;
    if (use_k) t = key_by_histograms<false>(key_at, weight_at, count, 0u, (unsigned long long)min(top_k, count), bins, cells);
    if (use_p) {
        if (use_k || use_m) {
            unsigned long long mine = 0;
            for (int i = threadIdx.x; i < count; i += kBlock) {
                const uint32_t key = heavy_key_at(i);
                if (key != 0 && key >= t) mine += units_of(weight_at(i));
            }
            whole = block_units(mine, cells);
        }
        unsigned long long target = (unsigned long long)((double)top_p * (double)whole);
        if (target == 0) target = 1;
        t = key_by_histograms<true>(heavy_key_at, weight_at, count, t, target, bins, cells);
    }
    return t;
}

// Calls f(token, logit) for every token of a row, each thread of the workgroup with a share of its own: four
// consecutive tokens a load where the row's alignment allows (four such loads in flight), single tokens at both ends.
// A thread meets its tokens in the same order in every pass.
template <typename F>
__device__ __forceinline__ void for_each_token(const float *__restrict__ src, int vocab, F f) {
    const int head = min(vocab, (int)((4 - (((uintptr_t)src >> 2) & 3)) & 3));      // tokens before the first 16-byte boundary
    if ((int)threadIdx.x < head) f((int)threadIdx.x, src[threadIdx.x]);
    const int quads = (vocab - head) / 4;
    const f32x4_t *q = (const f32x4_t *)(src + head);
    int i = threadIdx.x;
    for (; i + 3 * kBlock < quads; i += 4 * kBlock) {
        f32x4_t v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = q[i + u * kBlock];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int t = head + 4 * (i + u * kBlock);
#pragma unroll
            for (int e = 0; e < 4; e++) f(t + e, v[u][e]);
        }
    }
    for (; i < quads; i += kBlock) {
        const f32x4_t a = q[i];
        const int ta = head + 4 * i;
#pragma unroll
        for (int e = 0; e < 4; e++) f(ta + e, a[e]);
    }
    const int done = head + 4 * quads;
    if ((int)threadIdx.x < vocab - done) f(done + (int)threadIdx.x, src[done + threadIdx.x]);
}

// a row with a temperature and none of top-k, top-p and min-p: the draw looks at every token
__device__ __forceinline__ bool draws_from_all(const FllmSampleRow &p, int vocab) {
    return p.temperature > 1e-5f && !(p.top_k > 0 && p.top_k < vocab) && !(p.top_p > 0.f && p.top_p < 1.f) && !(p.min_p > 0.f);
}

// Such rows spend their time on the random numbers of all tokens, so several workgroups share a row, in two
// launches: the largest logit first (`row_max`), then the largest (v - max) / T - ln(-ln u), each as a split argmax.
// Rows of another kind leave at once.
template <int PHASE>
__global__ void __launch_bounds__(kBlock)
draw_from_all_kernel(const float *__restrict__ logits, const FllmSampleRow *__restrict__ params, int32_t *__restrict__ out,
                     int vocab, int parts, int per_part, float *partial_v, int *partial_i, int *counters, float *row_max) {
    __shared__ Cells cells;
    const int row = blockIdx.x, part = blockIdx.y;
    const FllmSampleRow p = params[row];
    if (!draws_from_all(p, vocab)) return;
    const float *src = logits + (size_t)row * vocab;
    const int lo = part * per_part, hi = min(vocab, lo + per_part);
    Pick best = {-INFINITY, kNone}, all;
    if (PHASE == 0) {
        best = block_best(best_in_range(src, lo, hi), cells);
        if (meet_and_merge(best, row, part, parts, partial_v, partial_i, counters, cells, &all) && threadIdx.x == 0)
            row_max[row] = all.value;
        return;
    }
    const float m = row_max[row];
    if (!(m > -INFINITY)) {                  // no finite logit: index 0, as the reference's argmax gives
        if (part == 0 && threadIdx.x == 0) out[row] = 0;
        return;
    }
    const float inv_t = (float)(1.0 / (double)p.temperature);
    for (int i = lo + (int)threadIdx.x; i < hi; i += kBlock) {
        const float v = usable(src[i]);
        if (!(v > -INFINITY)) continue;
        const float u = uniform_of(p.seed, p.draw, (uint32_t)i);
        const Pick here = {(v - m) * inv_t - logf(-logf(u)), i};
        best = better_of(best, here);
    }
    best = block_best(best, cells);
    if (meet_and_merge(best, row, part, parts, partial_v, partial_i, counters, cells, &all) && threadIdx.x == 0)
        out[row] = token_of(all);
}

// Rows with a small top-k (the usual setting: top-k 50 with or without top-p and min-p) are shared by several
// workgroups too.  Whatever else is asked, only the k largest logits and their equals can be chosen, and each of them
// is among the k largest of its own stretch of the vocabulary: every part hands over those (its tokens down to the
// bin of its k-th largest, found as the single workgroup finds them, from registers: a thread holds its eight
// tokens), and one workgroup a row then runs the exact thresholds and the draw over what the parts handed over, at
// most kParts x kPartCap candidates in LDS.  The parts and the order of their lists depend on the vocabulary alone,
// not on the rows of the launch.  A part with more candidates than it may hand over (thousands of equal logits), or
// with fewer than k tokens within reach of its largest, marks the row for `sample_kernel`, which runs behind.
constexpr int kSmallK = 64;          // the largest top-k that goes this way
constexpr int kParts = 16;           // parts a row at most
constexpr int kPartTokens = 8 * kBlock;   // tokens a part at most: eight a thread
constexpr int kPartCap = 128;        // candidates a part may hand over
struct PartHead {
    float largest;
    int count;                       // -1: the row goes to sample_kernel
};
__device__ __forceinline__ bool takes_small_k(const FllmSampleRow &p, int vocab) {
    return p.temperature > 1e-5f && p.top_k > 0 && p.top_k <= kSmallK && p.top_k < vocab;
}

__global__ void __launch_bounds__(kBlock)
small_k_parts_kernel(const float *__restrict__ logits, const FllmSampleRow *__restrict__ params, int vocab, int parts, int per_part,
                     float *__restrict__ part_v, int *__restrict__ part_i, PartHead *__restrict__ heads) {
    __shared__ Cells cells;
    __shared__ unsigned long long bins[kBins];
    const int row = blockIdx.x, part = blockIdx.y;
    const FllmSampleRow p = params[row];
    if (!takes_small_k(p, vocab)) return;
    const float *src = logits + (size_t)row * vocab;
    const int lo = part * per_part, hi = min(vocab, lo + per_part);
    float v[8];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int i = lo + (int)threadIdx.x + j * kBlock;
        v[j] = i < hi ? usable(src[i]) : -INFINITY;
        m = fmaxf(m, v[j]);
    }
    m = block_largest(m, cells);
    PartHead *head = heads + (size_t)row * parts + part;
    if (!(m > -INFINITY)) {                      // nothing finite here
        if (threadIdx.x == 0) head->largest = m, head->count = 0;
        return;
    }
    for (int i = threadIdx.x; i < kBins; i += kBlock) bins[i] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 8; j++) {
        if (!(v[j] > -INFINITY)) continue;
        const int b = bin_of(v[j], m);
        if (b < kBins) atomicAdd(&bins[b], 1ull);
    }
    const int last_bin = find_bin(bins, (unsigned long long)p.top_k, cells);
    int mine = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) mine += (v[j] > -INFINITY && bin_of(v[j], m) <= last_bin) ? 1 : 0;
    int count;
    int at = block_exclusive_scan(mine, cells, &count);
    // (with fewer than k tokens within the histogram's reach of the largest, last_bin is kBins and the list is every
    // finite token of the part, as in the single workgroup: handed over if that is few, else the row goes there)
    const bool too_many = count > kPartCap;
    if (threadIdx.x == 0) head->largest = m, head->count = too_many ? -1 : count;
    if (too_many) return;
    float *dst_v = part_v + ((size_t)row * parts + part) * kPartCap;
    int *dst_i = part_i + ((size_t)row * parts + part) * kPartCap;
#pragma unroll
    for (int j = 0; j < 8; j++)
        if (v[j] > -INFINITY && bin_of(v[j], m) <= last_bin) {
            dst_v[at] = v[j];
            dst_i[at] = lo + (int)threadIdx.x + j * kBlock;
            at++;
        }
}

// One workgroup a row.  The parts' candidates together hold the row's k largest logits and their equals, and many
// more (every part gave its own k largest): a histogram over their distance from the row's largest logit finds the
// bin of the k-th, as the single workgroup does over the whole row, and what lies beyond it is dropped before the
// exact thresholds and the draw run over the rest, with the same code.  done[row]: 1 the token is chosen, 0 the
// row is left to sample_kernel.
__global__ void __launch_bounds__(kBlock)
small_k_finish_kernel(const FllmSampleRow *__restrict__ params, int32_t *__restrict__ out, int vocab, int parts,
                      const float *__restrict__ part_v, const int *__restrict__ part_i, const PartHead *__restrict__ heads,
                      int *__restrict__ done) {
    constexpr int kMost = kParts * kPartCap;
    __shared__ Cells cells;
    __shared__ unsigned long long bins[kBins];       // the histogram; afterwards the candidates that are kept
    __shared__ float all_v[kMost];
    __shared__ int all_i[kMost];
    __shared__ int starts[kParts + 1];
    __shared__ int counts[kParts];
    __shared__ float largest_of[kParts];
    const int row = blockIdx.x;
    const FllmSampleRow p = params[row];
    if (!takes_small_k(p, vocab)) return;
    if ((int)threadIdx.x < parts) {
        const PartHead h = heads[(size_t)row * parts + threadIdx.x];
        counts[threadIdx.x] = h.count;
        largest_of[threadIdx.x] = h.largest;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
        bool whole = true;
        for (int q = 0; q < parts; q++) {
            starts[q] = total;
            if (counts[q] < 0) whole = false;
            else total += counts[q];
        }
        starts[parts] = whole ? total : -1;
    }
    __syncthreads();
    const int gathered = starts[parts];
    if (gathered < 0) {
        if (threadIdx.x == 0) done[row] = 0;
        return;
    }
    float m = -INFINITY;
    for (int q = 0; q < parts; q++) m = fmaxf(m, largest_of[q]);
    if (threadIdx.x == 0) done[row] = 1;
    if (!(m > -INFINITY)) {
        if (threadIdx.x == 0) out[row] = 0;   // no finite logit: index 0, as everywhere
        return;
    }
    for (int i = threadIdx.x; i < kBins; i += kBlock) bins[i] = 0;
    {   // every slot of every part's list has a thread: all loads are asked for before the first is stored
        constexpr int kSlots = kMost / kBlock;
        float v[kSlots];
        int id[kSlots], to[kSlots];
#pragma unroll
        for (int j = 0; j < kSlots; j++) {
            const int slot = (int)threadIdx.x + j * kBlock, q = slot / kPartCap, i = slot - q * kPartCap;
            to[j] = (q < parts && i < counts[q]) ? starts[q] + i : -1;
            if (to[j] >= 0) {
                v[j] = part_v[((size_t)row * parts + q) * kPartCap + i];
                id[j] = part_i[((size_t)row * parts + q) * kPartCap + i];
            }
        }
#pragma unroll
        for (int j = 0; j < kSlots; j++)
            if (to[j] >= 0) all_v[to[j]] = v[j], all_i[to[j]] = id[j];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < gathered; i += kBlock) {
        const int b = bin_of(all_v[i], m);
        if (b < kBins) atomicAdd(&bins[b], 1ull);
    }
    const int last_bin = find_bin(bins, (unsigned long long)p.top_k, cells);
    // thread t keeps what it holds of candidates t, t + kBlock, ...: an order that depends on the lists alone
    constexpr int kMine = kMost / kBlock;
    int mine = 0;
#pragma unroll
    for (int j = 0; j < kMine; j++) {
        const int i = (int)threadIdx.x + j * kBlock;
        mine += (i < gathered && bin_of(all_v[i], m) <= last_bin) ? 1 : 0;
    }
    int count;
    int at = block_exclusive_scan(mine, cells, &count);
    float *logit_of = (float *)bins, *weight_of = logit_of + kMost;      // the histogram is done with
    int *token_at = (int *)(weight_of + kMost);
    static_assert(3 * kMost * 4 <= kBins * 8, "the kept candidates fit into the histogram's memory");
    const float inv_t = (float)(1.0 / (double)p.temperature);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kMine; j++) {
        const int i = (int)threadIdx.x + j * kBlock;
        if (i < gathered && bin_of(all_v[i], m) <= last_bin) {
            const float v = all_v[i];
            logit_of[at] = v;
            weight_of[at] = expf((v - m) * inv_t);
            token_at[at] = all_i[i];
            at++;
        }
    }
    __syncthreads();
    const bool use_p = p.top_p > 0.f && p.top_p < 1.f;
    const bool use_m = p.min_p > 0.f;
    const float min_p = use_m ? p.min_p : 0.f;
    if (threadIdx.x < kWave) {
        auto key_at = [&](int i) { return ordered_key(logit_of[i]); };
        auto weight_at = [&](int i) { return weight_of[i]; };
        const uint32_t t = count <= kShortList
                               ? thresholds_of_short_list(key_at, weight_at, count, p.top_k, true, use_p, p.top_p, min_p, 0.0)
                               : thresholds<OneWave>(key_at, weight_at, count, p.top_k, true, use_p, p.top_p, min_p, 0.0, cells);
        if (threadIdx.x == 0) cells.key = t;
    }
    __syncthreads();
    const uint32_t threshold = cells.key;
    Pick best = {-INFINITY, kNone};
    for (int i = threadIdx.x; i < count; i += kBlock) {
        const float v = logit_of[i];
        if (ordered_key(v) < threshold) continue;
        if (use_m && weight_of[i] < min_p) continue;
        const int id = token_at[i];
        const float u = uniform_of(p.seed, p.draw, (uint32_t)id);
        const Pick here = {(v - m) * inv_t - logf(-logf(u)), id};
        best = better_of(best, here);
    }
    best = block_best(best, cells);
    if (threadIdx.x == 0) out[row] = token_of(best);
}

// `work` gives every row `vocab` 32-bit words of its own (the list of token ids); it must not overlap the logits.
// `skip_draws_from_all`: rows with a temperature and no filter are left to `draw_from_all_kernel`.
// `small_k_done`: rows with a small top-k whose entry is 1 have their token already (`small_k_finish_kernel`).
__global__ void __launch_bounds__(kBlock)
sample_kernel(const float *__restrict__ logits, float *__restrict__ work, const FllmSampleRow *__restrict__ params,
              int32_t *__restrict__ out, int vocab, int skip_draws_from_all, const int *__restrict__ small_k_done) {
    __shared__ Cells cells;
    __shared__ unsigned long long bins[kBins];       // the histogram; afterwards the staged candidates
    const int row = blockIdx.x;
    const FllmSampleRow p = params[row];
    if (skip_draws_from_all && draws_from_all(p, vocab)) return;
    if (small_k_done != nullptr && takes_small_k(p, vocab) && small_k_done[row] != 0) return;
    const float *src = logits + (size_t)row * vocab;
    if (p.temperature <= 1e-5f) {
        const Pick best = block_best(best_in_range(src, 0, vocab), cells);
        if (threadIdx.x == 0) out[row] = token_of(best);
        return;
    }
    int *list = (int *)(work + (size_t)row * vocab);
    float m = -INFINITY;
    for_each_token(src, vocab, [&](int, float v) { m = fmaxf(m, usable(v)); });
    m = block_largest(m, cells);
    if (!(m > -INFINITY)) {
        if (threadIdx.x == 0) out[row] = 0;   // no finite logit: the reference's argmax gives index 0 as well
        return;
    }
    const float inv_t = (float)(1.0 / (double)p.temperature);
    const bool use_k = p.top_k > 0 && p.top_k < vocab;
    const bool use_p = p.top_p > 0.f && p.top_p < 1.f;
    const bool use_m = p.min_p > 0.f;
    const float min_p = use_m ? p.min_p : 0.f;
    // min-p keeps the tokens with exp((v - max) / T) >= min_p: none of them lies below this bin (one to spare for rounding)
    int min_p_bin = kBins;
    if (use_m) {
        const float reach = -logf(min_p) * p.temperature;      // max - v of the lightest token that stays, about
        min_p_bin = reach < 63.f ? min(kBins, bin_of(m - reach, m) + 1) : kBins;
    }
    int count = vocab;                       // tokens the draw looks at: all of them, or the list
    uint32_t threshold = 0;                  // key below which a listed token is out
    if (use_k || use_p || use_m) {
        for (int i = threadIdx.x; i < kBins; i += kBlock) bins[i] = 0;
        __syncthreads();
        double total = 0.0;                  // mass of all finite logits (top-p without top-k)
        unsigned long long reach = 0;        // what this thread put into the histogram, in its units (top-p)
        unsigned long long all_units = 0;    // the same over the workgroup
        if (use_k || use_p) for_each_token(src, vocab, [&](int, float raw) {
            const float v = usable(raw);
            if (!(v > -INFINITY)) return;
            const int b = bin_of(v, m);
            if (use_k) {
                if (b < kBins) atomicAdd(&bins[b], 1ull);
            } else {
                const float e = expf((v - m) * inv_t);
                total += (double)e;
                const unsigned long long fixed = units_of(e);
                reach += fixed;
                if (b < kBins && fixed != 0) atomicAdd(&bins[b], fixed);
            }
        });
        int last_bin = kBins;
        if (use_k) {
            last_bin = find_bin(bins, (unsigned long long)p.top_k, cells);
        } else if (use_p) {
            total = WholeBlock::sum(total, cells);
            // the sum of every thread's share, far tokens included: integers, the same in any order
            all_units = block_units(reach, cells);
            last_bin = find_bin(bins, (unsigned long long)((double)p.top_p * (double)all_units), cells);
            if (last_bin < kBins) last_bin++;   // a bin to spare: the histogram's sums are rounded, the exact ones decide
        }
        last_bin = min(last_bin, min_p_bin);    // what every filter keeps lies within what any one of them keeps
        // gather the tokens up to that bin: thread t's tokens in the order it meets them, behind those of the threads before it
        int mine = 0;
        for_each_token(src, vocab, [&](int, float raw) {
            const float v = usable(raw);
            mine += (v > -INFINITY && bin_of(v, m) <= last_bin) ? 1 : 0;
        });
        int at = block_exclusive_scan(mine, cells, &count);
        for_each_token(src, vocab, [&](int token, float raw) {
            const float v = usable(raw);
            if (v > -INFINITY && bin_of(v, m) <= last_bin) list[at++] = token;
        });
        __syncthreads();                     // the list is written (global memory, read back by other threads below)
        if (count <= kStaged) {
            // the histogram is done with: its memory takes the candidates' logits and weights, and one wave finds both thresholds
            float *logit_of = (float *)bins, *weight_of = logit_of + kStaged;
            for (int i = threadIdx.x; i < count; i += kBlock) {
                const float v = usable(src[list[i]]);
                logit_of[i] = v;
                weight_of[i] = expf((v - m) * inv_t);
            }
            __syncthreads();
            if (threadIdx.x < kWave) {
                auto key_at = [&](int i) { return ordered_key(logit_of[i]); };
                auto weight_at = [&](int i) { return weight_of[i]; };
                const uint32_t t = count <= kShortList
                                       ? thresholds_of_short_list(key_at, weight_at, count, p.top_k, use_k, use_p, p.top_p, min_p, total)
                                       : thresholds<OneWave>(key_at, weight_at, count, p.top_k, use_k, use_p, p.top_p, min_p, total, cells);
                if (threadIdx.x == 0) cells.key = t;
            }
            __syncthreads();
            threshold = cells.key;
        } else {
            // a long list: histograms over the keys' bits, weights in units of 2^-40 (the histogram's memory again)
            auto key_at = [&](int i) { return ordered_key(usable(src[list[i]])); };
            auto weight_at = [&](int i) { return expf((usable(src[list[i]]) - m) * inv_t); };
            // top-p looks at what top-k and min-p left: a candidate below min_p has key 0 there
            auto heavy_key_at = [&](int i) {
                const float v = usable(src[list[i]]);
                return expf((v - m) * inv_t) >= min_p ? ordered_key(v) : 0u;
            };
            const uint32_t t = threshold_of_long_list(key_at, weight_at, heavy_key_at, count, p.top_k, use_k, use_p, use_m, p.top_p,
                                                      all_units, bins, cells);
            threshold = t;
        }
    }
    // Gumbel-max over what is left: the largest of (v - max) / T - ln(-ln u), u the token's uniform number
    Pick best = {-INFINITY, kNone};
    const bool whole = !(use_k || use_p || use_m);
    for (int i = threadIdx.x; i < count; i += kBlock) {
        const int id = whole ? i : list[i];
        const float v = usable(src[id]);
        if (!(v > -INFINITY) || ordered_key(v) < threshold) continue;
        if (use_m && expf((v - m) * inv_t) < min_p) continue;
        const float u = uniform_of(p.seed, p.draw, (uint32_t)id);
        const Pick here = {(v - m) * inv_t - logf(-logf(u)), id};
        best = better_of(best, here);
    }
    best = block_best(best, cells);
    if (threadIdx.x == 0) out[row] = token_of(best);
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

// ---------------------------------------------------------------------------------------------
// What a request asks to be done to its logits before a token is chosen
// ---------------------------------------------------------------------------------------------
// The reference's order (rust/engine/src/sampling.rs:220-229, :252-274): ids that may not be chosen yet go to -inf;
// every token seen before is penalised once (divided by the repetition penalty when its logit is positive,
// multiplied otherwise; then presence + frequency * count taken off); biases are added.  The host lists the tokens
// seen with their counts; the token that the step before chose may still be on the device only (steps launched
// ahead): `last_tokens[last_row]` then counts once more, as an entry of its own if the list does not hold it.
namespace {
constexpr int kAdjustBlock = 256;

__device__ __forceinline__ float penalised(float v, const FllmAdjustRow &a, int count) {
    if (fabsf(a.repetition_penalty - 1.f) >= 1e-5f) v = v > 0.f ? v / a.repetition_penalty : v * a.repetition_penalty;
    return v - (a.presence_penalty + a.frequency_penalty * (float)count);
}

__global__ void __launch_bounds__(kAdjustBlock)
adjust_logits_kernel(float *__restrict__ logits, int vocab, const FllmAdjustRow *__restrict__ rows, const FllmAdjustLists lists,
                     const int32_t *__restrict__ last_tokens) {
    __shared__ int last_was_listed;
    const FllmAdjustRow a = rows[blockIdx.x];
    float *w = logits + (size_t)blockIdx.x * vocab;
    const int last = a.last_row >= 0 ? last_tokens[a.last_row] : -1;
    if (threadIdx.x == 0) last_was_listed = 0;
    __syncthreads();
    for (int j = threadIdx.x; j < a.seen_len; j += kAdjustBlock) {        // ids of a row are distinct: no two threads meet
        const int id = lists.seen_ids[a.seen_off + j];
        if (id < 0 || id >= vocab) continue;
        int count = lists.seen_counts[a.seen_off + j];
        if (id == last) count++, last_was_listed = 1;
        w[id] = penalised(w[id], a, count);
    }
    __syncthreads();
    if (threadIdx.x == 0 && last >= 0 && last < vocab && !last_was_listed) w[last] = penalised(w[last], a, 1);
    __syncthreads();
    for (int j = threadIdx.x; j < a.bias_len; j += kAdjustBlock) {
        const int id = lists.bias_ids[a.bias_off + j];
        if (id >= 0 && id < vocab) w[id] += lists.bias_values[a.bias_off + j];
    }
    __syncthreads();
    for (int j = threadIdx.x; j < a.blocked_len; j += kAdjustBlock) {
        const int id = lists.blocked_ids[a.blocked_off + j];
        if (id >= 0 && id < vocab) w[id] = -INFINITY;
    }
    for (int j = threadIdx.x; j < a.pairs_len; j += kAdjustBlock) {
        const int id = lists.then_blocked[a.pairs_off + j];
        if (lists.if_last[a.pairs_off + j] == last && id >= 0 && id < vocab) w[id] = -INFINITY;
    }
    if (a.allowed_len > 0) {                       // every token that is not on the rising list
        const int32_t *allowed = lists.allowed_ids + a.allowed_off;
        for (int i = threadIdx.x; i < vocab; i += kAdjustBlock) {
            int lo = 0, hi = a.allowed_len;        // the first entry >= i lies in [lo, hi]
            while (lo < hi) {
                const int mid = (lo + hi) / 2;
                if (allowed[mid] < i) lo = mid + 1; else hi = mid;
            }
            if (lo == a.allowed_len || allowed[lo] != i) w[i] = -INFINITY;
        }
    }
}

// Log-probabilities in the distribution the model gave, the softmax of the logits as they are handed in
// (rust/engine/src/sampling.rs:937-965): of the token that was chosen for the row and of the `top` likeliest tokens,
// the lower id first among equals.  One workgroup a wanted row.  values[0] belongs to the chosen token, values[1..]
// and ids[1..] to the likeliest ones; ids[0] repeats the chosen token.  A row with a NaN or +inf, or with no finite
// value at all, has no distribution: all its values are NaN and its ids -1.
//
// Three passes over the row whatever `top` is: the largest value; the mass and a histogram of token counts over the
// distance from the largest value; the tokens down to the bin in which the `top`-th lies, gathered into LDS, from
// which the picks are then taken.  Where that list would not fit (thousands of tokens in the leading bins) or the
// histogram does not reach `top` tokens (-inf nearly everywhere), every pick is a pass over the row instead.
constexpr int kListed = 2048;
__global__ void __launch_bounds__(kBlock)
logprobs_kernel(const float *__restrict__ logits, int vocab, const int32_t *__restrict__ rows, const int32_t *__restrict__ tokens,
                int top, float *__restrict__ values, int32_t *__restrict__ ids) {
    __shared__ Cells cells;
    __shared__ unsigned long long bins[kBins];
    __shared__ float listed_v[kListed];
    __shared__ int listed_i[kListed];
    __shared__ int listed;
    const int row = rows[blockIdx.x];
    const float *w = logits + (size_t)row * vocab;
    float *out_v = values + (size_t)blockIdx.x * (1 + top);
    int32_t *out_i = ids + (size_t)blockIdx.x * (1 + top);
    float largest = -INFINITY;
    int bad = 0;
    for_each_token(w, vocab, [&](int, float v) {
        bad |= (v != v) || v == INFINITY;
        if (v > largest) largest = v;
    });
    largest = block_largest(largest, cells);
    bad = WholeBlock::sum(bad, cells) != 0 || !(fabsf(largest) < INFINITY);
    for (int i = threadIdx.x; i < kBins; i += kBlock) bins[i] = 0;
    if (threadIdx.x == 0) listed = 0;
    __syncthreads();
    double mass = 0.0;
    if (!bad)
        for_each_token(w, vocab, [&](int, float v) {
            mass += (double)__expf(v - largest);
            if (top > 0 && v > -INFINITY) {
                const int b = bin_of(v, largest);
                if (b < kBins) atomicAdd(&bins[b], 1ull);
            }
        });
    const float log_mass = (float)log(WholeBlock::sum(mass, cells));
    const int token = tokens[row];
    if (threadIdx.x == 0) {
        out_i[0] = token;
        out_v[0] = bad || token < 0 || token >= vocab ? NAN : (w[token] - largest) - log_mass;
    }
    if (top == 0) return;
    if (bad) {
        for (int k = 1 + (int)threadIdx.x; k <= top; k += kBlock) out_i[k] = -1, out_v[k] = NAN;
        return;
    }
    unsigned long long before = 0;
    const int last_bin = find_bin(bins, (unsigned long long)top, cells, &before);
    const bool from_list = last_bin < kBins && before + bins[last_bin] <= (unsigned long long)kListed;
    __syncthreads();
    if (from_list) {
        for_each_token(w, vocab, [&](int i, float v) {
            if (v > -INFINITY && bin_of(v, largest) <= last_bin) {
                const int at = atomicAdd(&listed, 1);
                listed_v[at] = v;
                listed_i[at] = i;
            }
        });
        __syncthreads();
    }
    const int count = listed;
    Pick last = {INFINITY, -1};                   // everything comes after this
    for (int k = 1; k <= top; k++) {
        Pick mine = {-INFINITY, kNone};
        auto offer = [&](int i, float v) {
            const bool after_last = v < last.value || (v == last.value && i > last.index);
            if (after_last && (v > mine.value || (v == mine.value && i < mine.index) || mine.index == kNone)) {
                mine.value = v;
                mine.index = i;
            }
        };
        if (from_list) {
            for (int j = threadIdx.x; j < count; j += kBlock) offer(listed_i[j], listed_v[j]);
        } else {
            for_each_token(w, vocab, offer);
        }
        last = block_best(mine, cells);
        if (threadIdx.x == 0) {
            out_i[k] = last.index == kNone ? -1 : last.index;
            out_v[k] = last.index == kNone ? NAN : (last.value - largest) - log_mass;
        }
        if (last.index == kNone) last.value = -INFINITY;      // nothing is left: the rest stays empty
    }
}
// Log-probabilities in the distribution a token was drawn from (rust/engine/src/sampling.rs, `logprobs_processed` and
// `processed_distribution`; its test :1542-1556): the softmax of logits / T over the tokens that top-k, min-p and top-p
// leave, in that order and with the ties kept as the sampler keeps them; a greedy row is a point mass on the first
// largest logit.  `logits` are the ones the sampler saw (penalties and biases applied).  values[0] belongs to the chosen
// token (-inf if the filters leave it out), values[1..] and ids[1..] to the likeliest of the tokens that are left, fewer
// than `top` if fewer are left (then ids -1, values NaN).  One workgroup a wanted row; the thresholds are found as
// `sample_kernel` finds them for a list that does not fit into LDS (histograms over the keys' bits), over the whole row.
__global__ void __launch_bounds__(kBlock)
processed_logprobs_kernel(const float *__restrict__ logits, int vocab, const int32_t *__restrict__ rows, const int32_t *__restrict__ tokens,
                          const FllmSampleRow *__restrict__ params, int top, float *__restrict__ values, int32_t *__restrict__ ids) {
    __shared__ Cells cells;
    __shared__ unsigned long long bins[kBins];
    const int row = rows[blockIdx.x];
    const FllmSampleRow p = params[row];
    const float *src = logits + (size_t)row * vocab;
    float *out_v = values + (size_t)blockIdx.x * (1 + top);
    int32_t *out_i = ids + (size_t)blockIdx.x * (1 + top);
    const int token = tokens[row];
    float m = -INFINITY;
    for_each_token(src, vocab, [&](int, float v) { m = fmaxf(m, usable(v)); });
    m = block_largest(m, cells);
    if (!(m > -INFINITY)) {      // no finite logit: no distribution
        for (int k = threadIdx.x; k <= top; k += kBlock) out_i[k] = k == 0 ? token : -1, out_v[k] = NAN;
        return;
    }
    const bool greedy = !(p.temperature > 1e-5f);
    const float inv_t = greedy ? 1.0f : (float)(1.0 / (double)p.temperature);
    const bool use_k = !greedy && p.top_k > 0 && p.top_k < vocab;
    const bool use_p = !greedy && p.top_p > 0.f && p.top_p < 1.f;
    const bool use_m = !greedy && p.min_p > 0.f;
    const float min_p = use_m ? p.min_p : 0.f;
    auto key_at = [&](int i) {
        const float v = usable(src[i]);
        return v > -INFINITY ? ordered_key(v) : 0u;      // key 0: not a candidate
    };
    auto weight_at = [&](int i) { return expf((usable(src[i]) - m) * inv_t); };
    auto heavy_key_at = [&](int i) {
        const float v = usable(src[i]);
        return (v > -INFINITY && expf((v - m) * inv_t) >= min_p) ? ordered_key(v) : 0u;
    };
    uint32_t threshold = 0;
    if (greedy) {
        threshold = ordered_key(m);                      // the largest logit alone; among equals the first (below)
    } else if (use_k || use_p) {
        unsigned long long mine = 0;
        if (use_p && !use_k && !use_m)
            for (int i = threadIdx.x; i < vocab; i += kBlock)
                if (key_at(i) != 0) mine += units_of(weight_at(i));
        const unsigned long long all_units = block_units(mine, cells);
        threshold = threshold_of_long_list(key_at, weight_at, heavy_key_at, vocab, p.top_k, use_k, use_p, use_m, p.top_p, all_units,
                                           bins, cells);
    }
    // what is left, and its mass
    auto left = [&](int i, float v) { return v > -INFINITY && ordered_key(v) >= threshold && (!use_m || expf((v - m) * inv_t) >= min_p); };
    double mass = 0.0;
    Pick first = {-INFINITY, kNone};
    for (int i = threadIdx.x; i < vocab; i += kBlock) {
        const float v = usable(src[i]);
        if (!left(i, v)) continue;
        mass += (double)expf((v - m) * inv_t);
        first = better_of(first, Pick{v, i});
    }
    first = block_best(first, cells);
    const float log_mass = greedy ? 0.f : (float)log(WholeBlock::sum(mass, cells));
    auto value_of = [&](int i, float v) { return greedy ? 0.f : (v - m) * inv_t - log_mass; };
    if (threadIdx.x == 0) {
        const float v = token >= 0 && token < vocab ? usable(src[token]) : -INFINITY;
        const bool in = token >= 0 && token < vocab && left(token, v) && (!greedy || token == first.index);
        out_i[0] = token;
        out_v[0] = in ? value_of(token, v) : -INFINITY;
    }
    Pick last = {INFINITY, -1};                   // everything comes after this
    for (int k = 1; k <= top; k++) {
        Pick mine = {-INFINITY, kNone};
        if (!(greedy && k > 1))
            for (int i = threadIdx.x; i < vocab; i += kBlock) {
                const float v = usable(src[i]);
                if (!left(i, v)) continue;
                const bool after_last = v < last.value || (v == last.value && i > last.index);
                if (after_last && (v > mine.value || (v == mine.value && i < mine.index) || mine.index == kNone)) mine = Pick{v, i};
            }
        last = block_best(mine, cells);
        if (threadIdx.x == 0) {
            out_i[k] = last.index == kNone ? -1 : last.index;
            out_v[k] = last.index == kNone ? NAN : value_of(last.index, last.value);
        }
        if (last.index == kNone) last.value = -INFINITY;      // nothing is left: the rest stays empty
    }
}
}  // namespace

extern "C" int fllm_logprobs_processed(const float *logits, int rows, int vocab, const int32_t *wanted_rows, int wanted,
                                       const int32_t *tokens, const FllmSampleRow *params, int top, float *values, int32_t *ids,
                                       hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && vocab > 0 && wanted >= 0, "logprobs_processed: bad sizes rows=%d vocab=%d wanted=%d", rows, vocab, wanted);
    FLLM_REQUIRE(top >= 0 && top <= 20 && top <= vocab, "logprobs_processed: %d alternatives asked for, at most min(20, vocabulary) are given", top);
    if (wanted == 0) return 0;
    FLLM_REQUIRE(logits != nullptr && wanted_rows != nullptr && tokens != nullptr && params != nullptr && values != nullptr && ids != nullptr,
                 "logprobs_processed: logits, rows, tokens, sampling records and both outputs are required");
    hipLaunchKernelGGL(processed_logprobs_kernel, dim3(wanted), dim3(kBlock), 0, stream, logits, vocab, wanted_rows, tokens, params, top,
                       values, ids);
    return fllm_check_launch("logprobs_processed");
}

extern "C" int fllm_logprobs(const float *logits, int rows, int vocab, const int32_t *wanted_rows, int wanted,
                             const int32_t *tokens, int top, float *values, int32_t *ids, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && vocab > 0 && wanted >= 0, "logprobs: bad sizes rows=%d vocab=%d wanted=%d", rows, vocab, wanted);
    FLLM_REQUIRE(top >= 0 && top <= 20 && top <= vocab, "logprobs: %d alternatives asked for, at most min(20, vocabulary) are given", top);
    if (wanted == 0) return 0;
    FLLM_REQUIRE(logits != nullptr && wanted_rows != nullptr && tokens != nullptr && values != nullptr && ids != nullptr,
                 "logprobs: logits, rows, tokens and both outputs are required");
    hipLaunchKernelGGL(logprobs_kernel, dim3(wanted), dim3(kBlock), 0, stream, logits, vocab, wanted_rows, tokens, top, values, ids);
    return fllm_check_launch("logprobs");
}

extern "C" int fllm_adjust_logits(float *logits, int rows, int vocab, const FllmAdjustRow *row_records, const FllmAdjustLists *lists,
                                  const int32_t *last_tokens, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && vocab > 0, "adjust_logits: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    FLLM_REQUIRE(logits != nullptr && row_records != nullptr && lists != nullptr, "adjust_logits: logits, row records and lists are required");
    hipLaunchKernelGGL(adjust_logits_kernel, dim3(rows), dim3(kAdjustBlock), 0, stream, logits, vocab, row_records, *lists, last_tokens);
    return fllm_check_launch("adjust_logits");
}

extern "C" int fllm_sample(const float *logits, float *work, const FllmSampleRow *params, int32_t *out, int rows,
                           int vocab, int kinds, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    FLLM_REQUIRE(work != nullptr && params != nullptr, "sample: work and params are required");
    FLLM_REQUIRE(kinds >= 1 && kinds <= 7,
                 "sample: kinds %d is no sum of 1 (rows that draw from all tokens), 2 (other rows), 4 (rows with a top-k of at most 64 among them)",
                 kinds);
    if (rows == 0) return 0;
    // rows with a temperature and no filter: several workgroups a row, if the device workspace is there to meet in
    void *ws = nullptr;
    size_t ws_bytes = 0;
    int parts = (vocab + 8191) / 8192;
    if (parts > 64) parts = 64;
    if (parts * rows > 2048) parts = 2048 / rows;
    const bool have_ws = fllm_device_workspace(&ws, &ws_bytes);
    if (!have_ws) ws = nullptr, ws_bytes = 0;
    const bool split = (kinds & 1) && parts > 1 && have_ws &&
                       (size_t)rows * sizeof(int) <= kWorkspaceCounterBytes &&
                       kWorkspaceCounterBytes + (size_t)rows * parts * 8 + (size_t)rows * 4 <= ws_bytes;
    if (split) {
        const int per_part = (vocab + parts - 1) / parts;
        float *pv = (float *)((unsigned char *)ws + kWorkspaceCounterBytes);
        int *pi = (int *)(pv + (size_t)rows * parts);
        float *row_max = (float *)(pi + (size_t)rows * parts);
        hipLaunchKernelGGL(draw_from_all_kernel<0>, dim3(rows, parts), dim3(kBlock), 0, stream, logits, params, out, vocab, parts,
                           per_part, pv, pi, (int *)ws, row_max);
        hipLaunchKernelGGL(draw_from_all_kernel<1>, dim3(rows, parts), dim3(kBlock), 0, stream, logits, params, out, vocab, parts,
                           per_part, pv, pi, (int *)ws, row_max);
        if (!(kinds & 6)) return fllm_check_launch("sample");
    }
    // rows with a small top-k: the parts of a row in workgroups of their own, then one workgroup a row; what they
    // leave undone (done[row] 0) and every other row is sample_kernel's.  Behind the partial results of the rows that
    // draw from all tokens in the workspace: lists, their heads, the rows' marks.
    const int *small_k_done = nullptr;
    const int k_parts = (vocab + kPartTokens - 1) / kPartTokens;
    if ((kinds & 4) && k_parts >= 2 && k_parts <= kParts && ws != nullptr) {
        const int per_part = (vocab + k_parts - 1) / k_parts;       // <= kPartTokens
        size_t at = kWorkspaceCounterBytes + (size_t)rows * parts * 8 + (size_t)rows * 4;
        at = (at + 255) / 256 * 256;
        const size_t lists = (size_t)rows * k_parts * kPartCap;
        if (at + lists * 8 + (size_t)rows * k_parts * sizeof(PartHead) + (size_t)rows * 4 <= ws_bytes) {
            float *part_v = (float *)((unsigned char *)ws + at);
            int *part_i = (int *)(part_v + lists);
            PartHead *heads = (PartHead *)(part_i + lists);
            int *done = (int *)(heads + (size_t)rows * k_parts);
            hipLaunchKernelGGL(small_k_parts_kernel, dim3(rows, k_parts), dim3(kBlock), 0, stream, logits, params, vocab, k_parts,
                               per_part, part_v, part_i, heads);
            hipLaunchKernelGGL(small_k_finish_kernel, dim3(rows), dim3(kBlock), 0, stream, params, out, vocab, k_parts, part_v,
                               part_i, heads, done);
            small_k_done = done;
        }
    }
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kBlock), 0, stream, logits, work, params, out, vocab, split ? 1 : 0,
                       small_k_done);
    return fllm_check_launch("sample");
}
