// How the kernels that meet across workgroups are launched: K slices, grid sizes, LDS bytes, where partial results
// lie in the device workspace.  Plain C++ without a device type in it, so that the same code that the launchers run
// is also compiled for the host alone and swept over shapes under the address and undefined-behaviour sanitizers
// (a mistake here is an access outside LDS or outside the workspace on the device).
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace fllm_plan {

constexpr size_t kLdsBytes = 160 * 1024;            // LDS of a compute unit
constexpr size_t kCounterBytes = 64 * 1024;         // the counters at the start of the device workspace
constexpr int kWaveLanes = 64;
constexpr size_t kBf16 = 2, kF32 = 4, kF32x4 = 16;

inline long ceil_div(long a, long b) { return (a + b - 1) / b; }

// ---- products of up to 16 rows: activations of a K slice resident in LDS, waves split the slice ----
struct ResidentPlan {
    int S = 0, slice = 0, waves = 8, per_cu = 0;      // S == 0: no plan
    size_t stage = 0, red = 0, smem = 0;
};
constexpr int kMaxSlices = 32;

// bytes of the workspace that S slices of `ntiles` tiles need, counters included: partial sums [tile][slice][rt][64][4]
// and sums of squares [tile][slice][16]
inline size_t resident_workspace_need(int ntiles, int S, int rt) {
    return kCounterBytes + (size_t)ntiles * S * ((size_t)rt * kWaveLanes * 4 + 16) * kF32;
}
inline size_t resident_ssq_offset_floats(int ntiles, int S, int rt) { return (size_t)ntiles * S * rt * kWaveLanes * 4; }

// The fewest K slices whose activations fit into LDS (slicing costs more than it gains wherever it is not needed):
// twice into a compute unit's as two workgroups of 8 waves, else once as one workgroup of 16 waves, so that as
// many loads are in flight.  `forced`: 0, or the number of slices asked for by hand.
inline ResidentPlan plan_resident(int M, int K, int ntiles, int rt, size_t ws_bytes, bool have_ws, bool x_direct, int forced) {
    ResidentPlan best;
    if (x_direct) {   // nothing is staged: one slice, two workgroups of 8 waves a compute unit
        best.S = 1;
        best.slice = (K + 127) / 128 * 128;
        best.waves = 8;
        best.per_cu = 2;
        best.stage = 0;
        best.red = 8 * kWaveLanes * kF32x4;
        best.smem = best.red + 8 * 16 * kF32;
        return best;
    }
    for (int S = 1; S <= kMaxSlices; S *= 2) {
        const int slice = ((K + S - 1) / S + 127) / 128 * 128;
        if (S > 1 && (slice < 1024 || (long)(S - 1) * slice >= K)) break;
        if (S > 1) {
            if (!have_ws || resident_workspace_need(ntiles, S, rt) > ws_bytes || (size_t)ntiles * sizeof(int) > kCounterBytes) break;
        }
        ResidentPlan p;
        p.S = S;
        p.slice = slice;
        p.stage = ((size_t)M * (slice + 8) * kBf16 + 15) / 16 * 16;
        const size_t small = p.stage + 8 * (kWaveLanes * kF32x4 + 16 * kF32);
        const size_t large = p.stage + 16 * (kWaveLanes * kF32x4 + 16 * kF32);
        if (small <= 76 * 1024) p.waves = 8, p.per_cu = 2, p.smem = small;
        else if (large <= kLdsBytes) p.waves = 16, p.per_cu = 1, p.smem = large;
        else continue;
        p.red = (size_t)p.waves * kWaveLanes * kF32x4;
        if (forced == 0 || S == forced || best.S == 0) best = p;
        if (forced == 0 || S == forced) break;
    }
    return best;
}

// workgroups of a resident launch: one per slot of the device and slice, no more than there are tiles
inline int resident_groups(const ResidentPlan &p, int ntiles, int cus) {
    int groups = cus * p.per_cu / p.S;
    if (groups < 1) groups = 1;
    if (groups > ntiles) groups = ntiles;
    // no more workgroups than give every one the same number of tiles: 1,792 tiles on 512 slots are 448 workgroups of 4
    // tiles, not 256 of 4 beside 256 of 3 that wait for them (gate/up of the 8B sizes at 8 rows: 40.2 -> 39.6 us)
    const int rounds = (ntiles + groups - 1) / groups;
    groups = (ntiles + rounds - 1) / rounds;
    return groups;       // the grid is groups * S
}

// ---- products of 17 to 64 rows, activations in chunks through LDS ----
struct ChunkPlan {
    int S = 1, slice = 0, grid = 0, waves = 4;
};
inline size_t chunk_workspace_need(int ntiles, int S, int mt, int rt) {
    return kCounterBytes + (size_t)ntiles * S * mt * rt * kWaveLanes * 4 * kF32;
}
// `waves`: row tiles (waves) of a workgroup; a compute unit holds eight waves of this kernel, two workgroups of four or
// one of five to eight
inline ChunkPlan plan_chunks(int K, int ntiles, int mt, int rt, size_t ws_bytes, bool have_ws, int cus, int forced, int waves = 4) {
    const int ngroups = (ntiles + waves - 1) / waves;
    const int slots = 8 / waves * cus;
    // K slices: as many as fill the chip with the row groups there are, each at least two chunks long
    int S = 1;
    while (S < 8 && ngroups * S * 2 <= slots && (K + 2 * S - 1) / (2 * S) >= 512) S *= 2;
    if (forced > 0) S = forced;
    while (S > 1) {
        const size_t need = chunk_workspace_need(ntiles, S, mt, rt);      // the kernel's offsets into it are 32 bits
        if (have_ws && need <= ws_bytes && need - kCounterBytes <= 0x7fffffffu && (size_t)ntiles * sizeof(int) <= kCounterBytes &&
            (K + S - 1) / S >= 256)
            break;
        S /= 2;
    }
    ChunkPlan p;
    p.waves = waves;
    p.S = S;
    p.slice = ((K + S - 1) / S + 255) / 256 * 256;
    if (S > 1 && (long)(S - 1) * p.slice >= K) p.S = S = (K + p.slice - 1) / p.slice;   // no empty slice
    int per_slice = slots / S;
    if (per_slice < 1) per_slice = 1;
    if (per_slice > ngroups) per_slice = ngroups;
    p.grid = per_slice * S;
    return p;
}
// What the busiest compute unit streams under a plan, in weight rows x columns: its workgroups' row tiles over their
// slices, as often as the row groups of a slice come round.
inline long chunk_plan_cost(const ChunkPlan &p, int ntiles) {
    const int ngroups = (ntiles + p.waves - 1) / p.waves;
    const int per_slice = p.grid / p.S;
    const long rounds = (ngroups + per_slice - 1) / per_slice;
    return rounds * (8 / p.waves) * p.waves * (long)p.slice;
}
// The number of waves (four, seven or eight) whose plan leaves the least to the busiest compute unit; on a tie four,
// but see below.
// 1,792 tiles over 256 compute units are seven a unit: workgroups of seven waves take a tile each in one round, where
// four or eight waves leave an eighth of the device idle in the last round.
inline ChunkPlan plan_chunks_balanced(int K, int ntiles, int mt, int rt, size_t ws_bytes, bool have_ws, int cus, int forced,
                                      int forced_waves) {
    if (forced_waves == 4 || forced_waves == 7 || forced_waves == 8)
        return plan_chunks(K, ntiles, mt, rt, ws_bytes, have_ws, cus, forced, forced_waves);
    ChunkPlan best = plan_chunks(K, ntiles, mt, rt, ws_bytes, have_ws, cus, forced, 4);
    long best_cost = chunk_plan_cost(best, ntiles);
    for (int waves = 7; waves <= 8; waves++) {
        const ChunkPlan p = plan_chunks(K, ntiles, mt, rt, ws_bytes, have_ws, cus, forced, waves);
        const long cost = chunk_plan_cost(p, ntiles);
        // a tie between four and eight waves, no slices either way, three or four row tiles of activations: eight waves
        // share one copy of a chunk in LDS where two workgroups of four hold one each (the vocabulary projection at
        // 64 rows: 207 -> 194 us)
        const bool shares = waves == 8 && cost == best_cost && mt >= 3 && p.S == 1 && best.S == 1 && best.waves == 4;
        if (cost < best_cost || shares) best = p, best_cost = cost;
    }
    return best;
}

// ---- products of 17 to 64 rows, a K slice of the activations resident in LDS ----
struct SlabPlan {
    int S = 0, slice = 0, grid = 0;       // S == 0: no plan
    size_t smem = 0, cells_off = 0;
};
inline size_t slab_workspace_need(int ntiles, int S, int mt, int rt) {
    return kCounterBytes + (size_t)ntiles * S * ((size_t)mt * rt * kWaveLanes * 4 + (size_t)mt * 16) * kF32;
}
inline size_t slab_ssq_offset_floats(int ntiles, int S, int mt, int rt) { return (size_t)ntiles * S * mt * rt * kWaveLanes * 4; }

// The slice length (256 to 1,024 columns; multiples of 512 for the norm prologue, whose sums of squares are kept per
// 512 columns) that costs a workgroup the fewest bytes: its items' weights, its staged slice, and its share of the
// partial sums that slices cost.
inline SlabPlan plan_slab(int M, int n_tiles, int K, int mt, int rt, bool norm, int nt, size_t ws_bytes, bool have_ws, int cus,
                          int forced) {
    SlabPlan best;
    double best_cost = 0.0;
    const int rows = mt * 16;
    const int ngroups = (n_tiles + 7) / 8;
    for (int slice = 1024; slice >= 256; slice -= 256) {
        if (norm && slice % 512 != 0) continue;
        int S = (K + slice - 1) / slice;
        int len = slice;
        const int step = norm ? 512 : 256;
        if (S == 1) len = (K + step - 1) / step * step;   // one slice: no longer than K needs
        if (forced > 0 && S != forced) continue;
        SlabPlan p;
        p.S = S;
        p.slice = len;
        p.cells_off = ((size_t)rows * (len + 8) * kBf16 + 15) / 16 * 16;
        p.smem = p.cells_off + (norm ? (size_t)rows * ((len + 511) / 512) * kF32 : 0);
        if (p.smem > kLdsBytes) continue;
        if (S > 1) {
            if (!have_ws || slab_workspace_need(n_tiles, S, mt, rt) > ws_bytes || (size_t)n_tiles * sizeof(int) > kCounterBytes) continue;
            if ((slab_workspace_need(n_tiles, S, mt, rt) - kCounterBytes) > 0x7fffffffu) continue;   // offsets of the 16-byte pieces are 32 bits
        }
        int per_slice = cus / S;
        if (per_slice < 1) per_slice = 1;
        if (per_slice > ngroups) per_slice = ngroups;
        p.grid = per_slice * S;
        const int items = (ngroups + per_slice - 1) / per_slice;
        const double weights = (double)items * 8 * (rt * nt) * len * 2.0;
        const double staged = (double)rows * len * (norm ? 4.0 : 2.0);
        const double parts = S > 1 ? (double)items * 8 * (double)M * rt * nt * 4.0 * 2.0 : 0.0;   // written, and read again by somebody
        const double cost = weights + staged + parts;
        if (best.S == 0 || cost < best_cost) best = p, best_cost = cost;
        if (S == 1) break;      // shorter slices of a K that fits in one gain nothing
    }
    return best;
}

// ---- decode attention: contexts split over workgroups ----
// How a decode step of `rows` rows is split over the context.  A workgroup takes `unit` keys per round (32 a
// wave).  Contexts are split when the rows alone do not fill the machine: down to one round per workgroup when
// the parts are merged by the split that arrives last (`fused`), and only for long contexts when merging costs
// a second kernel.
inline void decode_split_plan(int rows, int kv_heads, int qtiles, int max_context, int unit, bool fused, int *splits,
                              int *keys_per_split) {
    const long base = (long)rows * kv_heads * qtiles;
    const long span = (long)max_context + 31;   // the first split starts at a multiple of 32 at or below the first key
    long want = 1;
    if (fused) {
        if (base < 512) want = (512 + base - 1) / base;
        const long most = (span + unit - 1) / unit;
        if (want > most) want = most;
    } else if (max_context > 2048 && base < 256) {
        want = (256 + base - 1) / base;
        const long most = (span + 2047) / 2048;
        if (want > most) want = most;
    }
    if (want > 64) want = 64;
    long per = (span + want - 1) / want;
    per = (per + unit - 1) / unit * unit;
    *splits = (int)((span + per - 1) / per);
    *keys_per_split = (int)per;
}
inline int decode_waves(int head_dim) { return head_dim >= 128 ? 8 : 16; }
inline size_t decode_workspace_need(int rows, int heads, int head_dim, int splits) {
    return splits > 1 ? (size_t)rows * heads * splits * (head_dim + 2) * kF32 : 0;
}
inline size_t decode_lds_bytes(int head_dim, int group) {
    const int waves = decode_waves(head_dim), gq = group < 16 ? group : 16;
    return (size_t)(2 * waves * 16 + waves * gq * (head_dim + 1)) * kF32;
}
inline bool decode_counters_fit(int rows, int kv_heads, int qtiles) { return (size_t)rows * kv_heads * qtiles * sizeof(int) <= kCounterBytes; }

// ---- prompt attention: the key tiles of a row tile shared among workgroups ----
// what a part of a row tile leaves behind, in floats: every thread of the workgroup its outputs (head_dim / 2), a maximum and a sum
constexpr size_t part_floats(int head_dim, int threads = 256) { return (size_t)threads * (head_dim / 2 + 2); }
// The most key tiles one workgroup takes (0: row tiles are not shared) and the most parts a row tile can have.  Row
// tiles are shared when, one workgroup each, they would leave workgroup slots of the device empty: a part then has
// about the key tiles that a slot sees in all when every slot is taken, and at least 8, since every part pays for
// leaving its results and the last one for adding them up.  A step whose rows are as many as its longest context (a
// prompt from its first token on) has row tiles of every length up to the longest, half of it on average: up to 2,048
// tokens the long ones are shared in halves (8 to 16 key tiles a part), or the slots of the short ones would idle
// through the second half of the launch (longer prompts have row tiles enough to keep every slot busy).  `room`: parts that the workspace holds; `by_hand`: key tiles a part when set by hand (> 1).
inline int prefill_part_plan(int tiles, int kv_heads, int rows, int max_context, int window, size_t room, int slots, int by_hand,
                             int *max_parts) {
    *max_parts = 1;
    if (window > 0) return 0;     // a window keeps every context short
    const long groups = (long)tiles * kv_heads;
    if (groups <= 0 || groups * (long)sizeof(int) > (long)kCounterBytes) return 0;
    const long most_tiles = ((long)max_context + 63) / 64;        // key tiles of the longest context
    const long per_slot = (groups * most_tiles + slots - 1) / slots;
    long per_part = per_slot > 8 ? per_slot : 8;
    if (rows + 63 >= max_context && most_tiles <= 32) {       // contexts of every length; measured a gain up to 2,048 tokens only
        long half = most_tiles / 2;
        half = half < 8 ? 8 : (half > 16 ? 16 : half);
        if (half < per_part) per_part = half;
    }
    if (by_hand > 1) per_part = by_hand;
    long cap = (long)(room / (size_t)groups);   // parts a row tile may have
    if (cap > 16) cap = 16;
    if (cap < 2) return 0;
    const long least = (most_tiles + cap - 1) / cap;
    if (per_part < least) per_part = least;
    if (per_part >= most_tiles) return 0;
    *max_parts = (int)((most_tiles + per_part - 1) / per_part);
    return (int)per_part;
}

}  // namespace fllm_plan
