// Sweeps the launch plans of csrc/plans.h over shapes, on the host: every plan keeps LDS within a compute unit's, its
// counters within the counters' part of the workspace, cuts K into slices none of which is empty, and addresses
// partial results inside the bytes it said it needs (the buffers here have exactly that size, so that the address
// sanitizer sees a step outside them).  Built and run by tests/test_plans.py.
#include "plans.h"

#include <stdio.h>
#include <stdlib.h>
#include <vector>

using namespace fllm_plan;

static long checks = 0;
#define REQUIRE(cond, ...)                                   \
    do {                                                     \
        checks++;                                            \
        if (!(cond)) {                                       \
            fprintf(stderr, "FAILED %s: ", #cond);           \
            fprintf(stderr, __VA_ARGS__);                    \
            fprintf(stderr, "\n");                           \
            exit(1);                                         \
        }                                                    \
    } while (0)

static void slices_cover(int K, int S, int slice, const char *what) {
    REQUIRE(S >= 1 && slice > 0, "%s K=%d S=%d slice=%d", what, K, S, slice);
    REQUIRE((long)S * slice >= K, "%s: slices do not cover K=%d (S=%d slice=%d)", what, K, S, slice);
    REQUIRE((long)(S - 1) * slice < K, "%s: an empty slice at K=%d (S=%d slice=%d)", what, K, S, slice);
}

// A stretch of the workspace of exactly the floats a plan said it needs.  Small ones are real memory, so that the
// address sanitizer sees a step outside them; large ones (up to the 192 MiB of a workspace) are checked by arithmetic.
struct Stretch {
    size_t floats;
    std::vector<float> real;
    explicit Stretch(size_t n) : floats(n), real(n <= (1u << 18) ? n : 0) {}
};
// touches the first and last float that a (tile, slice) part of `floats` floats would use
static void touch(Stretch &buf, size_t offset, size_t floats) {
    REQUIRE(floats > 0 && offset + floats <= buf.floats, "a part at %zu + %zu lies outside the %zu floats planned", offset, floats, buf.floats);
    if (!buf.real.empty()) {
        buf.real[offset] = 1.f;
        buf.real[offset + floats - 1] = 1.f;
    }
}

int main() {
    const int Ks[] = {8, 72, 264, 1000, 1024, 2072, 4096, 8192, 14336, 30008, 65536};
    const int Ns[] = {16, 30, 1000, 4096, 5001, 28672, 128256, 262144};
    const size_t workspaces[] = {0, (size_t)1 << 20, (size_t)192 << 20};
    const int cus_list[] = {1, 256, 304};
    for (size_t ws_bytes : workspaces)
        for (int cus : cus_list)
            for (int K : Ks)
                for (int N : Ns) {
                    const bool have_ws = ws_bytes > 0;
                    // ---- up to 16 rows ----
                    for (int M : {1, 3, 8, 9, 16})
                        for (int rt = 1; rt <= 2; rt++)
                            for (int forced : {0, 2, 4, 8})
                                for (int xd = 0; xd < 2; xd++) {
                                    const int nt = rt == 2 ? 8 : 16;
                                    const int ntiles = (int)ceil_div(rt == 2 ? N / 2 : N, nt);
                                    if (ntiles == 0) continue;
                                    const ResidentPlan p = plan_resident(M, K, ntiles, rt, ws_bytes, have_ws, xd != 0, forced);
                                    if (p.S == 0) continue;      // declined: the caller says so
                                    slices_cover(K, p.S, p.slice, "resident");
                                    REQUIRE(p.slice % 128 == 0, "resident slice %d", p.slice);
                                    REQUIRE(p.smem * p.per_cu <= kLdsBytes, "resident LDS %zu x %d", p.smem, p.per_cu);
                                    REQUIRE(p.stage + p.red + (size_t)p.waves * 16 * 4 <= p.smem, "resident LDS layout");
                                    REQUIRE(xd || p.stage >= (size_t)M * (p.slice + 8) * 2, "resident staging");
                                    const int groups = resident_groups(p, ntiles, cus);
                                    REQUIRE(groups >= 1 && groups <= ntiles, "resident groups %d of %d tiles", groups, ntiles);
                                    if (p.S > 1) {
                                        REQUIRE(have_ws && (size_t)ntiles * 4 <= kCounterBytes, "resident counters");
                                        const size_t need = resident_workspace_need(ntiles, p.S, rt);
                                        REQUIRE(need <= ws_bytes, "resident workspace %zu of %zu", need, ws_bytes);
                                        Stretch buf((need - kCounterBytes) / 4);
                                        const size_t ssq = resident_ssq_offset_floats(ntiles, p.S, rt);
                                        for (int tile : {0, ntiles - 1})
                                            for (int sl : {0, p.S - 1}) {
                                                touch(buf, ((size_t)(tile * p.S + sl) * rt * kWaveLanes) * 4, (size_t)rt * kWaveLanes * 4);
                                                touch(buf, ssq + (size_t)(tile * p.S + sl) * 16, 16);
                                            }
                                    }
                                }
                    // ---- 17 to 64 rows ----
                    for (int mt = 2; mt <= 4; mt++)
                        for (int rt = 1; rt <= 2; rt++)
                            for (int forced : {0, 1, 2, 4, 8, 14}) {
                                const int nt = rt == 2 ? 8 : 16;
                                const int ntiles = (int)ceil_div(rt == 2 ? N / 2 : N, nt);
                                if (ntiles == 0) continue;
                              for (int waves : {0, 4, 7, 8}) {
                                const ChunkPlan c = plan_chunks_balanced(K, ntiles, mt, rt, ws_bytes, have_ws, cus, forced, waves);
                                REQUIRE(c.waves == 4 || c.waves == 7 || c.waves == 8, "chunks waves %d", c.waves);
                                REQUIRE(waves == 0 || c.waves == waves, "chunks waves %d forced %d", c.waves, waves);
                                REQUIRE(c.grid / c.S <= (int)ceil_div(ntiles, c.waves), "chunks grid %d beyond the row groups", c.grid);
                                slices_cover(K, c.S, c.slice, "chunks");
                                REQUIRE(c.grid >= 1 && c.grid % c.S == 0, "chunks grid %d S %d", c.grid, c.S);
                                if (c.S > 1) {
                                    REQUIRE(have_ws && (size_t)ntiles * 4 <= kCounterBytes, "chunks counters");
                                    const size_t need = chunk_workspace_need(ntiles, c.S, mt, rt);
                                    REQUIRE(need <= ws_bytes, "chunks workspace");
                                    Stretch buf((need - kCounterBytes) / 4);
                                    for (int tile : {0, ntiles - 1})
                                        for (int sl : {0, c.S - 1})
                                            touch(buf, (((size_t)tile * c.S + sl) * mt) * rt * kWaveLanes * 4, (size_t)mt * rt * kWaveLanes * 4);
                                    REQUIRE(need - kCounterBytes <= 0x7fffffffu, "chunks workspace offsets");
                                }
                              }
                                for (int norm = 0; norm < 2; norm++) {
                                    const int M = mt * 16 - 3;
                                    const SlabPlan s = plan_slab(M, ntiles, K, mt, rt, norm != 0, nt, ws_bytes, have_ws, cus, forced);
                                    if (s.S == 0) continue;
                                    slices_cover(K, s.S, s.slice, "slab");
                                    REQUIRE(s.slice % 256 == 0 && (!norm || s.slice % 512 == 0) && s.slice <= 1024 + 0 * K, "slab slice %d", s.slice);
                                    REQUIRE(s.smem <= kLdsBytes, "slab LDS %zu", s.smem);
                                    REQUIRE(s.cells_off >= (size_t)mt * 16 * (s.slice + 8) * 2 && s.cells_off % 16 == 0, "slab staging");
                                    REQUIRE(!norm || s.smem >= s.cells_off + (size_t)mt * 16 * ((s.slice + 511) / 512) * 4, "slab cells");
                                    REQUIRE(s.grid >= 1 && s.grid % s.S == 0 && s.grid <= (cus > s.S ? cus : s.S), "slab grid %d S %d", s.grid, s.S);
                                    if (s.S > 1) {
                                        REQUIRE(have_ws && (size_t)ntiles * 4 <= kCounterBytes, "slab counters");
                                        const size_t need = slab_workspace_need(ntiles, s.S, mt, rt);
                                        REQUIRE(need <= ws_bytes && need - kCounterBytes <= 0x7fffffffu, "slab workspace");
                                        Stretch buf((need - kCounterBytes) / 4);
                                        const size_t ssq = slab_ssq_offset_floats(ntiles, s.S, mt, rt);
                                        for (int tile : {0, ntiles - 1})
                                            for (int sl : {0, s.S - 1}) {
                                                touch(buf, ((size_t)tile * s.S + sl) * mt * rt * kWaveLanes * 4, (size_t)mt * rt * kWaveLanes * 4);
                                                touch(buf, ssq + ((size_t)tile * s.S + sl) * mt * 16, (size_t)mt * 16);
                                            }
                                    }
                                }
                            }
                }
    // ---- decode attention ----
    for (int rows : {1, 2, 8, 24, 64, 256})
        for (int kv_heads : {1, 2, 8, 64})
            for (int group : {1, 4, 7, 16, 40})
                for (int head_dim : {32, 64, 128})
                    for (int context : {1, 31, 256, 1000, 4096, 40000, 131072})
                        for (int fused = 0; fused < 2; fused++) {
                            const int qtiles = (group + 15) / 16, unit = decode_waves(head_dim) * 32;
                            int splits = 0, per = 0;
                            decode_split_plan(rows, kv_heads, qtiles, context, unit, fused != 0, &splits, &per);
                            const long span = (long)context + 31;
                            REQUIRE(splits >= 1 && splits <= 64 && per % unit == 0, "decode splits %d per %d", splits, per);
                            REQUIRE((long)splits * per >= span && (long)(splits - 1) * per < span, "decode: %d splits of %d keys for %d", splits, per, context);
                            REQUIRE(decode_lds_bytes(head_dim, group) + 1024 <= kLdsBytes, "decode LDS");
                            const size_t need = decode_workspace_need(rows, kv_heads * group, head_dim, splits);
                            if (splits > 1) {
                                Stretch buf(need / 4);
                                const size_t heads = (size_t)kv_heads * group, ml = (size_t)rows * heads * splits * 2;
                                touch(buf, 0, 2);
                                touch(buf, (((size_t)rows - 1) * heads + heads - 1) * splits * 2 + (splits - 1) * 2, 2);
                                touch(buf, ml + ((((size_t)rows - 1) * heads + heads - 1) * splits + splits - 1) * head_dim, head_dim);
                            } else {
                                REQUIRE(need == 0, "decode workspace of an unsplit step");
                            }
                        }
    // ---- prompt attention ----
    for (int tiles : {1, 3, 17, 64, 513, 20000})
        for (int kv_heads : {1, 8})
            for (int context : {64, 1000, 2048, 30000, 131072})
                for (int window : {0, 512})
                    for (size_t room : {(size_t)0, (size_t)40, (size_t)4096, (size_t)1 << 20})
                        for (int slots : {2, 512})
                            for (int by_hand : {0, 1, 3, 40})
                            for (int rows : {1, context / 2, context, 4 * context}) {
                                int max_parts = -1;
                                const int per_part = prefill_part_plan(tiles, kv_heads, rows, context, window, room, slots, by_hand, &max_parts);
                                REQUIRE(max_parts >= 1 && max_parts <= 16, "parts %d", max_parts);
                                if (per_part == 0) {
                                    REQUIRE(max_parts == 1, "an unshared row tile has one part");
                                    continue;
                                }
                                const long most_tiles = ((long)context + 63) / 64, groups = (long)tiles * kv_heads;
                                REQUIRE(window == 0 && groups * 4 <= (long)kCounterBytes, "shared row tiles need counters");
                                REQUIRE((long)max_parts * per_part >= most_tiles && (long)(max_parts - 1) * per_part < most_tiles,
                                        "parts %d of %d key tiles for %ld", max_parts, per_part, most_tiles);
                                REQUIRE((size_t)groups * max_parts <= room, "parts %ld x %d in room %zu", groups, max_parts, room);
                            }
    printf("plans ok: %ld checks\n", checks);
    return 0;
}
