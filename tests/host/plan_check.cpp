// Host-logic check, built with AddressSanitizer and UBSan by tests/test_host_logic.py: descriptor gate, layout,
// repack round trips on exactly sized buffers, and the invariants every launch plan must satisfy before a kernel
// may be launched with it.  No GPU: the kernel launchers are stubbed out (launch_stubs.h) and never called.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "ovfcc_internal.h"

#include "launch_stubs.h"

static int g_failures = 0;
#define CHECK(cond, ...)                                   \
    do {                                                   \
        if (!(cond)) {                                     \
            std::printf("FAILED %s: ", #cond);             \
            std::printf(__VA_ARGS__);                      \
            std::printf("\n");                             \
            ++g_failures;                                  \
        }                                                  \
    } while (0)

static ovfcc_fc_desc desc(int64_t N, int64_t K, int64_t G, int w_type, int zp_type, int flags) {
    ovfcc_fc_desc d{};
    d.N = N, d.K = K, d.group_size = G, d.w_type = w_type, d.scale_type = OVFCC_F16, d.zp_type = zp_type;
    d.bias_type = OVFCC_NONE, d.act_type = OVFCC_F16, d.out_type = OVFCC_F16, d.flags = flags;
    return d;
}

static void round_trip(const ovfcc_fc_desc& d, std::mt19937& rng) {
    const ovfcc::Layout L = ovfcc::make_layout(d);
    if (!L.tiled)
        return;
    const bool four = L.bits == 4;
    const size_t wb = four ? (size_t)d.N * d.K / 2 : (size_t)d.N * d.K, cnt = (size_t)d.N * L.groups;
    const size_t zb = d.zp_type == OVFCC_NONE ? 0 : (d.zp_type == OVFCC_U4 ? (cnt + 1) / 2 : cnt);
    std::vector<uint8_t> w(wb), z(zb), w2(wb), z2(zb), wt(L.w_bytes), zt(L.zp_bytes);
    std::vector<uint16_t> s(cnt), s2(cnt), st(L.scale_bytes / 2);
    for (auto& v : w) v = (uint8_t)rng();
    for (auto& v : z) v = (uint8_t)rng();
    for (auto& v : s) v = (uint16_t)rng();
    ovfcc::repack_weights(d, L, w.data(), wt.data());
    ovfcc::repack_params(d, L, s.data(), zb ? z.data() : nullptr, st.data(), zt.data());
    ovfcc::unrepack_weights(d, L, wt.data(), w2.data());
    ovfcc::unrepack_params(d, L, st.data(), zt.data(), s2.data(), zb ? z2.data() : nullptr);
    CHECK(w == w2 && s == s2 && z == z2, "round trip N=%ld K=%ld G=%ld type=%d zp=%d flags=%d", (long)d.N, (long)d.K,
          (long)d.group_size, d.w_type, d.zp_type, d.flags);
}

static void check_plan(const ovfcc_fc_desc& d, int64_t M, int force, int force_split, int n_cus) {
    ovfcc::FcDeviceArgs a{};
    a.M = M, a.N = d.N, a.K = d.K, a.group_size = d.group_size, a.w_type = d.w_type, a.zp_type = d.zp_type;
    a.layout = ovfcc::make_layout(d);
    a.N_out = a.layout.glu ? d.N / 2 : d.N;
    // what the API does when a node is created: nodes the matrix-vector kernel fits carry its parameter tables
    static const int placeholder = 0;
    if (a.layout.tiled && a.layout.bits == 4 && a.layout.groups_per_kblock == 1 && a.layout.kblocks_per_group == 1) {
        a.layout.gemv_c = ovfcc::gemv_kblocks_per_wave(a.layout, n_cus);
        if (a.layout.gemv_c)
            a.scale_cm = &placeholder, a.zp_cm = a.layout.zp_table ? &placeholder : nullptr;
    }
    const ovfcc::Layout& L = a.layout;
    ovfcc::LaunchPlan p;
    const int rc = ovfcc::plan_launch(a, force, force_split, n_cus, &p);
    if (rc != 0)
        return;  // refusals are legitimate; the API turns them into errors or falls back
    char what[160];
    std::snprintf(what, sizeof(what), "%s M=%ld N=%ld K=%ld G=%ld bits=%d glu=%d force=%d/%d", p.name, (long)M, (long)d.N,
                  (long)d.K, (long)d.group_size, L.bits, L.glu, force, force_split);
    CHECK(p.grid[0] >= 1 && p.grid[1] >= 1 && p.grid[2] >= 1, "%s", what);
    CHECK((uint64_t)p.grid[0] * p.grid[1] * p.grid[2] < (1ull << 31) && p.grid[1] < 65536 && p.grid[2] < 65536, "%s", what);
    CHECK(p.block >= 64 && p.block <= 1024 && p.block % 64 == 0, "%s block=%u", what, p.block);
    CHECK(p.dynamic_lds <= 160 * 1024, "%s lds=%u", what, p.dynamic_lds);
    CHECK(p.split_k >= 1, "%s", what);
    // (the 16-row kernel's parts meet in a second launch: a workspace, no counters)
    CHECK((p.split_k > 1) == (p.workspace_bytes > 0) && (p.gemv16 ? p.counter_count == 0 : (p.split_k > 1) == (p.counter_count > 0)),
          "%s ws=%zu counters=%zu split=%d", what, p.workspace_bytes, p.counter_count, p.split_k);
    if (p.kernel == OVFCC_KERNEL_PLAIN) {
        CHECK(!L.tiled && p.grid[0] == (unsigned)a.N_out && p.grid[1] == (unsigned)M, "%s", what);
        return;
    }
    CHECK(L.tiled, "%s", what);
    const int kb = (int)L.k_blocks;
    if (p.kernel == OVFCC_KERNEL_DECODE || p.direct) {
        CHECK((int64_t)p.split_k * p.kblocks_per_split >= kb, "%s split=%d per=%d kb=%d", what, p.split_k, p.kblocks_per_split, kb);
        CHECK((int64_t)(p.split_k - 1) * p.kblocks_per_split < kb, "%s empty split: split=%d per=%d kb=%d", what, p.split_k,
              p.kblocks_per_split, kb);
    }
    if (p.kernel == OVFCC_KERNEL_DECODE) {
        CHECK(M <= ovfcc::kDecodeMaxRows, "%s", what);
        const int nw = (int)p.block / 64, rt = p.tiles_per_group;
        if (p.gemv) {
            const int c = p.gemv_c, per_wg = L.glu ? 2 : 1;
            CHECK(M <= 4 && L.bits == 4 && L.groups_per_kblock == 1 && L.kblocks_per_group == 1 && c == L.gemv_c, "%s", what);
            CHECK((c == 2 || c == 4 || c == 8) && kb % c == 0 && nw == (kb / c) * per_wg && nw <= 16, "%s c=%d nw=%d", what, c, nw);
            CHECK((int64_t)p.grid[0] * per_wg == L.n_tiles && p.grid[1] == 1 && p.split_k == 1, "%s", what);
            CHECK(p.dynamic_lds == ovfcc::gemv_lds_bytes(c, (int)M, nw) && p.dynamic_lds <= 150 * 1024, "%s lds=%u", what, p.dynamic_lds);
        } else if (p.gemv16) {
            const int c = ovfcc::gemv16_kblocks_per_wave(p.gemv_c, p.split_k);
            const int64_t units = L.glu ? L.n_tiles / 2 : L.n_tiles;
            const int per_unit = L.glu ? 2 : 1;
            CHECK(M > 4 && M <= 48 && L.bits == 4 && L.groups_per_kblock == 1 && L.kblocks_per_group == 1 && p.gemv_c == L.gemv_c &&
                      (!L.glu || (L.n_tiles % 2 == 0 && p.split_k == 1)),
                  "%s", what);
            CHECK((c == 2 || c == 4) && kb % (c * p.split_k) == 0 && nw == kb / c / p.split_k && nw <= (c == 4 ? 8 : 16) &&
                      p.gemv_c % p.split_k == 0,
                  "%s c=%d nw=%d", what, c, nw);
            CHECK(rt % per_unit == 0 && (int64_t)p.grid[0] <= units && (int64_t)p.grid[0] * (rt / per_unit) >= units &&
                      (int64_t)p.grid[0] * (rt / per_unit - 1) < units && p.grid[1] == (unsigned)((M + 15) / 16) &&
                      p.grid[2] == (unsigned)p.split_k,
                  "%s grid=%u visits=%d", what, p.grid[0], rt);
            CHECK(p.dynamic_lds == ovfcc::gemv16_lds_bytes(c, nw, (L.glu || (int64_t)p.grid[0] < units) ? 2 : 1) &&
                      p.dynamic_lds <= 160 * 1024 - 64,
                  "%s lds=%u", what, p.dynamic_lds);
            CHECK(p.workspace_bytes == (p.split_k > 1 ? (size_t)p.split_k * 16 * p.grid[1] * d.N * sizeof(float) : 0), "%s", what);
        } else if (p.gemv16_stream) {
            const int c = p.gemv_c;
            CHECK(M > 4 && M <= 16 && L.bits == 4 && L.groups_per_kblock == 1 && L.kblocks_per_group == 1 && c == L.gemv_c && !L.glu,
                  "%s", what);
            CHECK((c == 2 || c == 4 || c == 8) && kb % c == 0 && nw == kb / c && nw <= 16, "%s c=%d nw=%d", what, c, nw);
            CHECK((rt == 1 || rt == 2 || rt == 4) && (int64_t)p.grid[0] * rt == L.n_tiles && p.grid[1] == 1 && p.grid[2] == 1 &&
                      p.split_k == 1 && p.workspace_bytes == 0,
                  "%s grid=%u tiles=%d", what, p.grid[0], rt);
            CHECK(p.dynamic_lds == ovfcc::gemv16s_lds_bytes(nw, rt) && p.dynamic_lds <= 160 * 1024 - 64, "%s lds=%u", what, p.dynamic_lds);
        } else if (p.batch) {
            const int mt = (int)(M + 15) / 16;
            CHECK(p.tile_m == 16 * mt && (rt == 1 || rt == 2), "%s", what);
            CHECK((int64_t)p.grid[0] * nw * rt >= L.n_tiles && p.grid[1] == (unsigned)p.split_k, "%s", what);
            CHECK(p.dynamic_lds <= 96 * 1024 && p.dynamic_lds == (unsigned)(16 * mt * ((size_t)p.kblocks_per_split * 128 + 8) * 2),
                  "%s lds=%u", what, p.dynamic_lds);
            CHECK(p.workspace_bytes == (p.split_k > 1 ? (size_t)p.grid[0] * p.split_k * nw * rt * mt * 1024 : 0), "%s", what);
            if (L.glu)  // gate and up tile in one wave, or in neighbouring waves with room for the hand-over
                CHECK((rt == 2 || nw % 2 == 0) && p.dynamic_lds >= (unsigned)(nw / 2) * p.tile_m * 64u, "%s", what);
        } else {
            CHECK(M <= 32 && (int64_t)p.grid[0] * rt == L.n_tiles && p.grid[1] == (unsigned)p.split_k, "%s rt=%d", what, rt);
            CHECK(!L.glu || (p.x_in_lds && rt % 2 == 0 && M <= 16), "%s rt=%d xlds=%d", what, rt, (int)p.x_in_lds);
            CHECK(p.dynamic_lds <= 64 * 1024, "%s lds=%u", what, p.dynamic_lds);
        }
        return;
    }
    CHECK(d.N % 128 == 0, "%s", what);
    CHECK(!p.async_dma || (p.direct && L.bits == 4), "%s", what);
    // several groups per k-block: only the all-asynchronous and the square kernel carry them
    CHECK(L.groups_per_kblock == 1 || (L.bits == 4 && (p.async_dma || p.tile_n == 128)), "%s gpb=%d", what, L.groups_per_kblock);
    if (p.direct) {
        const int64_t tiles = (int64_t)p.tiles_x * p.tiles_y;
        CHECK(p.tile_m == 128 || (p.async_dma && p.tile_m == 64) || (p.big && p.tile_m == 256), "%s tile_m=%d", what, p.tile_m);
        // 256 x 256 tiles: 4-bit nodes with one group per k-block at most, whole tiles, a tile for every compute unit
        if (p.big)
            CHECK(p.async_dma && L.bits == 4 && L.groups_per_kblock == 1 && p.split_k == 1 && p.block == 256 &&
                      p.tiles_x == (int)(d.N / 256) && p.tiles_y == (int)((M + 255) / 256) &&
                      p.full_tiles == p.tiles_x * p.tiles_y && p.full_tiles >= n_cus, "%s big", what);
        CHECK(d.N % 256 == 0 && p.tiles_x == d.N / 256 && p.tiles_y == (M + p.tile_m - 1) / p.tile_m, "%s", what);
        CHECK(p.full_tiles >= 0 && p.full_tiles <= tiles && (p.split_k > 1 || p.full_tiles == tiles), "%s full=%d", what, p.full_tiles);
        CHECK(p.grid[0] == (unsigned)(p.full_tiles + (tiles - p.full_tiles) * p.split_k) && p.grid[1] == 1 && p.grid[2] == 1, "%s", what);
        CHECK(p.workspace_bytes == (p.split_k > 1 ? (size_t)(tiles - p.full_tiles) * p.split_k * p.tile_m * 256 * 4 : 0), "%s", what);
        CHECK(M * d.K * 2 < (1ll << 31), "%s", what);
    } else {
        CHECK(p.split_k == 1, "%s", what);
        CHECK(p.grid[0] == (unsigned)(d.N / p.tile_n) && p.grid[1] == (unsigned)((M + 127) / 128), "%s", what);
        CHECK(p.tile_n == 128 || (d.N % 256 == 0 && d.K % 256 == 0), "%s", what);
    }
}

// The environment overrides are read once and again only on request.
static void check_env_cache() {
    unsetenv("OVFCC_PREFILL_ROWS");
    ovfcc::env_reload();
    const unsigned g0 = ovfcc::env_generation();
    CHECK(ovfcc::env_int("OVFCC_PREFILL_ROWS", 7) == 7, "unset variable gives the fallback");
    setenv("OVFCC_PREFILL_ROWS", "64", 1);
    CHECK(ovfcc::env_int("OVFCC_PREFILL_ROWS", 7) == 7, "a change of the environment is not seen before a reload");
    CHECK(ovfcc::env_generation() == g0, "generation unchanged without a reload");
    ovfcc::env_reload();
    CHECK(ovfcc::env_int("OVFCC_PREFILL_ROWS", 7) == 64 && ovfcc::env_generation() != g0, "reload takes the change over");
    unsetenv("OVFCC_PREFILL_ROWS");
    ovfcc::env_reload();
    CHECK(ovfcc::env_int("OVFCC_PREFILL_ROWS", 7) == 7, "and its removal");
}

int main() {
    check_env_cache();
    std::mt19937 rng(12345);
    const int64_t Ns[] = {16, 32, 48, 96, 128, 256, 272, 1024, 4096, 14336};
    const int64_t Ks[] = {128, 256, 384, 1024, 4096, 14336};
    const int64_t Ms[] = {1, 2, 4, 5, 15, 16, 17, 31, 32, 33, 47, 48, 49, 127, 128, 129, 300, 2048, 8192};
    const int types[] = {OVFCC_U4, OVFCC_I4, OVFCC_U8, OVFCC_I8};
    const int flags[] = {0, OVFCC_GLU_SWISH, OVFCC_GLU_GELU | OVFCC_GLU_GATE_SECOND};
    int plans = 0;
    for (int64_t N : Ns)
        for (int64_t K : Ks)
            for (int64_t G : {(int64_t)32, (int64_t)64, (int64_t)128, K})
                for (int t : types)
                    for (int fl : flags) {
                        const int zp = (t == OVFCC_U4) ? OVFCC_U4 : (t == OVFCC_U8 ? OVFCC_U8 : OVFCC_NONE);
                        const ovfcc_fc_desc d = desc(N, K, G, t, zp, fl);
                        if (ovfcc::validate_desc(&d) != 0)
                            continue;
                        if (N <= 1024 && K <= 1024)
                            round_trip(d, rng);
                        for (int64_t M : Ms)
                            for (int force : {OVFCC_KERNEL_AUTO, OVFCC_KERNEL_DECODE, OVFCC_KERNEL_PREFILL})
                                for (int split : {0, 1, 3, 8, 64})
                                    for (int cus : {256, 64}) {
                                        check_plan(d, M, force, split, cus);
                                        ++plans;
                                    }
                    }
    // untiled shapes: plain kernel only
    for (int fl : flags) {
        const ovfcc_fc_desc d = desc(40, 200, 50, OVFCC_U4, OVFCC_U4, fl);
        CHECK(ovfcc::validate_desc(&d) == 0 && !ovfcc::make_layout(d).tiled, "untiled");
        for (int64_t M : Ms)
            check_plan(d, M, OVFCC_KERNEL_AUTO, 0, 256);
    }
    // a grouped run fixes the tile height: its plan keeps one row tile per slice whatever the tile counts say
    {
        const ovfcc_fc_desc d = desc(14336, 4096, 128, OVFCC_U4, OVFCC_U4, 0);
        ovfcc::FcDeviceArgs a{};
        a.M = 16 * 128, a.N = d.N, a.K = d.K, a.group_size = d.group_size, a.w_type = d.w_type, a.zp_type = d.zp_type;
        a.layout = ovfcc::make_layout(d);
        a.N_out = d.N;
        ovfcc::LaunchPlan p;
        CHECK(ovfcc::plan_launch(a, OVFCC_KERNEL_PREFILL, 0, 256, &p) == 0 && p.big && p.tiles_y == 8, "one node: 256-row tiles");
        a.tile_rows = 128;
        CHECK(ovfcc::plan_launch(a, OVFCC_KERNEL_PREFILL, 0, 256, &p) == 0 && !p.big && p.async_dma && p.tiles_y == 16,
              "grouped: 128-row tiles");
        // the slice heights of a grouped run: one tile row per slice, whatever the height
        for (int rows : {64, 80, 96}) {
            a.tile_rows = rows;
            a.M = 15 * rows;
            CHECK(ovfcc::plan_launch(a, OVFCC_KERNEL_PREFILL, 0, 256, &p) == 0 && !p.big && p.async_dma && p.tile_m == rows &&
                      p.tiles_y == 15 && (int64_t)p.tiles_x * p.tiles_y * p.split_k >= (int64_t)p.grid[0] - p.full_tiles,
                  "grouped: 64-, 80- and 96-row tiles");
        }
    }
    // slice heights of grouped runs by cost
    {
        const int64_t mixtral[8] = {65, 64, 54, 71, 70, 70, 56, 62}, two[2] = {90, 66}, full[4] = {128, 128, 128, 128},
                      small[2] = {50, 60}, tall[3] = {200, 130, 129}, one[1] = {81};
        CHECK(ovfcc::rows_cap_for(mixtral, 8, true) == 80, "54-71 rows: 80-row slices");
        CHECK(ovfcc::rows_cap_for(mixtral, 8, false) == 128, "54-71 rows without the middle heights: 128");
        CHECK(ovfcc::rows_cap_for(two, 2, true) == 96, "66 and 90 rows: 96");
        CHECK(ovfcc::rows_cap_for(full, 4, true) == 128, "full tiles: 128");
        CHECK(ovfcc::rows_cap_for(small, 2, true) == 64, "up to 64 rows: 64");
        CHECK(ovfcc::rows_cap_for(tall, 3, true) == 80 || ovfcc::rows_cap_for(tall, 3, true) == 128, "tall items: fewest tiles");
        CHECK(ovfcc::rows_cap_for(one, 1, true) == 96, "81 rows: 96");
        ++plans;
    }
    // the gate refuses what the kernels cannot index
    ovfcc_fc_desc bad = desc(64, 256, 96, OVFCC_U4, OVFCC_NONE, 0);
    CHECK(ovfcc::validate_desc(&bad) != 0, "group size must divide K");
    bad = desc(63, 256, 128, OVFCC_U4, OVFCC_NONE, OVFCC_GLU_SWISH);
    CHECK(ovfcc::validate_desc(&bad) != 0, "odd N with a gated linear unit");
    std::printf("%d plans checked, %d failures\n", plans, g_failures);
    return g_failures ? 1 : 0;
}
