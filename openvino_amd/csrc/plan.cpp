// Kernel choice and launch decomposition (host only).
//
// Policy: shapes that keep OpenVINO's layout run the plain kernel; tiled nodes run a decode kernel for
// M <= 48 (the streaming kernel for a few rows, the small-batch kernel above) and the prefill kernel for more
// (the roofline ridge of int4 g128 sits near M = 83).  The caller cuts 48 < M <= 128 into decode launches:
// a single 128-row prefill tile per column block leaves most of the chip idle.
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "ovfcc_internal.h"

namespace ovfcc {

// Overrides from the process environment, read once -- at the first use, which ovfcc_init forces -- and again only
// by env_reload (tests and experiments that change the environment of a running process).
//   tuning:  OVFCC_DECODE_WAVES = 4 | 8 | 16 (workgroup size), OVFCC_DECODE_RT = 1 | 2 | 4 (channel tiles per
//            workgroup or wave), OVFCC_DECODE_XLDS = 0 | 1 (activations via LDS), OVFCC_DECODE_BATCH = 0 | 1
//            (small-batch kernel instead of the streaming kernel), OVFCC_GEMV = 0 | 1, OVFCC_GEMV_C = 2 | 4 | 8,
//            OVFCC_GEMV16 = 0 | 1 (the 16-row kernel with stationary activations for 5-48 rows),
//            OVFCC_GEMV16_GRID = n (its workgroups per row tile), OVFCC_GEMV16_SPLIT = 1 | 2 | 4 | 8 (parts it cuts K in),
//            OVFCC_GEMV16_STREAM = 0 | 1 (the 16-row kernel that streams its activations, 5-16 rows),
//            OVFCC_GEMV16_STREAM_TILES = 1 | 2 | 4 (its channel tiles per workgroup),
//            OVFCC_PREFILL_{DIRECT, ASYNC, WIDE, BIG, TAIL} = 0 | 1, OVFCC_PREFILL_ROWS = 64 | 128,
//            OVFCC_MOE_HOST_ROUTING = 1, OVFCC_MLP_FUSED = 1 (an MLP node of up to four rows as one launch instead of two),
//            OVFCC_MLP_GRID = n (its workgroups), OVFCC_MLP_SPIN_LIMIT = n (polls after which that launch's wait for its workgroups gives up; tests);
//   logging: OVFCC_VERBOSE = 1 (one line per launch on stderr), 2 (also weights and requests as they come and go).
namespace {
struct EnvEntry {
    const char* name;
    std::atomic<int> set{0};
    std::atomic<int> value{0};
    explicit EnvEntry(const char* n) : name(n) {}
};
EnvEntry g_env[] = {EnvEntry("OVFCC_DECODE_WAVES"),   EnvEntry("OVFCC_DECODE_RT"),      EnvEntry("OVFCC_DECODE_XLDS"),
                    EnvEntry("OVFCC_DECODE_BATCH"),   EnvEntry("OVFCC_GEMV"),           EnvEntry("OVFCC_GEMV_C"),
                    EnvEntry("OVFCC_GEMV16"),         EnvEntry("OVFCC_GEMV16_GRID"),    EnvEntry("OVFCC_GEMV16_SPLIT"),
                    EnvEntry("OVFCC_GEMV16_STREAM"),  EnvEntry("OVFCC_GEMV16_STREAM_TILES"),
                    EnvEntry("OVFCC_PREFILL_DIRECT"), EnvEntry("OVFCC_PREFILL_ASYNC"),  EnvEntry("OVFCC_PREFILL_WIDE"),
                    EnvEntry("OVFCC_PREFILL_BIG"),    EnvEntry("OVFCC_PREFILL_TAIL"),   EnvEntry("OVFCC_PREFILL_ROWS"),
                    EnvEntry("OVFCC_MOE_HOST_ROUTING"), EnvEntry("OVFCC_MLP_FUSED"),      EnvEntry("OVFCC_MLP_SPIN_LIMIT"),
                    EnvEntry("OVFCC_MLP_GRID"),
                    EnvEntry("OVFCC_VERBOSE")};
std::atomic<unsigned> g_env_generation{0};
std::once_flag g_env_once;

void env_read_all() {
    for (EnvEntry& e : g_env) {
        const char* v = std::getenv(e.name);
        e.value.store(v ? std::atoi(v) : 0, std::memory_order_relaxed);
        e.set.store(v ? 1 : 0, std::memory_order_release);
    }
    g_env_generation.fetch_add(1, std::memory_order_acq_rel);
}
}  // namespace

void env_reload() {
    std::call_once(g_env_once, [] {});  // a later first use must not read again on top of this
    env_read_all();
}

unsigned env_generation() {
    std::call_once(g_env_once, env_read_all);
    return g_env_generation.load(std::memory_order_acquire);
}

int env_int(const char* name, int fallback) {
    std::call_once(g_env_once, env_read_all);
    for (EnvEntry& e : g_env)
        if (std::strcmp(e.name, name) == 0)
            return e.set.load(std::memory_order_acquire) ? e.value.load(std::memory_order_relaxed) : fallback;
    const char* v = std::getenv(name);  // a name the table does not know
    return v ? std::atoi(v) : fallback;
}

// k-blocks per wave of the matrix-vector kernel for this node (0: the kernel does not fit it).  The waves of one
// channel tile (of a gate / up tile pair) share a workgroup of at most 16 waves and each takes 2, 4 or 8 whole
// k-blocks; of the divisions that fit, the coarsest one that still gives every SIMD of the chip about two waves,
// but no coarser than a workgroup of eight waves needs.
// OVFCC_GEMV_C overrides for experiments.
int gemv_kblocks_per_wave(const Layout& L, int n_cus) {
    const int tiles_per_wg = L.glu ? 2 : 1;
    if (L.glu && (L.n_tiles & 1))
        return 0;
    auto fits = [&](int c) { return L.k_blocks % c == 0 && (L.k_blocks / c) * tiles_per_wg <= 16; };
    const int forced = env_int("OVFCC_GEMV_C", 0);
    if ((forced == 2 || forced == 4 || forced == 8) && fits(forced))
        return forced;
    int best = 0;
    for (int c : {2, 4, 8})
        if (fits(c) && (best == 0 || L.n_tiles * (L.k_blocks / c) >= (int64_t)8 * n_cus))
            best = c;
    // Eight k-blocks per wave leave a plain node of K = 4096 with four waves per workgroup; eight waves of four
    // k-blocks stream the same bytes faster (gate / up at one row: 7.0 against 7.3 us) and give the 16-row kernel
    // two waves per SIMD (16 rows: 10.7 against 12.8 us).
    if (best == 8 && !L.glu && fits(4) && L.k_blocks / 4 <= 8)
        best = 4;
    return best;
}

// Dynamic LDS of the matrix-vector kernel: every wave stages its rows (1, 2 or 4 carried; c k-blocks of 256 bytes
// each plus a 64-byte pad per row) and leaves 16 partial sums per row.
size_t gemv_lds_bytes(int c, int m, int waves) {
    const int mr = m == 1 ? 1 : m == 2 ? 2 : 4;
    return (size_t)waves * mr * (c * 256 + 64) + (size_t)waves * mr * 16 * sizeof(float);
}

int plan_launch(const FcDeviceArgs& a, int force_kernel, int force_split, int n_cus, LaunchPlan* plan) {
    LaunchPlan p;
    const Layout& L = a.layout;
    int kernel = force_kernel;
    if (kernel == OVFCC_KERNEL_AUTO)
        kernel = !L.tiled ? OVFCC_KERNEL_PLAIN : (a.M <= kDecodeMaxRows ? OVFCC_KERNEL_DECODE : OVFCC_KERNEL_PREFILL);
    if (kernel != OVFCC_KERNEL_PLAIN && !L.tiled)
        return fail(OVFCC_EUNSUPPORTED, "this node keeps the OpenVINO layout; only the plain kernel can run it");
    if (kernel == OVFCC_KERNEL_PLAIN && L.tiled)
        return fail(OVFCC_EUNSUPPORTED, "this node was repacked into tiles; the plain kernel needs the OpenVINO layout");
    if (kernel == OVFCC_KERNEL_DECODE && a.M > kDecodeMaxRows)
        return fail(OVFCC_EUNSUPPORTED, "the decode kernels handle at most 48 rows per launch");
    if (kernel == OVFCC_KERNEL_PREFILL && (a.N % kPrefillTileN) != 0)
        return fail(OVFCC_EUNSUPPORTED, "the prefill kernel needs N % 128 == 0");
    p.kernel = kernel;
    // Small-batch kernel: waves own channel tiles, the workgroup shares one staged slice of X.  It pays
    // for its split-K epilogue, so the streaming kernel keeps M <= 4 and, for small nodes, M <= 16.
    const bool want_batch =
        env_int("OVFCC_DECODE_BATCH", (a.M > 16 || (a.M > 4 && L.w_bytes >= ((size_t)16 << 20))) ? 1 : 0) != 0;
    auto plan_batch = [&]() -> int {
        const int kb = (int)L.k_blocks;
        const int mt = (int)((a.M + 15) / 16);
        int rt = 1;
        const int rt_env = env_int("OVFCC_DECODE_RT", 0);
        if (rt_env == 1 || rt_env == 2)
            rt = rt_env;
        int nw = 8;
        const int nw_env = env_int("OVFCC_DECODE_WAVES", 0);
        if (nw_env == 4 || nw_env == 8)
            nw = nw_env;
        const int64_t groups = (L.n_tiles + nw * rt - 1) / (nw * rt);
        auto x_bytes = [&](int per) { return (size_t)16 * mt * ((size_t)per * kBlockK + 8) * 2; };
        const size_t lds_budget = 96 * 1024;
        int split = force_split;
        if (split <= 0) {
            // split K until the grid covers the compute units (keeping at least two k-blocks per workgroup)
            split = 1;
            while (groups * split < n_cus && split < 8 && kb / (split * 2) >= 2)
                split *= 2;
        }
        if (split > kb)
            split = kb;
        while (split < kb && x_bytes((kb + split - 1) / split) > lds_budget)
            split = split * 2 < kb ? split * 2 : kb;  // the staged slice of X has to fit in LDS
        const int per = (kb + split - 1) / split;
        split = (kb + per - 1) / per;  // no empty splits
        if (x_bytes(per) > lds_budget)
            return fail(OVFCC_EUNSUPPORTED, "one k-block of the activations does not fit in LDS");
        p.batch = true;
        p.split_k = split;
        p.kblocks_per_split = per;
        p.tiles_per_group = rt;
        p.grid[0] = (unsigned)groups;
        p.grid[1] = (unsigned)split;
        p.block = 64u * nw;
        p.tile_m = 16 * mt;
        p.tile_n = 16 * rt * nw;
        p.workspace_bytes = split > 1 ? (size_t)groups * split * nw * rt * mt * 256 * sizeof(float) : 0;
        p.counter_count = split > 1 ? (size_t)groups : 0;
        p.dynamic_lds = (unsigned)x_bytes(per);
        p.name = L.bits == 4 ? "fcc_batch_w4" : "fcc_batch_w8";
        return OVFCC_OK;
    };
    // Five to 48 rows of a 4-bit node with groups of 128 inputs whose 16 rows x K of activations fit in LDS (and,
    // divided among the waves, in registers): the 16-row sibling of the matrix-vector kernel.  Every workgroup
    // keeps its row tile of the activations and walks channel tiles; the grid is as many workgroups as the chip
    // holds at once, rounded so that all of them visit the same number of tiles.
    auto plan_gemv16 = [&]() -> bool {
        if (a.M <= 4 || a.M > kDecodeMaxRows || !a.scale_cm || L.bits != 4 || L.groups_per_kblock != 1 ||
            L.kblocks_per_group != 1 || force_split > 0 || L.gemv_c == 0 || (L.glu && (L.n_tiles & 1)) ||
            env_int("OVFCC_GEMV16", 1) == 0 ||
            env_int("OVFCC_DECODE_BATCH", -1) >= 0 || L.n_tiles * L.k_blocks * kTileBytes >= ((int64_t)1 << 30))
            return false;
        const size_t lds_limit = 160 * 1024 - 64;
        const int64_t rows = (a.M + 15) / 16;
        const int64_t units = L.glu ? L.n_tiles / 2 : L.n_tiles;  // visited in one go: tiles, or pairs of gate and up tile
        // K whole where 16 rows x K fit in LDS and the waves in the register file; else cut in 2, 4 or 8 parts whose
        // partial sums a second launch adds (OVFCC_GEMV16_SPLIT picks the number of parts)
        const int split_env = env_int("OVFCC_GEMV16_SPLIT", 0);
        for (int split : {1, 2, 4, 8}) {
            if (split_env > 0 && split != split_env)
                continue;
            // (up to 16 rows, four parts and their second launch only tie with the small-batch kernel -- 14336 -> 4096:
            // 12.8 against 12.7 us; from 17 rows on they are ahead, 16.2 against 21.5 us at 32 rows -- while two
            // parts are ahead from the start: 8192 -> 8192 at 16 rows 12.5 against 14.7 us)
            if (split > 1 && (L.glu || L.gemv_c % split != 0 || (a.N & 3) || (a.M <= 16 && split > 2 && split_env <= 0)))
                continue;
            // the kernel's registers allow 8 and 16 waves per compute unit with 4 and 2 k-blocks per wave
            const int c = gemv16_kblocks_per_wave(L.gemv_c, split);
            if (c != 2 && c != 4)
                continue;
            const int waves = (int)(L.k_blocks / c / split);
            const int cu_waves = c == 4 ? 8 : 16;
            if (waves < 1 || waves > cu_waves)
                continue;
            const size_t lds2 = gemv16_lds_bytes(c, waves, 2);
            const int64_t per_cu = std::max<int64_t>(1, std::min<int64_t>((int64_t)(160 * 1024 / lds2), cu_waves / waves));
            const int64_t at_once = std::max<int64_t>(1, (int64_t)n_cus * per_cu / (rows * split));
            int64_t visits = (units + at_once - 1) / at_once;
            int64_t grid = (units + visits - 1) / visits;
            const int grid_env = env_int("OVFCC_GEMV16_GRID", 0);
            if (grid_env > 0) {
                grid = std::min<int64_t>(grid_env, units);
                visits = (units + grid - 1) / grid;
            }
            const size_t lds = gemv16_lds_bytes(c, waves, (L.glu || grid < units) ? 2 : 1);
            if (lds > lds_limit)
                continue;
            p.gemv16 = true;
            p.gemv_c = L.gemv_c;
            p.split_k = split;
            p.kblocks_per_split = (int)(L.k_blocks / split);
            p.tiles_per_group = (int)(visits * (L.glu ? 2 : 1));
            p.grid[0] = (unsigned)grid;
            p.grid[1] = (unsigned)rows;
            p.grid[2] = (unsigned)split;
            p.block = 64u * waves;
            p.tile_m = 16;
            p.tile_n = 16;
            p.dynamic_lds = (unsigned)lds;
            p.workspace_bytes = split > 1 ? (size_t)split * 16 * rows * a.N * sizeof(float) : 0;
            p.name = "fcc_gemv16_w4";
            return true;
        }
        return false;
    };
    // Five to sixteen rows where the kernel above has nothing to keep -- K too long for it (the down projection of
    // an MLP), or no more channel tiles than compute units, so that every workgroup would visit one tile and wait
    // for all of its activations first: the 16-row kernel that streams its activations k-block by k-block, one
    // workgroup per channel tile over all of K -- no split along K, no second launch (4096 -> 4096 at 16 rows:
    // 4.8 against 5.4 us; 14336 -> 4096 at 8 rows: 10.1 against 12.4 us for the small-batch kernel, at 16 rows 12.1
    // against 12.7; 4096 -> 1024, a quarter of the compute units: 3.75-4.7 against 3.9-4.8).  From 17 rows on every
    // tile's weights would be streamed twice.  OVFCC_GEMV16_STREAM = 0 switches it off, = 1 takes
    // it wherever it can run (before the kernel above, and whatever the number of channel tiles).
    const int stream_env = env_int("OVFCC_GEMV16_STREAM", -1);
    // Channel tiles per workgroup (their activations travel once for all of them): two where the node has more
    // tiles than the chip has compute units; OVFCC_GEMV16_STREAM_TILES = 1 | 2 | 4 overrides.  Measured against the
    // kernel above (8 / 16 rows): 4096 -> 8192 5.96 / 6.55 against 6.92 / 7.71 us, 4096 -> 6144 5.51 / 6.02 against
    // 6.53 / 7.22, 8192 -> 8192 9.08 / 10.29 against 11.90 / 12.45 (K in two parts and a summing launch) -- one round
    // of workgroups, taken up to 16 rows; 4096 -> 14336 (448 workgroups) 8.60 / 9.90 against 9.19 / 9.96 -- taken up
    // to 8 rows; 4096 -> 28672 (896 workgroups) 14.7 against 13.3 -- left to the kernel above.
    const int stream_tiles =
        env_int("OVFCC_GEMV16_STREAM_TILES", L.n_tiles > n_cus && L.n_tiles % 2 == 0 ? 2 : 1);
    const int64_t stream_wgs = L.n_tiles / (stream_tiles == 2 || stream_tiles == 4 ? stream_tiles : 1);
    const bool stream_first = stream_env == 1 || stream_wgs <= n_cus || (stream_wgs <= 2 * (int64_t)n_cus && a.M <= 8);
    auto plan_gemv16_stream = [&]() -> bool {
        if (a.M <= 4 || a.M > 16 || !a.scale_cm || L.bits != 4 || L.groups_per_kblock != 1 || L.kblocks_per_group != 1 ||
            force_split > 0 || L.gemv_c == 0 || L.glu || env_int("OVFCC_GEMV16", 1) == 0 ||
            stream_env == 0 || env_int("OVFCC_GEMV16_SPLIT", 0) > 0 || env_int("OVFCC_GEMV16_GRID", 0) > 0 ||
            env_int("OVFCC_DECODE_BATCH", -1) >= 0 || L.n_tiles * L.k_blocks * kTileBytes >= ((int64_t)1 << 31))
            return false;
        const int waves = (int)(L.k_blocks / L.gemv_c);
        if (L.k_blocks % L.gemv_c != 0 || waves < 1 || waves > 16 || (stream_env != 1 && L.n_tiles * 4 < n_cus))
            return false;
        int tiles = stream_tiles;
        if ((tiles != 1 && tiles != 2 && tiles != 4) || L.n_tiles % tiles != 0)
            tiles = 1;
        while (tiles > 1 && gemv16s_lds_bytes(waves, tiles) > 160 * 1024 - 64)
            tiles >>= 1;
        if (gemv16s_lds_bytes(waves, tiles) > 160 * 1024 - 64)
            return false;
        p.gemv16_stream = true;
        p.gemv_c = L.gemv_c;
        p.split_k = 1;
        p.kblocks_per_split = (int)L.k_blocks;
        p.tiles_per_group = tiles;
        p.grid[0] = (unsigned)(L.n_tiles / tiles);
        p.grid[1] = 1;
        p.grid[2] = 1;
        p.block = 64u * waves;
        p.tile_m = 16;
        p.tile_n = 16;
        p.dynamic_lds = (unsigned)gemv16s_lds_bytes(waves, tiles);
        p.workspace_bytes = 0;
        p.name = "fcc_gemv16s_w4";
        return true;
    };
    if (kernel == OVFCC_KERNEL_PLAIN) {
        if (a.M > 65535)
            return fail(OVFCC_EUNSUPPORTED, "the plain kernel handles at most 65535 rows");
        p.grid[0] = (unsigned)a.N_out;
        p.grid[1] = (unsigned)a.M;
        p.block = 64;
        p.name = "fcc_plain";
    } else if (kernel == OVFCC_KERNEL_DECODE && ((stream_first && plan_gemv16_stream()) || plan_gemv16() || plan_gemv16_stream())) {
        // planned
    } else if (kernel == OVFCC_KERNEL_DECODE && want_batch) {
        if (int rc = plan_batch())
            return rc;
    } else if (kernel == OVFCC_KERNEL_DECODE && a.M <= 4 && a.scale_cm && L.bits == 4 && L.groups_per_kblock == 1 &&
               L.kblocks_per_group == 1 && force_split <= 0 && env_int("OVFCC_GEMV", 1) != 0 && L.gemv_c != 0) {
        // One to four rows of a 4-bit node with groups of 128 inputs: the matrix-vector kernel.
        const int c = L.gemv_c;
        const int tiles_per_wg = L.glu ? 2 : 1;
        const int waves = (int)(L.k_blocks / c) * tiles_per_wg;
        p.gemv = true;
        p.gemv_c = c;
        p.split_k = 1;
        p.kblocks_per_split = (int)L.k_blocks;
        p.tiles_per_group = tiles_per_wg;
        p.grid[0] = (unsigned)(L.n_tiles / tiles_per_wg);
        p.block = 64u * waves;
        p.tile_m = 16;
        p.tile_n = 16 * tiles_per_wg;
        p.dynamic_lds = (unsigned)gemv_lds_bytes(c, (int)a.M, waves);
        p.name = "fcc_gemv_w4";
    } else if (kernel == OVFCC_KERNEL_DECODE) {
        if (a.M > 32)
            return fail(OVFCC_EUNSUPPORTED, "the streaming decode kernel handles at most 32 rows");
        const int kb = (int)L.k_blocks;
        const int mt = a.M <= 16 ? 1 : 2;
        // Activations go through LDS for M <= 4 when the k-range of one workgroup fits 40 KiB.
        bool xlds = a.M <= 4;
        const int x_env = env_int("OVFCC_DECODE_XLDS", -1);
        if (x_env == 0)
            xlds = false;
        int split = force_split;
        if (split <= 0) {
            split = 1;
            // K is split over workgroups only when the grid would otherwise leave compute units idle
            // (few channel tiles, long rows)
            const int64_t want_waves = (int64_t)16 * n_cus;
            while (split < 8 && L.n_tiles * 16 * split * 2 <= want_waves && kb / (split * 2) >= 32)
                split *= 2;
        }
        if (split > kb)
            split = kb;
        const int per = (kb + split - 1) / split;
        split = (kb + per - 1) / per;  // no empty splits
        const size_t x_bytes = (size_t)a.M * ((size_t)per * kBlockK + 8) * 2;
        if (x_bytes > 40 * 1024)  // does not fit beside the reduction buffer: read the operand from L2 instead
            xlds = false;
        // Two to four rows of a long-K, large node whose activations do not fit: the small-batch kernel's
        // shared staged slice beats per-lane reads of X from L2 (measured on K = 14336, N = 4096).
        if (!xlds && x_env != 0 && a.M > 1 && a.M <= 4 && L.w_bytes >= ((size_t)16 << 20) &&
            env_int("OVFCC_DECODE_BATCH", -1) < 0 && force_split <= 0) {
            if (int rc = plan_batch())
                return rc;
            *plan = p;
            return OVFCC_OK;
        }
        // Channel tiles per workgroup: one.  More tiles would share a staged activation copy between more
        // weights, but measured slower at M <= 4 (fewer, longer workgroups); the override stays for experiments.
        int rt = 1;
        if (xlds) {
            const int rt_max = L.bits == 4 ? 4 : 2;
            const int rt_env = env_int("OVFCC_DECODE_RT", 0);
            if ((rt_env == 1 || rt_env == 2 || rt_env == 4) && rt_env <= rt_max && L.n_tiles % rt_env == 0)
                rt = rt_env;
        }
        // A gated linear unit needs a gate tile and its up tile in one workgroup, which only the LDS-staged form
        // of this kernel offers; otherwise the small-batch kernel takes the node.
        if (L.glu && !xlds) {
            if (int rc = plan_batch())
                return rc;
            *plan = p;
            return OVFCC_OK;
        }
        if (L.glu && rt < 2)
            rt = 2;
        const int64_t groups = L.n_tiles / rt;
        // waves per workgroup: as many as the k-range feeds with four k-blocks each (the prefetch depth),
        // at most 16, and no more than about 16 waves per compute unit in total
        int nw = 16;
        while (nw > 4 && (per < 4 * nw || groups * split * nw > (int64_t)16 * n_cus || nw * rt > 32))
            nw >>= 1;
        const int nw_env = env_int("OVFCC_DECODE_WAVES", 0);
        if ((nw_env == 4 || nw_env == 8 || nw_env == 16) && nw_env * rt <= 32)
            nw = nw_env;
        p.split_k = split;
        p.kblocks_per_split = per;
        p.tiles_per_group = rt;
        p.x_in_lds = xlds;
        p.grid[0] = (unsigned)groups;
        p.grid[1] = (unsigned)split;
        p.block = 64u * nw;
        p.tile_m = 16 * mt;
        p.tile_n = 16 * rt;
        p.workspace_bytes = split > 1 ? (size_t)groups * split * rt * mt * 256 * sizeof(float) : 0;
        p.counter_count = split > 1 ? (size_t)groups : 0;
        p.dynamic_lds = (unsigned)((size_t)nw * rt * mt * 256 * sizeof(float) + (xlds ? x_bytes : 0));
        p.name = L.bits == 4 ? "fcc_decode_w4" : "fcc_decode_w8";
    } else {
        // The kernels with 128 x 256 tiles run when their grid still gives every second compute unit a tile;
        // otherwise, or when N is not a multiple of 256, the square kernel's smaller tiles spread the work
        // further.  Of the two, the register-fed kernel is the faster one; the LDS-dequantising one also needs
        // K % 256 == 0.  OVFCC_PREFILL_WIDE = 0 | 1 and OVFCC_PREFILL_DIRECT = 0 | 1 override for experiments.
        const int64_t m_tiles = (a.M + kPrefillTileM - 1) / kPrefillTileM;
        const int tiles_per_kb = L.bits == 4 ? 1 : 2;
        const bool direct_ok = (a.N % kPrefillWideN) == 0 && a.M * a.K * 2 < ((int64_t)1 << 31) &&
                               (int64_t)16 * L.k_blocks * tiles_per_kb * kTileBytes < ((int64_t)1 << 31);
        const bool wide_ok = direct_ok && (a.K % 256) == 0;
        // (the register-fed kernels can also split K, which multiplies their grid by up to eight)
        const bool may_split = direct_ok && env_int("OVFCC_PREFILL_DIRECT", 1) != 0;
        const bool may_async = may_split && L.bits == 4 && env_int("OVFCC_PREFILL_ASYNC", 1) != 0;
        // (and the 4-bit one has a form with 64-row tiles, which doubles the tile count of a grid that fits one round)
        int64_t reach = (a.N / kPrefillWideN) * m_tiles;
        if (may_split) {
            const int64_t tiles64 = (a.N / kPrefillWideN) * ((a.M + 63) / 64);
            if (may_async && tiles64 <= n_cus)
                reach = tiles64;
            for (int split = 1; split < 8 && reach * 2 <= n_cus && L.k_blocks / (split * 2) >= 8; split *= 2)
                reach *= 2;
        }
        bool big = reach * 2 >= n_cus || (a.want_async && may_async);
        const int wide_env = env_int("OVFCC_PREFILL_WIDE", -1);
        if (wide_env >= 0)
            big = wide_env != 0;
        // Groups of 32 or 64 inputs: only the all-asynchronous kernel and the square kernel carry several groups
        // per k-block.
        const bool small_groups = L.groups_per_kblock != 1;
        p.direct = big && direct_ok && env_int("OVFCC_PREFILL_DIRECT", 1) != 0 && (!small_groups || may_async);
        const bool wide = p.direct || (big && wide_ok && !small_groups);
        // 4-bit nodes take the variant whose operands all travel by direct-to-LDS loads
        p.async_dma = p.direct && L.bits == 4 && env_int("OVFCC_PREFILL_ASYNC", 1) != 0;
        p.tile_m = kPrefillTileM;
        p.tile_n = wide ? kPrefillWideN : kPrefillTileN;
        p.grid[0] = (unsigned)(a.N / p.tile_n);
        p.grid[1] = (unsigned)m_tiles;
        if (p.async_dma) {
            // 64-row tiles while they still fit the compute units in one round: a 64-row tile takes two thirds of
            // the time of a 128-row tile (same weight traffic and unpack work, half the MFMAs), so it pays only
            // where 128-row tiles would leave half the chip idle.  (OVFCC_PREFILL_ROWS = 64 | 128 overrides;
            // a.tile_rows, set by the grouped run, wins over both.)
            int rows = (int64_t)p.grid[0] * ((a.M + 63) / 64) <= n_cus ? 64 : 128;
            if (const int env_rows = env_int("OVFCC_PREFILL_ROWS", 0); env_rows == 64 || env_rows == 128)
                rows = env_rows;
            if (a.tile_rows == 64 || a.tile_rows == 128)
                rows = a.tile_rows;
            // (80 and 96 rows: grouped runs only, one group per k-block)
            if ((a.tile_rows == 80 || a.tile_rows == 96) && L.groups_per_kblock == 1)
                rows = a.tile_rows;
            if (rows != 128) {
                p.tile_m = rows == 80 || rows == 96 ? rows : 64;
                p.grid[1] = (unsigned)((a.M + p.tile_m - 1) / p.tile_m);
            }
        }
        p.kblocks_per_split = (int)L.k_blocks;
        if (p.direct) {
            // Split K while the tiles alone leave compute units idle (at least eight k-blocks per workgroup): the
            // f32 tiles are parked in the workspace and added by the last workgroup to arrive.
            // OVFCC_PREFILL_TAIL = 1 (an experiment, off by default) also splits, with more tiles than compute
            // units, the tiles of the last, partial round.  It does not pay: the chip is power-limited, a
            // half-empty round runs at a higher clock, and time is linear in tiles rather than in rounds.
            const int64_t tiles = (int64_t)p.grid[0] * p.grid[1];
            int split = force_split > 0 ? force_split : 1;
            int64_t full = 0;
            if (force_split <= 0) {
                while (split < 8 && tiles * split * 2 <= n_cus && L.k_blocks / (split * 2) >= 8)
                    split *= 2;
                const int64_t rest = tiles % n_cus;
                if (split == 1 && tiles > n_cus && rest * 2 <= n_cus && rest > 0 && L.k_blocks >= 16 &&
                    env_int("OVFCC_PREFILL_TAIL", 0) != 0) {
                    full = tiles - rest;
                    split = 2;
                    while (split < 8 && rest * split * 2 <= n_cus && L.k_blocks / (split * 2) >= 8)
                        split *= 2;
                }
            }
            if (split > L.k_blocks)
                split = (int)L.k_blocks;
            const int per = (int)((L.k_blocks + split - 1) / split);
            split = (int)((L.k_blocks + per - 1) / per);
            if (split == 1)
                full = tiles;
            p.split_k = split;
            p.kblocks_per_split = per;
            p.tiles_x = (int)p.grid[0];
            p.tiles_y = (int)p.grid[1];
            p.full_tiles = (int)full;
            p.grid[0] = (unsigned)(full + (tiles - full) * split);
            p.grid[1] = 1;
            p.workspace_bytes = split > 1 ? (size_t)(tiles - full) * split * p.tile_m * kPrefillWideN * sizeof(float) : 0;
            p.counter_count = split > 1 ? (size_t)(tiles - full) : 0;
        }
        p.block = wide ? 512 : 256;
        // 256 x 256 tiles (four waves with 512 registers each), where every unpacked weight meets twice the rows:
        // measured, such a tile costs 1.7 to 1.8 times a 128 x 256 tile.  It is whole tiles only, so it pays where
        // its rounds of tiles over the compute units, at that price, are no more than the rounds of the smaller
        // tiles: 256, 448, 512, 896, 1792 tiles yes; 128 or 300 no.  OVFCC_PREFILL_BIG = 0 | 1 overrides (1: whenever
        // the kernel can run the node).  A grouped run (a.tile_rows set) keeps its one row tile per slice.
        if (p.async_dma && p.split_k == 1 && p.tile_m == kPrefillTileM && L.groups_per_kblock == 1 && force_split <= 0 &&
            a.tile_rows == 0) {
            const int64_t big_tiles = (a.N / kPrefillWideN) * ((a.M + 255) / 256);
            const int64_t big_rounds = (big_tiles + n_cus - 1) / n_cus;
            const int64_t small_rounds = ((int64_t)p.tiles_x * p.tiles_y + n_cus - 1) / n_cus;
            const int big_env = env_int("OVFCC_PREFILL_BIG", -1);
            if (big_env > 0 || (big_env < 0 && big_tiles >= n_cus && big_rounds * 100 <= small_rounds * 58)) {
                p.big = true;
                p.tile_m = 256;
                p.tiles_y = (int)((a.M + 255) / 256);
                p.full_tiles = p.tiles_x * p.tiles_y;
                p.grid[0] = (unsigned)p.full_tiles;
                p.block = 256;
            }
        }
        if (p.big)
            p.name = "fcc_prefill_big_w4";
        else
        p.name = L.bits == 4 ? (p.async_dma ? "fcc_prefill_async_w4" : p.direct ? "fcc_prefill_direct_w4" : wide ? "fcc_prefill_wide_w4" : "fcc_prefill_w4")
                             : (p.direct ? "fcc_prefill_direct_w8" : wide ? "fcc_prefill_wide_w8" : "fcc_prefill_w8");
    }
    *plan = p;
    return OVFCC_OK;
}

int launch_fc(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    if (a.M == 0)
        return 0;
    switch (p.kernel) {
    case OVFCC_KERNEL_PLAIN:
        return launch_plain(a, p, stream);
    case OVFCC_KERNEL_DECODE:
        return p.gemv     ? launch_gemv(a, p, stream)
               : p.gemv16 ? launch_gemv16(a, p, stream)
               : p.gemv16_stream ? launch_gemv16_stream(a, p, stream)
               : p.batch  ? launch_batch(a, p, stream)
                          : launch_decode(a, p, stream);
    default:
        if (p.big)
            return launch_prefill_big(a, p, stream);
        if (p.async_dma)
            return launch_prefill_async(a, p, stream);
        if (p.direct)
            return launch_prefill_direct(a, p, stream);
        return p.tile_n == kPrefillWideN ? launch_prefill_wide(a, p, stream) : launch_prefill(a, p, stream);
    }
}

// Slice height of a grouped prefill launch over items of these row counts: every item is cut into equal slices of
// at most that many rows and every slice is one tile.  Measured on a mixture-of-experts layer, a tile of 64 / 80 /
// 96 rows costs 0.78 / 0.84 / 0.89 of a 128-row tile (the unpack work and the data movement of a tile do not
// depend on its height), so the height that needs the fewest tiles wins unless a lower one needs no more.
// mid_ok: tiles of 80 and 96 rows exist (one group per k-block).  OVFCC_PREFILL_ROWS = 64 | 80 | 96 | 128 overrides.
int rows_cap_for(const int64_t* rows, int n, bool mid_ok) {
    static const int caps[4] = {64, 80, 96, 128}, cost[4] = {780, 836, 890, 1000};
    if (const int forced = env_int("OVFCC_PREFILL_ROWS", 0))
        return forced == 64 ? 64 : ((forced == 80 || forced == 96) && mid_ok) ? forced : kPrefillGroupRows;
    int best = kPrefillGroupRows;
    int64_t best_cost = -1;
    for (int c = 0; c < 4; ++c) {
        if (!mid_ok && (caps[c] == 80 || caps[c] == 96))
            continue;
        int64_t total = 0;
        for (int i = 0; i < n; ++i)
            total += (rows[i] + caps[c] - 1) / caps[c] * cost[c];
        if (best_cost < 0 || total < best_cost)
            best_cost = total, best = caps[c];
    }
    return best;
}

}  // namespace ovfcc
