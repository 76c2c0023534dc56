// Kernel choice and launch decomposition (host only).
//
// Policy: shapes that keep OpenVINO's layout run the plain kernel; tiled nodes run the decode kernel
// for M <= 32 and the prefill kernel above (the roofline ridge of int4 g128 sits near M = 83; the
// decode kernel's activation operand stops scaling at two 16-row tiles).
#include <cstdlib>

#include "ovfcc_internal.h"

namespace ovfcc {

// Tuning override for experiments: OVFCC_DECODE_WAVES = 4 | 8 | 16 fixes the decode workgroup size.
static int env_decode_waves() {
    const char* e = std::getenv("OVFCC_DECODE_WAVES");
    if (!e)
        return 0;
    const int v = std::atoi(e);
    return (v == 4 || v == 8 || v == 16) ? v : 0;
}

int plan_launch(const FcDeviceArgs& a, int force_kernel, int force_split, int n_cus, LaunchPlan* plan) {
    LaunchPlan p;
    const Layout& L = a.layout;
    int kernel = force_kernel;
    if (kernel == OVFCC_KERNEL_AUTO)
        kernel = !L.tiled ? OVFCC_KERNEL_PLAIN : (a.M <= 32 ? OVFCC_KERNEL_DECODE : OVFCC_KERNEL_PREFILL);
    if (kernel != OVFCC_KERNEL_PLAIN && !L.tiled)
        return fail(OVFCC_EUNSUPPORTED, "this node keeps the OpenVINO layout; only the plain kernel can run it");
    if (kernel == OVFCC_KERNEL_PLAIN && L.tiled)
        return fail(OVFCC_EUNSUPPORTED, "this node was repacked into tiles; the plain kernel needs the OpenVINO layout");
    if (kernel == OVFCC_KERNEL_DECODE && a.M > 32)
        return fail(OVFCC_EUNSUPPORTED, "the decode kernel handles at most 32 rows");
    if (kernel == OVFCC_KERNEL_PREFILL && (a.N % kPrefillTileN) != 0)
        return fail(OVFCC_EUNSUPPORTED, "the prefill kernel needs N % 128 == 0");
    p.kernel = kernel;
    if (kernel == OVFCC_KERNEL_PLAIN) {
        if (a.M > 65535)
            return fail(OVFCC_EUNSUPPORTED, "the plain kernel handles at most 65535 rows");
        p.grid[0] = (unsigned)a.N;
        p.grid[1] = (unsigned)a.M;
        p.block = 64;
        p.name = "fcc_plain";
    } else if (kernel == OVFCC_KERNEL_DECODE) {
        const int kb = (int)L.k_blocks;
        const int mt = a.M <= 16 ? 1 : 2;
        // Waves per workgroup: as many as the k-range feeds (one k-block each at least), up to 16, so that
        // a 16-channel tile is reduced inside one workgroup whenever possible.  K is split over workgroups
        // only when the grid would otherwise leave compute units idle (few channel tiles, long rows).
        int split = force_split;
        if (split <= 0) {
            split = 1;
            const int64_t want_waves = (int64_t)16 * n_cus;
            while (split < 8 && L.n_tiles * 16 * split * 2 <= want_waves && kb / (split * 2) >= 32)
                split *= 2;
        }
        if (split > kb)
            split = kb;
        const int per = (kb + split - 1) / split;
        split = (kb + per - 1) / per;  // no empty splits
        int nw = 16;
        while (nw > 4 && (per < nw || L.n_tiles * split * nw > (int64_t)24 * n_cus))
            nw >>= 1;
        if (const int forced = env_decode_waves())
            nw = forced;
        p.split_k = split;
        p.kblocks_per_split = per;
        p.grid[0] = (unsigned)L.n_tiles;
        p.grid[1] = (unsigned)split;
        p.block = 64u * nw;
        p.tile_m = 16 * mt;
        p.tile_n = 16;
        p.workspace_bytes = split > 1 ? (size_t)L.n_tiles * split * mt * 256 * sizeof(float) : 0;
        p.counter_count = split > 1 ? (size_t)L.n_tiles : 0;
        p.dynamic_lds = (unsigned)(nw * mt * 256 * sizeof(float));
        p.name = L.bits == 4 ? "fcc_decode_w4" : "fcc_decode_w8";
    } else {
        p.grid[0] = (unsigned)(a.N / kPrefillTileN);
        p.grid[1] = (unsigned)((a.M + kPrefillTileM - 1) / kPrefillTileM);
        p.block = 256;
        p.tile_m = kPrefillTileM;
        p.tile_n = kPrefillTileN;
        p.name = L.bits == 4 ? "fcc_prefill_w4" : "fcc_prefill_w8";
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
        return launch_decode(a, p, stream);
    default:
        return launch_prefill(a, p, stream);
    }
}

}  // namespace ovfcc
