// Stand-ins for the kernel launchers, so that the host sources link without the device code.  Never called: the
// host checks exercise descriptors, layouts, plans and graph decisions only.
#pragma once

#include "ovfcc_internal.h"

namespace ovfcc {
int launch_plain(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_decode(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_batch(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_gemv(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_gemv16(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_gemv16_stream(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
size_t gemv16s_lds_bytes(int waves, int tiles) { return tiles >= 1 && tiles <= 8 ? (size_t)waves * (2 * 4096) : (size_t)-1; }
int gemv16_kblocks_per_wave(int c_table, int split_k) { return split_k > 1 ? c_table / split_k : (c_table == 2 ? 2 : 4); }
size_t gemv16_lds_bytes(int c, int waves, int red_bufs) { return (size_t)waves * c * 4096 + (size_t)red_bufs * waves * 1024; }
int launch_prefill(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_prefill_wide(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_prefill_direct(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_prefill_async(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
int launch_prefill_big(const FcDeviceArgs&, const LaunchPlan&, void*) { return -1; }
}  // namespace ovfcc
