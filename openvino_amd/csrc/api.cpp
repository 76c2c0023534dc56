// C ABI over the HIP runtime: contexts, repacked weights, requests, execution, benchmarking loops.
// Every function returns an OVFCC_* code and records the reason with ovfcc::fail.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "api_types.h"
#include "ovfcc_graph.h"
#include "ovfcc_internal.h"

namespace {

using ovfcc::fail;

constexpr size_t kHostStageMax = (size_t)1 << 20;  // host transfers up to this size (x and y together) are staged

int hip_fail(hipError_t e, const char* what) {
    return fail(e == hipErrorOutOfMemory ? OVFCC_ENOMEM : OVFCC_EDEVICE,
                std::string(what) + ": " + hipGetErrorString(e));
}

#define HIP_TRY(expr)                       \
    do {                                    \
        hipError_t _e = (expr);             \
        if (_e != hipSuccess)               \
            return hip_fail(_e, #expr);     \
    } while (0)

int grow(void** p, size_t* cap, size_t need) {
    if (need <= *cap)
        return OVFCC_OK;
    if (*p)
        HIP_TRY(hipFree(*p));
    *p = nullptr;
    *cap = 0;
    HIP_TRY(hipMalloc(p, need));
    *cap = need;
    return OVFCC_OK;
}

int ensure_split_buffers(ovfcc_request* r, const ovfcc::LaunchPlan& plan) {
    if (plan.workspace_bytes > r->ws_cap) {
        HIP_TRY(hipStreamSynchronize(r->stream));
        int rc = grow(reinterpret_cast<void**>(&r->workspace), &r->ws_cap, plan.workspace_bytes);
        if (rc)
            return rc;
    }
    if (plan.counter_count > r->counter_cap) {
        HIP_TRY(hipStreamSynchronize(r->stream));
        size_t cap_bytes = r->counter_cap * sizeof(unsigned);
        int rc = grow(reinterpret_cast<void**>(&r->counters), &cap_bytes, plan.counter_count * sizeof(unsigned));
        if (rc)
            return rc;
        r->counter_cap = plan.counter_count;
        // counters return to zero at the end of every launch; they only need clearing once
        HIP_TRY(hipMemsetAsync(r->counters, 0, plan.counter_count * sizeof(unsigned), r->stream));
        HIP_TRY(hipStreamSynchronize(r->stream));
    }
    return OVFCC_OK;
}

// The fixed scratch array of ovfcc_fc_run_device_static is one per device, shared by every context and request on
// it: a launch that uses it waits, on its stream, for the event recorded behind the last such launch.  The event is
// created by the first ovfcc_init on the device and lives as long as the array, so that the entry point itself
// creates nothing.
struct StaticGuard {
    std::mutex mu;
    hipEvent_t done = nullptr;
    bool recorded = false;
};
constexpr int kGuardedDevices = 64;
StaticGuard g_static_guard[kGuardedDevices];

StaticGuard* static_guard(int device) {
    return device >= 0 && device < kGuardedDevices ? &g_static_guard[device] : nullptr;
}

// Split-K workspace and arrival counters for one launch: the request's own buffers (grown on demand), or -- for
// the entry point that allocates nothing -- the device's fixed scratch array, whose counters are cleared by a fill
// kernel ahead of the launch (the array keeps whatever the last call left, on this or any other request).
int split_buffers(ovfcc_request* r, const ovfcc::LaunchPlan& plan, bool static_scratch, ovfcc::FcDeviceArgs* a) {
    if (!static_scratch) {
        int rc = ensure_split_buffers(r, plan);
        a->workspace = r->workspace;
        a->counters = r->counters;
        return rc;
    }
    a->workspace = nullptr;
    a->counters = nullptr;
    if (plan.workspace_bytes == 0 && plan.counter_count == 0)
        return OVFCC_OK;
    if (plan.workspace_bytes > ovfcc::kStaticWorkspaceBytes ||
        plan.counter_count * sizeof(unsigned) > ovfcc::kStaticCounterBytes)
        return fail(OVFCC_EUNSUPPORTED,
                    "this launch splits K and needs " + std::to_string(plan.workspace_bytes) + " bytes of partial tiles and " +
                        std::to_string(plan.counter_count) + " counters; the fixed scratch array holds " +
                        std::to_string(ovfcc::kStaticWorkspaceBytes) + " bytes and " +
                        std::to_string(ovfcc::kStaticCounterBytes / sizeof(unsigned)) + " counters");
    unsigned char* base = static_cast<unsigned char*>(ovfcc::static_scratch_ptr(r->ctx->device));
    if (!base)
        return fail(OVFCC_EDEVICE, "the fixed scratch array was not set up on this device");
    a->counters = reinterpret_cast<unsigned*>(base);
    a->workspace = reinterpret_cast<float*>(base + ovfcc::kStaticCounterBytes);
    // every request of the device shares the array: order this launch behind the last one that used it, whichever
    // stream that ran on.  (A capturing stream cannot wait for an event from outside its capture; a caller that
    // captures keeps such launches of different requests apart itself.)
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    HIP_TRY(hipStreamIsCapturing(r->stream, &cap));
    StaticGuard* g = static_guard(r->ctx->device);
    if (cap == hipStreamCaptureStatusNone && g && g->done) {
        std::lock_guard<std::mutex> lock(g->mu);
        if (g->recorded)
            HIP_TRY(hipStreamWaitEvent(r->stream, g->done, 0));
    }
    int e = ovfcc::launch_zero_u32(a->counters, plan.counter_count, r->stream);
    if (e)
        return hip_fail((hipError_t)e, "counter fill launch");
    return OVFCC_OK;
}

// Behind a launch that used the fixed scratch array: the point the next such launch waits for.
int static_scratch_released(ovfcc_request* r, const ovfcc::FcDeviceArgs& a) {
    unsigned char* base = static_cast<unsigned char*>(ovfcc::static_scratch_ptr(r->ctx->device));
    if (!base || reinterpret_cast<unsigned char*>(a.counters) != base)
        return OVFCC_OK;  // the launch did not split K: nothing of the array was used
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    HIP_TRY(hipStreamIsCapturing(r->stream, &cap));
    if (cap != hipStreamCaptureStatusNone)
        return OVFCC_OK;
    StaticGuard* g = static_guard(r->ctx->device);
    if (!g || !g->done)
        return OVFCC_OK;
    std::lock_guard<std::mutex> lock(g->mu);
    HIP_TRY(hipEventRecord(g->done, r->stream));
    g->recorded = true;
    return OVFCC_OK;
}

// row length of the node's output
int64_t out_channels(const ovfcc_weights* w) {
    return w->layout.glu ? w->desc.N / 2 : w->desc.N;
}

// the node whose output leaves the object: the down projection of an MLP node, else the node itself
const ovfcc_weights* output_node(const ovfcc_weights* w) {
    return w->mlp_down ? w->mlp_down : w;
}

void fill_args(const ovfcc_weights* w, const void* x, void* y, int64_t M, ovfcc::FcDeviceArgs* a) {
    a->w = w->d_w;
    a->scale = w->d_scale;
    a->zp = w->d_zp;
    a->bias = w->d_bias;
    a->scale_cm = w->d_scale_cm;
    a->zp_cm = w->d_zp_cm;
    a->x = x;
    a->y = y;
    a->workspace = nullptr;
    a->counters = nullptr;
    a->M = M;
    a->N = w->desc.N;
    a->K = w->desc.K;
    a->group_size = w->desc.group_size;
    a->w_type = w->desc.w_type;
    a->zp_type = w->desc.zp_type;
    a->zp_scalar = w->desc.zp_scalar;
    a->out_f32 = w->desc.out_type == OVFCC_F32 ? 1 : 0;
    a->N_out = out_channels(w);
    a->gate_offset = w->layout.glu_gate_second ? (int)(w->desc.N / 2) : 0;
    a->up_offset = w->layout.glu_gate_second ? 0 : (int)(w->desc.N / 2);
    a->layout = w->layout;
}

// Last step of every way a node comes into being: tiled 4-bit nodes with groups of 128 inputs get channel-major
// copies of their scales and zero-point table, [N/16][16][K/128], which the matrix-vector kernel reads.
int finish_weights(ovfcc_weights* W) {
    ovfcc::Layout& L = W->layout;
    L.gemv_c = 0;
    // 8-bit nodes with one scale per channel whose activations may be quantised asymmetrically: the sums of their
    // zero-point-corrected weights per channel, which the activations' zero-points multiply
    if (L.dynquant_asym && L.tiled && L.bits == 8 && L.groups == 1 && W->desc.K <= ovfcc::kI8AsymMaxK && !W->d_colsum) {
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&W->d_colsum), (size_t)W->desc.N * sizeof(int)));
        W->bytes += (size_t)W->desc.N * sizeof(int);
        int e = ovfcc::launch_i8_colsum(W->d_w, L.zp_table ? W->d_zp : nullptr, L.zp_const, W->d_colsum, L.n_tiles,
                                        L.k_blocks, nullptr);
        if (e)
            return hip_fail((hipError_t)e, "column sum launch");
        HIP_TRY(hipStreamSynchronize(nullptr));
    }
    if (!L.tiled || L.bits != 4 || L.groups_per_kblock != 1 || L.kblocks_per_group != 1 || !W->d_scale)
        return OVFCC_OK;
    const int c = ovfcc::gemv_kblocks_per_wave(L, W->ctx->n_cus);
    if (c == 0)
        return OVFCC_OK;
    HIP_TRY(hipMalloc(&W->d_scale_cm, L.scale_bytes));
    W->bytes += L.scale_bytes;
    if (L.zp_table) {
        HIP_TRY(hipMalloc(&W->d_zp_cm, L.zp_bytes));
        W->bytes += L.zp_bytes;
    }
    int e = ovfcc::launch_gemv_params(W->d_scale, L.zp_table ? W->d_zp : nullptr, W->d_scale_cm, W->d_zp_cm, L.n_tiles,
                                      L.groups, c, nullptr);
    if (e)
        return hip_fail((hipError_t)e, "parameter transposition launch");
    HIP_TRY(hipStreamSynchronize(nullptr));
    L.gemv_c = c;
    return OVFCC_OK;
}

// Buckets the (row, selected expert) pairs of a routed batch by expert, rows in ascending order inside a bucket:
// the bucketing of the reference's CPU executor
// (src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_gathermatmul_executor.cpp:492-509).  count / start receive
// the bucket sizes and offsets.  Two maps of R = M * top_k entries each are left in the request's pinned buffer for
// upload: first[slot] = the row of A that bucket slot `slot` reads (m, or i * M + m when A has one batch per
// selection), and second[slot] = i * M + m, the row of a [top_k, M, .] result (inverse == false), or
// second[m * top_k + i] = slot (inverse == true).  Waits for the previous call's upload to have left the buffer.
int bucket_rows(ovfcc_request* r, const int32_t* indices, int64_t M, int top_k, int n_experts, int a_batches,
                bool inverse, std::vector<int>* count, std::vector<int>* start) {
    const int64_t R = M * top_k;
    count->assign(n_experts, 0);
    start->assign(n_experts + 1, 0);
    for (int64_t m = 0; m < M; ++m)
        for (int i = 0; i < top_k; ++i) {
            const int32_t e = indices[m * top_k + i];
            if (e < 0 || e >= n_experts)
                return fail(OVFCC_EINVAL, "an expert index is out of range");
            ++(*count)[e];
        }
    for (int e = 0; e < n_experts; ++e)
        (*start)[e + 1] = (*start)[e] + (*count)[e];
    const size_t map_bytes = (size_t)2 * R * sizeof(int);
    if (!r->maps_uploaded)
        HIP_TRY(hipEventCreateWithFlags(&r->maps_uploaded, hipEventDisableTiming));
    else
        HIP_TRY(hipEventSynchronize(r->maps_uploaded));
    if (map_bytes > r->h_maps_cap) {
        if (r->h_maps)
            HIP_TRY(hipHostFree(r->h_maps));
        r->h_maps = nullptr, r->h_maps_cap = 0;
        HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&r->h_maps), map_bytes, hipHostMallocDefault));
        r->h_maps_cap = map_bytes;
    }
    std::vector<int> at(start->begin(), start->end() - 1);
    int* first = r->h_maps;
    int* second = r->h_maps + R;
    for (int64_t m = 0; m < M; ++m)
        for (int i = 0; i < top_k; ++i) {
            const int slot = at[indices[m * top_k + i]]++;
            first[slot] = (int)(a_batches == 1 ? m : (int64_t)i * M + m);
            if (inverse)
                second[m * top_k + i] = slot;
            else
                second[slot] = (int)((int64_t)i * M + m);
        }
    return OVFCC_OK;
}

void record(ovfcc_request* r, const ovfcc::LaunchPlan& p) {
    ovfcc_kernel_info& i = r->last;
    std::memset(&i, 0, sizeof(i));
    i.kernel = p.kernel;
    i.grid[0] = (int32_t)p.grid[0];
    i.grid[1] = (int32_t)p.grid[1];
    i.grid[2] = (int32_t)p.grid[2];
    i.block = (int32_t)p.block;
    i.split_k = p.split_k;
    i.tile_m = p.tile_m;
    i.tile_n = p.tile_n;
    std::snprintf(i.name, sizeof(i.name), "%s", p.name);
    if (ovfcc::env_int("OVFCC_VERBOSE", 0) >= 1)
        std::fprintf(stderr, "ovfcc: launch %s grid=(%u,%u,%u) block=%u tile=%dx%d split_k=%d\n", p.name, p.grid[0],
                     p.grid[1], p.grid[2], p.block, p.tile_m, p.tile_n, p.split_k);
}

// OVFCC_VERBOSE >= 2: the call is bracketed by events and waited for, and its time and algorithmic bandwidth
// (weights, scales, zero-points, activations and results once each) are printed.  Serialises the stream.
struct VerboseTimer {
    ovfcc_request* r;
    const ovfcc_weights* w;
    int64_t M;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    VerboseTimer(ovfcc_request* req, const ovfcc_weights* wt, int64_t rows) : r(req), w(wt), M(rows) {
        if (ovfcc::env_int("OVFCC_VERBOSE", 0) < 2 || M == 0)
            return;
        if (hipEventCreate(&t0) != hipSuccess || hipEventCreate(&t1) != hipSuccess) {
            (void)hipGetLastError();
            t0 = t1 = nullptr;
            return;
        }
        (void)hipEventRecord(t0, r->stream);
    }
    ~VerboseTimer() {
        if (!t0 || !t1)
            return;
        float ms = 0.f;
        if (hipEventRecord(t1, r->stream) == hipSuccess && hipEventSynchronize(t1) == hipSuccess &&
            hipEventElapsedTime(&ms, t0, t1) == hipSuccess && ms > 0.f) {
            const ovfcc_fc_desc& d = w->desc;
            const double out_n = (double)((d.flags & OVFCC_GLU_TYPE_MASK) ? d.N / 2 : d.N);
            const double bytes = (double)w->bytes + (double)M * d.K * 2 + (double)M * out_n * (d.out_type == OVFCC_F32 ? 4 : 2);
            std::fprintf(stderr, "ovfcc: run M=%lld N=%lld K=%lld %s: %.2f us, %.0f GB/s, %.1f TFLOP/s\n", (long long)M,
                         (long long)d.N, (long long)d.K, r->last.name, ms * 1e3, bytes / ms / 1e6,
                         2.0 * M * d.N * d.K / ms / 1e9);
        }
        (void)hipEventDestroy(t0);
        (void)hipEventDestroy(t1);
    }
};

int enqueue_rows(ovfcc_request* r, const ovfcc_weights* w, const void* x, void* y, int64_t M, bool static_scratch);

// Enqueue one node.  The fast kernels address the activations with 32-bit byte offsets and the plain kernel puts
// the rows on a 16-bit grid axis: a longer node runs as consecutive row blocks on the same stream.
int enqueue_mlp(ovfcc_request* r, const ovfcc_weights* w, const void* x, void* y, int64_t M, bool static_scratch);

int enqueue(ovfcc_request* r, const ovfcc_weights* w, const void* x, void* y, int64_t M, bool static_scratch = false,
            bool first_node_only = false) {
    if (w->mlp_down && !first_node_only)
        return enqueue_mlp(r, w, x, y, M, static_scratch);
    int64_t block = M;
    if (w->layout.tiled) {
        const int64_t lim = ((((int64_t)1 << 31) - 1) / (2 * w->desc.K)) & ~(int64_t)127;
        if (M > lim && lim >= 128)
            block = lim;
    } else if (M > 65535) {
        block = 65535;
    }
    const size_t out_row = (size_t)out_channels(w) * (w->desc.out_type == OVFCC_F32 ? 4 : 2);
    for (int64_t m0 = 0; m0 < M; m0 += block) {
        const int64_t rows = M - m0 < block ? M - m0 : block;
        int rc = enqueue_rows(r, w, static_cast<const char*>(x) + (size_t)m0 * w->desc.K * 2,
                              static_cast<char*>(y) + (size_t)m0 * out_row, rows, static_scratch);
        if (rc)
            return rc;
    }
    return OVFCC_OK;
}

// plan_launch for a call of the node on its own (fill_args's arguments, nothing set by a grouped run), through the
// node's cache: the plan depends on the node, M, the request's overrides, the chip and the environment overrides.
int cached_plan(const ovfcc_request* r, const ovfcc_weights* w, const ovfcc::FcDeviceArgs& a, int force,
                ovfcc::LaunchPlan* p) {
    const unsigned gen = ovfcc::env_generation();
    {
        std::lock_guard<std::mutex> lock(w->plan_mu);
        for (const auto& e : w->plans)
            if (e.M == a.M && e.force_kernel == force && e.force_split == r->force_split && e.n_cus == r->ctx->n_cus &&
                e.env_generation == gen) {
                *p = e.plan;
                return OVFCC_OK;
            }
    }
    int rc = ovfcc::plan_launch(a, force, r->force_split, r->ctx->n_cus, p);
    if (rc)
        return rc;
    std::lock_guard<std::mutex> lock(w->plan_mu);
    auto& e = w->plans[w->plan_next++ % 8];
    e.M = a.M, e.force_kernel = force, e.force_split = r->force_split, e.n_cus = r->ctx->n_cus, e.env_generation = gen;
    e.plan = *p;
    return OVFCC_OK;
}

// One block of rows.  A tiled node is cut into decode-family launches of at most 48 rows when M is small
// enough that they beat one sparse prefill grid, or when N is not a multiple of the prefill tile.
int enqueue_rows(ovfcc_request* r, const ovfcc_weights* w, const void* x, void* y, int64_t M, bool static_scratch) {
    if (M == 0)
        return OVFCC_OK;
    ovfcc::FcDeviceArgs a;
    fill_args(w, x, y, M, &a);
    int force = r->force_kernel;
    // Per-token int8 activations where the node allows them and the integer kernel applies: prefill row counts,
    // 8-bit weights with one scale per channel, whole 256-channel tiles.
    const ovfcc::Layout& L0 = w->layout;
    if (L0.dynquant && L0.tiled && L0.bits == 8 && L0.groups == 1 && (w->desc.N % 256) == 0 &&
        M > ovfcc::kDecodeMaxRows && (force == OVFCC_KERNEL_AUTO || force == OVFCC_KERNEL_PREFILL) &&
        M * w->desc.K < ((int64_t)1 << 31) && (M + 127) / 128 <= 65535 &&
        // (it has no split-K: a grid that leaves half the chip idle stays with the f16 kernels, which have;
        // OVFCC_PREFILL_WIDE = 1 forces the 256-wide kernels onto small shapes, for tests)
        ((w->desc.N / 256) * ((M + 127) / 128) * 2 >= r->ctx->n_cus ||
         ovfcc::env_int("OVFCC_PREFILL_WIDE", -1) == 1)) {
        if (static_scratch)
            return fail(OVFCC_EUNSUPPORTED, "a node with int8 activations needs a quantisation buffer of the request");
        const size_t q_bytes = ((size_t)M * w->desc.K + 255) & ~(size_t)255;
        const size_t need = q_bytes + (size_t)M * 12;
        if (need > r->quant_cap)
            HIP_TRY(hipStreamSynchronize(r->stream));
        int rc = grow(&r->d_quant, &r->quant_cap, need);
        if (rc)
            return rc;
        char* base = static_cast<char*>(r->d_quant);
        float* inv_scale = reinterpret_cast<float*>(base + q_bytes);
        int* qsum = reinterpret_cast<int*>(base + q_bytes + (size_t)M * 4);
        // unsigned bytes with a zero-point per token where the node asks for them (and has its column sums)
        int* za = w->d_colsum ? reinterpret_cast<int*>(base + q_bytes + (size_t)M * 8) : nullptr;
        int e = za ? ovfcc::launch_dynquant_asym(x, base, inv_scale, qsum, za, M, w->desc.K, r->stream)
                   : ovfcc::launch_dynquant(x, base, inv_scale, qsum, M, w->desc.K, r->stream);
        if (!e)
            e = ovfcc::launch_prefill_i8(a, base, inv_scale, qsum, za, w->d_colsum, r->stream);
        if (e)
            return hip_fail((hipError_t)e, "integer kernel launch");
        ovfcc::LaunchPlan shown;
        shown.kernel = OVFCC_KERNEL_PREFILL;
        shown.tile_m = 128, shown.tile_n = 256, shown.block = 512;
        shown.grid[0] = (unsigned)(w->desc.N / 256), shown.grid[1] = (unsigned)((M + 127) / 128);
        shown.name = za ? "fcc_prefill_i8_w8_asym" : "fcc_prefill_i8_w8";
        record(r, shown);
        return OVFCC_OK;
    }
    // The same permission for 4-bit weights with groups of 128 inputs (W4A8): activations per token, or per row
    // and group where the node asks for it.
    if (L0.dynquant && ovfcc::prefill_i8w4_applies(L0, w->desc.N, w->desc.zp_type) && M > ovfcc::kDecodeMaxRows &&
        (force == OVFCC_KERNEL_AUTO || force == OVFCC_KERNEL_PREFILL) && M * w->desc.K < ((int64_t)1 << 31) &&
        (M + 127) / 128 <= 65535 &&
        ((w->desc.N / 256) * ((M + 127) / 128) * 2 >= r->ctx->n_cus ||
         ovfcc::env_int("OVFCC_PREFILL_WIDE", -1) == 1)) {
        if (static_scratch)
            return fail(OVFCC_EUNSUPPORTED, "a node with int8 activations needs a quantisation buffer of the request");
        const bool grouped = L0.dynquant_grouped;
        const size_t q_bytes = ((size_t)M * w->desc.K + 255) & ~(size_t)255;
        const size_t need = q_bytes + ovfcc::dynquant_w4_scale_floats(M, w->desc.K, grouped) * sizeof(float);
        if (need > r->quant_cap)
            HIP_TRY(hipStreamSynchronize(r->stream));
        int rc = grow(&r->d_quant, &r->quant_cap, need);
        if (rc)
            return rc;
        char* base = static_cast<char*>(r->d_quant);
        float* inv_scale = reinterpret_cast<float*>(base + q_bytes);
        int e = ovfcc::launch_dynquant_w4(x, base, inv_scale, M, w->desc.K, grouped, r->stream);
        if (!e)
            e = ovfcc::launch_prefill_i8w4(a, base, inv_scale, grouped, r->stream);
        if (e)
            return hip_fail((hipError_t)e, "integer kernel launch");
        ovfcc::LaunchPlan shown;
        shown.kernel = OVFCC_KERNEL_PREFILL;
        shown.tile_m = 128, shown.tile_n = 256, shown.block = 512;
        shown.grid[0] = (unsigned)(w->desc.N / 256), shown.grid[1] = (unsigned)((M + 127) / 128);
        shown.name = grouped ? "fcc_prefill_i8_w4_grouped" : "fcc_prefill_i8_w4";
        record(r, shown);
        return OVFCC_OK;
    }
    bool chunked = w->layout.tiled && M > ovfcc::kDecodeMaxRows &&
                   ((force == OVFCC_KERNEL_AUTO && M <= ovfcc::kChunkedMaxRows) ||
                    ((w->desc.N % 128) != 0 && (force == OVFCC_KERNEL_AUTO || force == OVFCC_KERNEL_PREFILL)));
    if (chunked && force == OVFCC_KERNEL_AUTO && M > ovfcc::kChunkedMinPrefillRows && (w->desc.N % 128) == 0) {
        // a register-fed prefill kernel (K split; 64-row tiles for 4-bit weights) beats two or three decode
        // launches wherever its grid fills the chip; measured on the Llama-3-8B and -70B shapes
        ovfcc::LaunchPlan p;
        if (ovfcc::plan_launch(a, OVFCC_KERNEL_PREFILL, r->force_split, r->ctx->n_cus, &p) == OVFCC_OK && p.direct)
            chunked = false;
    }
    if (chunked) {
        const int64_t chunks = (M + ovfcc::kDecodeMaxRows - 1) / ovfcc::kDecodeMaxRows;
        const int64_t step = (M + chunks - 1) / chunks;  // equal shares rather than 48 + remainder
        for (int64_t m0 = 0; m0 < M; m0 += step) {
            const int64_t rows = M - m0 < step ? M - m0 : step;
            fill_args(w, static_cast<const char*>(x) + (size_t)m0 * w->desc.K * 2,
                      static_cast<char*>(y) + (size_t)m0 * out_channels(w) * (w->desc.out_type == OVFCC_F32 ? 4 : 2), rows, &a);
            ovfcc::LaunchPlan p;
            int rc = ovfcc::plan_launch(a, OVFCC_KERNEL_DECODE, r->force_split, r->ctx->n_cus, &p);
            if (rc)
                return rc;
            rc = split_buffers(r, p, static_scratch, &a);
            if (rc)
                return rc;
            int e = ovfcc::launch_fc(a, p, r->stream);
            if (e)
                return hip_fail((hipError_t)e, "kernel launch");
            if (static_scratch && (rc = static_scratch_released(r, a)))
                return rc;
            record(r, p);
        }
        return OVFCC_OK;
    }
    ovfcc::LaunchPlan p;
    int rc = cached_plan(r, w, a, force, &p);
    if (rc)
        return rc;
    rc = split_buffers(r, p, static_scratch, &a);
    if (rc)
        return rc;
    int e = ovfcc::launch_fc(a, p, r->stream);
    if (e)
        return hip_fail((hipError_t)e, "kernel launch");
    if (static_scratch && (rc = static_scratch_released(r, a)))
        return rc;
    record(r, p);
    return OVFCC_OK;
}


// ---- mixture-of-experts layers with the routing done on the device --------------------------------------------
// The grouped launch whose slices the routing kernel cuts: tiled 4-bit experts that the all-asynchronous prefill
// kernel runs, at most kMaxGroupItems of them (their pointers travel in the routing kernel's arguments).  The
// slice height is fixed from the average bucket (the counts stay on the device; rows_cap_for).  How many slices the buckets make is known on the device only, where
// the routing kernel also chooses the cut along K for that count; grid, workspace and counters are sized for the
// worst count up to ceil(R / cap) + n_experts, and workgroups beyond the header's grid return at once.
struct RoutedLaunch {
    int cap = 0, n_slices = 0;
    ovfcc::LaunchPlan plan;
    ovfcc::FcDeviceArgs args;
};

bool plan_routed(ovfcc_request* r, const ovfcc_weights* w0, int64_t R, int n_experts, RoutedLaunch* out) {
    if (n_experts > ovfcc::kMaxGroupItems || !w0->layout.tiled || w0->layout.bits != 4 ||
        r->force_kernel != OVFCC_KERNEL_AUTO || R <= 0)
        return false;
    // the counts stay on the device: plan for buckets of the average size plus twice its square root (what random
    // routing stays under)
    const double avg = (double)R / n_experts;
    const int64_t likely = (int64_t)std::ceil(avg + 2.0 * std::sqrt(avg));
    int cap = ovfcc::rows_cap_for(&likely, 1, w0->layout.groups_per_kblock == 1);
    const int64_t n = (R + cap - 1) / cap + n_experts;
    if (n * cap * w0->desc.K * 2 >= ((int64_t)1 << 31) || n > 65535)
        return false;
    fill_args(w0, nullptr, nullptr, n * cap, &out->args);
    out->args.tile_rows = cap;
    out->args.want_async = true;
    if (ovfcc::plan_launch(out->args, OVFCC_KERNEL_PREFILL, r->force_split, r->ctx->n_cus, &out->plan) != OVFCC_OK ||
        !out->plan.async_dma || out->plan.big || out->plan.tiles_y != (int)n)
        return false;
    ovfcc::LaunchPlan& p = out->plan;
    int grid = 0;
    long long parked = 0;
    for (int t = 1; t <= (int)n; ++t) {
        const ovfcc::RoutedHeader h = ovfcc::routed_header(p.tiles_x, t, (int)w0->layout.k_blocks, r->ctx->n_cus);
        grid = std::max(grid, h.grid);
        parked = std::max(parked, ovfcc::routed_parked_tiles(h, p.tiles_x));
    }
    p.n_cus = r->ctx->n_cus;
    p.grid[0] = (unsigned)grid, p.grid[1] = p.grid[2] = 1;
    p.workspace_bytes = (size_t)parked * p.tile_m * ovfcc::kPrefillWideN * sizeof(float);
    p.counter_count = parked ? (size_t)p.tiles_x * n : 0;
    out->cap = cap;
    out->n_slices = (int)n;
    return true;
}

int run_routed(ovfcc_request* r, const ovfcc_weights* const* experts, int n_experts, RoutedLaunch& L,
               const int* indices_dev, int64_t M, int top_k, int a_batches, int inverse, int x_mapped, const void* x_base,
               size_t x_row_bytes, void* y_base, size_t y_row_bytes, int* d_maps, ovfcc::RoutedHeader* d_header,
               const ovfcc::SecondTable* second_table = nullptr, void* unrouted_y = nullptr) {
    auto* d_table = reinterpret_cast<ovfcc::BatchGroupItem*>(d_header + 1);
    ovfcc::ExpertPointers ptrs{};
    for (int e = 0; e < n_experts; ++e)
        ptrs.w[e] = experts[e]->d_w, ptrs.scale[e] = experts[e]->d_scale, ptrs.zp[e] = experts[e]->d_zp,
        ptrs.bias[e] = experts[e]->d_bias;
    const int64_t R = M * top_k;
    L.args.row_map = x_mapped ? d_maps : nullptr;
    L.args.x_rows = x_mapped ? (int64_t)a_batches * M : 0;
    int e1 = ovfcc::launch_moe_route(indices_dev, M, top_k, n_experts, a_batches, inverse, L.cap, x_mapped, ptrs, x_base,
                                     x_row_bytes, y_base, y_row_bytes, d_maps, d_maps + R, d_table, L.n_slices, d_header,
                                     L.plan.tiles_x, (int)experts[0]->layout.k_blocks, L.plan.n_cus, r->stream,
                                     second_table, unrouted_y, y_row_bytes);
    if (e1)
        return hip_fail((hipError_t)e1, "routing kernel launch");
    return OVFCC_OK;
}

int launch_routed(ovfcc_request* r, RoutedLaunch& L, const ovfcc::RoutedHeader* d_header) {
    auto* d_table = reinterpret_cast<const ovfcc::BatchGroupItem*>(d_header + 1);
    int rc = ensure_split_buffers(r, L.plan);
    if (rc)
        return rc;
    L.args.workspace = r->workspace;
    L.args.counters = r->counters;
    const ovfcc::BatchGroupTable none{};
    const int e = ovfcc::launch_prefill_async_grouped(none, L.n_slices, L.args, L.plan, r->stream, d_table, d_header);
    if (e)
        return hip_fail((hipError_t)e, "grouped kernel launch");
    ovfcc::LaunchPlan shown = L.plan;
    shown.name = "fcc_prefill_async_grouped_w4";
    record(r, shown);
    return OVFCC_OK;
}

// Same shape, format, bias presence and scalar zero-point for every expert (one grouped launch carries one of each).
int experts_agree(const ovfcc_request* r, const ovfcc_weights* const* experts, int n_experts, bool* same_zp) {
    const ovfcc_weights* w0 = experts[0];
    *same_zp = true;
    for (int e = 0; e < n_experts; ++e) {
        const ovfcc_weights* w = experts[e];
        if (!w || w->ctx != r->ctx)
            return fail(OVFCC_EINVAL, "an expert's weights are null or belong to another context");
        if (std::memcmp(&w->desc, &w0->desc, sizeof(ovfcc_fc_desc)) != 0 || (w->d_bias != nullptr) != (w0->d_bias != nullptr))
            return fail(OVFCC_EUNSUPPORTED, "experts differ in shape, types, bias or output type");
        if (w->layout.zp_const != w0->layout.zp_const)
            *same_zp = false;
    }
    return OVFCC_OK;
}

// Indices given in host memory: checked there, then copied to the device through the request's pinned buffer.
int upload_indices(ovfcc_request* r, const int32_t* indices, int64_t R, int n_experts, int* d_indices) {
    for (int64_t j = 0; j < R; ++j)
        if (indices[j] < 0 || indices[j] >= n_experts)
            return fail(OVFCC_EINVAL, "an expert index is out of range");
    const size_t bytes = (size_t)R * sizeof(int);
    if (!r->maps_uploaded)
        HIP_TRY(hipEventCreateWithFlags(&r->maps_uploaded, hipEventDisableTiming));
    else
        HIP_TRY(hipEventSynchronize(r->maps_uploaded));  // the previous call's copy has left the buffer
    if (bytes > r->h_maps_cap) {
        if (r->h_maps)
            HIP_TRY(hipHostFree(r->h_maps));
        r->h_maps = nullptr, r->h_maps_cap = 0;
        HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&r->h_maps), bytes, hipHostMallocDefault));
        r->h_maps_cap = bytes;
    }
    std::memcpy(r->h_maps, indices, bytes);
    HIP_TRY(hipMemcpyAsync(d_indices, r->h_maps, bytes, hipMemcpyHostToDevice, r->stream));
    HIP_TRY(hipEventRecord(r->maps_uploaded, r->stream));
    return OVFCC_OK;
}

// GatherMatmul with the routing on the device.  indices_dev is in device memory, or indices_host is given and
// copied there.  Returns OVFCC_EUNSUPPORTED (without an error string of its own) when no routed launch fits.
int gather_matmul_routed(ovfcc_request* r, const ovfcc_weights* const* experts, int n_experts, const void* a_dev,
                         int a_batches, const int32_t* indices_dev, const int32_t* indices_host, int64_t M, int top_k,
                         void* y_dev, bool* ran) {
    *ran = false;
    const ovfcc_weights* w0 = experts[0];
    const int64_t K = w0->desc.K, N_out = out_channels(w0), R = M * top_k;
    const size_t out_bytes = w0->desc.out_type == OVFCC_F32 ? 4 : 2;
    RoutedLaunch L;
    if (!plan_routed(r, w0, R, n_experts, &L))
        return OVFCC_OK;
    auto up256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t x_bytes = (size_t)R * K * 2, y_bytes = (size_t)R * N_out * out_bytes;
    const size_t y_off = up256(x_bytes), m_off = up256(y_off + y_bytes), t_off = up256(m_off + (size_t)2 * R * sizeof(int));
    const size_t i_off = up256(t_off + sizeof(ovfcc::RoutedHeader) + (size_t)L.n_slices * sizeof(ovfcc::BatchGroupItem));
    const size_t need = i_off + (size_t)R * sizeof(int);
    if (need > r->gather_cap)
        HIP_TRY(hipStreamSynchronize(r->stream));
    int rc = grow(&r->d_gather, &r->gather_cap, need);
    if (rc)
        return rc;
    char* base = static_cast<char*>(r->d_gather);
    int* d_maps = reinterpret_cast<int*>(base + m_off);
    auto* d_table = reinterpret_cast<ovfcc::RoutedHeader*>(base + t_off);  // header, then the slices
    if (!indices_dev) {
        rc = upload_indices(r, indices_host, R, n_experts, reinterpret_cast<int*>(base + i_off));
        if (rc)
            return rc;
        indices_dev = reinterpret_cast<const int32_t*>(base + i_off);
    }
    // (the grouped launch reads the rows of A through the map: no gathered copy)
    rc = run_routed(r, experts, n_experts, L, indices_dev, M, top_k, a_batches, 0, 1, a_dev, (size_t)K * 2, base + y_off,
                    (size_t)N_out * out_bytes, d_maps, d_table, nullptr, y_dev);
    if (rc)
        return rc;
    rc = launch_routed(r, L, d_table);
    if (rc)
        return rc;
    int e1 = ovfcc::launch_rows(y_dev, base + y_off, nullptr, d_maps + R, (int)R, (int)(N_out * out_bytes), r->stream);
    if (e1)
        return hip_fail((hipError_t)e1, "row scatter launch");
    *ran = true;
    return OVFCC_OK;
}

int moe_routed(ovfcc_request* r, const ovfcc_weights* const* gate_up, const ovfcc_weights* const* down, int n_experts,
               const void* x_dev, const void* routing_dev, const int32_t* indices_dev, const int32_t* indices_host,
               int64_t M, int top_k, void* y_dev, bool* ran) {
    *ran = false;
    const ovfcc_weights *g0 = gate_up[0], *d0 = down[0];
    const int64_t H = g0->desc.K, I = out_channels(g0), R = M * top_k;
    const int d_f32 = d0->desc.out_type == OVFCC_F32 ? 1 : 0;
    RoutedLaunch Lg, Ld;
    if (!plan_routed(r, g0, R, n_experts, &Lg) || !plan_routed(r, d0, R, n_experts, &Ld))
        return OVFCC_OK;
    auto up256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t x_bytes = (size_t)R * H * 2, h_bytes = (size_t)R * I * 2, d_bytes = (size_t)R * H * (d_f32 ? 4 : 2);
    const size_t h_off = up256(x_bytes), d_off = up256(h_off + h_bytes), m_off = up256(d_off + d_bytes);
    const size_t tg_off = up256(m_off + (size_t)2 * R * sizeof(int));
    const size_t td_off = up256(tg_off + sizeof(ovfcc::RoutedHeader) + (size_t)Lg.n_slices * sizeof(ovfcc::BatchGroupItem));
    const size_t i_off = up256(td_off + sizeof(ovfcc::RoutedHeader) + (size_t)Ld.n_slices * sizeof(ovfcc::BatchGroupItem));
    const size_t need = i_off + (size_t)R * sizeof(int);
    if (need > r->gather_cap)
        HIP_TRY(hipStreamSynchronize(r->stream));
    int rc = grow(&r->d_gather, &r->gather_cap, need);
    if (rc)
        return rc;
    char* base = static_cast<char*>(r->d_gather);
    int* d_maps = reinterpret_cast<int*>(base + m_off);
    auto* tab_g = reinterpret_cast<ovfcc::RoutedHeader*>(base + tg_off);  // header, then the slices
    auto* tab_d = reinterpret_cast<ovfcc::RoutedHeader*>(base + td_off);
    if (!indices_dev) {
        rc = upload_indices(r, indices_host, R, n_experts, reinterpret_cast<int*>(base + i_off));
        if (rc)
            return rc;
        indices_dev = reinterpret_cast<const int32_t*>(base + i_off);
    }
    // the routing kernel runs once per projection: same buckets and maps, a slice table each
    // (gate/up read the hidden states through the map: no gathered copy of them)
    if (n_experts <= ovfcc::kMaxSecondTableItems && Lg.cap == Ld.cap && Lg.n_slices == Ld.n_slices) {
        // one routing launch writes both slice tables: the buckets are the same, the down projection reads the
        // bucket slots of the gate/up results in place
        ovfcc::SecondTable t2{};
        for (int e = 0; e < n_experts; ++e)
            t2.w[e] = down[e]->d_w, t2.scale[e] = down[e]->d_scale, t2.zp[e] = down[e]->d_zp, t2.bias[e] = down[e]->d_bias;
        t2.x_base = base + h_off, t2.x_row_bytes = (size_t)I * 2;
        t2.y_base = base + d_off, t2.y_row_bytes = (size_t)H * (d_f32 ? 4 : 2);
        t2.table = reinterpret_cast<ovfcc::BatchGroupItem*>(tab_d + 1), t2.header = tab_d;
        t2.tiles_x = Ld.plan.tiles_x, t2.kb_total = (int)d0->layout.k_blocks;
        rc = run_routed(r, gate_up, n_experts, Lg, indices_dev, M, top_k, 1, 1, 1, x_dev, (size_t)H * 2, base + h_off,
                        (size_t)I * 2, d_maps, tab_g, &t2);
    } else {
        rc = run_routed(r, gate_up, n_experts, Lg, indices_dev, M, top_k, 1, 1, 1, x_dev, (size_t)H * 2, base + h_off,
                        (size_t)I * 2, d_maps, tab_g);
        if (!rc)
            rc = run_routed(r, down, n_experts, Ld, indices_dev, M, top_k, 1, 1, 0, base + h_off, (size_t)I * 2,
                            base + d_off, (size_t)H * (d_f32 ? 4 : 2), d_maps, tab_d);
    }
    if (rc)
        return rc;
    rc = launch_routed(r, Lg, tab_g);
    if (!rc)
        rc = launch_routed(r, Ld, tab_d);
    if (rc)
        return rc;
    const int e1 = ovfcc::launch_moe_combine(y_dev, base + d_off, routing_dev, d_maps + R, (int)M, top_k, (int)H, d_f32, d_f32,
                                   r->stream);
    if (e1)
        return hip_fail((hipError_t)e1, "expert combine launch");
    *ran = true;
    return OVFCC_OK;
}

// An MLP node: the gate / up node into the request's intermediate buffer and the down node out of it, as two
// launches; with OVFCC_MLP_FUSED = 1 the one-launch kernel for one to four rows of nodes it can run.  (Measured on
// the Llama-3-8B block at one row: one launch 21.7 us, two launches 18.9 us -- publishing the intermediate row,
// raising the flags and reading the row back are three trips through a memory system whose queues hold the down
// projection's weights, and cost more than the second launch they replace.  The kernel stays an option.)
int enqueue_mlp(ovfcc_request* r, const ovfcc_weights* w, const void* x, void* y, int64_t M, bool static_scratch) {
    if (M == 0)
        return OVFCC_OK;
    if (static_scratch)
        return fail(OVFCC_EUNSUPPORTED, "an MLP node needs the request's intermediate buffer");
    const ovfcc_weights* d = w->mlp_down;
    const int64_t I = out_channels(w);
    const size_t mid_bytes = (size_t)M * I * 2;
    if (mid_bytes > r->mid_cap) {
        HIP_TRY(hipStreamSynchronize(r->stream));
        int rc = grow(&r->d_mid, &r->mid_cap, mid_bytes);
        if (rc)
            return rc;
    }
    // One workgroup per compute unit (OVFCC_MLP_GRID overrides).  Fewer workgroups that share the tile pairs evenly
    // were measured and lose: a compute unit's throughput is what its sixteen waves keep in flight, so the weight
    // stream slows with the number of workgroups (Llama-3-8B block: 256 workgroups 21.6 us, 224 23.9, 128 26.4).
    int grid = r->ctx->n_cus;
    if (const int forced = ovfcc::env_int("OVFCC_MLP_GRID", 0); forced > 0 && forced <= r->ctx->n_cus)
        grid = forced;
    const bool fused = M <= 4 && r->force_kernel == OVFCC_KERNEL_AUTO && r->force_split == 0 &&
                       ovfcc::env_int("OVFCC_MLP_FUSED", 0) != 0 && w->d_scale_cm && d->d_scale_cm &&
                       ovfcc::mlp_fused_applies(w->layout, d->layout, M, grid);
    if (!fused) {
        int rc = enqueue(r, w, x, r->d_mid, M, false, true);
        if (rc)
            return rc;
        return enqueue(r, d, r->d_mid, y, M);
    }
    const size_t sync_bytes = ovfcc::mlp_sync_bytes(r->ctx->n_cus);
    if (!r->d_sync) {
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&r->d_sync), sync_bytes));
        HIP_TRY(hipMemset(r->d_sync, 0, sync_bytes));
        HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&r->h_error), 64, hipHostMallocDefault));
        *r->h_error = 0;
    }
    if (*r->h_error) {
        // an earlier launch gave up its wait: its counters may be anywhere; start from zero again
        HIP_TRY(hipStreamSynchronize(r->stream));
        HIP_TRY(hipMemset(r->d_sync, 0, sync_bytes));
        *r->h_error = 0;
        return fail(OVFCC_EDEVICE, "an earlier MLP launch on this request gave up waiting for its workgroups");
    }
    ovfcc::FcDeviceArgs ga, da;
    fill_args(w, x, r->d_mid, M, &ga);
    fill_args(d, r->d_mid, y, M, &da);
    const int spin_env = ovfcc::env_int("OVFCC_MLP_SPIN_LIMIT", 0);
    const unsigned spin_limit = spin_env > 0 ? (unsigned)spin_env : (1u << 20);
    // One launch of this kind on the device at a time: its workgroups wait for each other, and two such grids that
    // each hold half the compute units would wait for good.  The launch waits for the one before it on any stream.
    // (A capturing stream cannot wait for an event from outside its capture; a caller that captures keeps such
    // launches of different requests apart itself.)
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    HIP_TRY(hipStreamIsCapturing(r->stream, &cap));
    std::lock_guard<std::mutex> lock(r->ctx->coop_mu);
    if (cap == hipStreamCaptureStatusNone) {
        if (!r->ctx->coop_done)
            HIP_TRY(hipEventCreateWithFlags(&r->ctx->coop_done, hipEventDisableTiming));
        else
            HIP_TRY(hipStreamWaitEvent(r->stream, r->ctx->coop_done, 0));
    }
    int e = ovfcc::launch_mlp(ga, da, r->d_mid, r->d_sync, r->h_error, grid, r->ctx->n_cus, spin_limit, r->stream);
    if (e)
        return hip_fail((hipError_t)e, "MLP kernel launch");
    if (cap == hipStreamCaptureStatusNone)
        HIP_TRY(hipEventRecord(r->ctx->coop_done, r->stream));
    ovfcc::LaunchPlan shown;
    shown.kernel = OVFCC_KERNEL_DECODE;
    shown.tile_m = 16, shown.tile_n = 16, shown.block = 1024;
    shown.grid[0] = (unsigned)grid;
    shown.name = "fcc_mlp_gemv_w4";
    record(r, shown);
    return OVFCC_OK;
}

}  // namespace

extern "C" {

int ovfcc_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

void ovfcc_env_reload(void) {
    ovfcc::env_reload();
}

int ovfcc_init(int device, ovfcc_ctx** out) {
    if (!out)
        return fail(OVFCC_EINVAL, "out is null");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        (void)hipGetLastError();
        return fail(OVFCC_EDEVICE, "no HIP device is visible; this library has no CPU path");
    }
    if (device < 0 || device >= n)
        return fail(OVFCC_EINVAL, "device index out of range");
    (void)ovfcc::env_generation();  // the OVFCC_* overrides are read here, once
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    std::string arch = prop.gcnArchName;
    if (arch.rfind("gfx950", 0) != 0)
        return fail(OVFCC_EDEVICE, "device is " + arch + "; the kernels are built for gfx950 only");
    // the fixed scratch array of ovfcc_fc_run_device_static: its address on this device, looked up once
    if (int se = ovfcc::static_scratch_setup(device))
        return hip_fail((hipError_t)se, "hipGetSymbolAddress of the fixed scratch array");
    if (StaticGuard* g = static_guard(device)) {
        std::lock_guard<std::mutex> lock(g->mu);
        if (!g->done)
            HIP_TRY(hipEventCreateWithFlags(&g->done, hipEventDisableTiming));
    }
    ovfcc_ctx* c = new ovfcc_ctx();
    c->device = device;
    c->n_cus = prop.multiProcessorCount;
    c->arch = arch;
    *out = c;
    return OVFCC_OK;
}

void ovfcc_destroy(ovfcc_ctx* ctx) {
    if (ctx && ctx->coop_done)
        (void)hipEventDestroy(ctx->coop_done);
    delete ctx;
}

int ovfcc_device_mem_info(ovfcc_ctx* ctx, size_t* free_bytes, size_t* total_bytes) {
    if (!ctx || !free_bytes || !total_bytes)
        return fail(OVFCC_EINVAL, "null argument");
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
    return OVFCC_OK;
}

int ovfcc_weights_create(ovfcc_ctx* ctx, const ovfcc_fc_desc* desc, const void* w, const void* scales, const void* zp,
                         const void* bias, ovfcc_weights** out) {
    if (!ctx || !out)
        return fail(OVFCC_EINVAL, "ctx or out is null");
    *out = nullptr;
    int rc = ovfcc::validate_desc(desc);
    if (rc)
        return rc;
    if (!w || !scales)
        return fail(OVFCC_EINVAL, "weights and scales are required");
    if (desc->zp_type != OVFCC_NONE && !zp)
        return fail(OVFCC_EINVAL, "zero-point type given without a buffer");
    if (desc->bias_type != OVFCC_NONE && !bias)
        return fail(OVFCC_EINVAL, "bias type given without a buffer");
    HIP_TRY(hipSetDevice(ctx->device));

    // Input-major constants are transposed once, here; from then on the node is the [N, K] node.
    ovfcc::OutputMajorCopy nk;
    ovfcc_fc_desc own = *desc;
    if (own.flags & OVFCC_W_INPUT_MAJOR) {
        ovfcc::transpose_input_major(own, w, scales, zp, &nk);
        w = nk.w.data(), scales = nk.scales.data(), zp = nk.zp.empty() ? zp : nk.zp.data();
        own.flags &= ~OVFCC_W_INPUT_MAJOR;
    }
    desc = &own;

    ovfcc_weights* W = new ovfcc_weights();
    W->ctx = ctx;
    W->desc = *desc;
    W->layout = ovfcc::make_layout(*desc);
    ovfcc::Layout& L = W->layout;
    if (desc->zp_type != OVFCC_NONE && desc->zp_scalar)
        L.zp_const = ovfcc::scalar_zero_point(*desc, zp) + L.zp_offset;

    auto upload = [&](void** dst, const void* src, size_t bytes) -> int {
        if (bytes == 0)
            return OVFCC_OK;
        HIP_TRY(hipMalloc(dst, bytes));
        HIP_TRY(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        W->bytes += bytes;
        return OVFCC_OK;
    };

    const int64_t N = desc->N, K = desc->K, ng = L.groups;
    const auto t_start = std::chrono::steady_clock::now();
    auto t_repacked = t_start;
    if (L.tiled) {
        std::vector<uint8_t> wt(L.w_bytes), st(L.scale_bytes), zt(L.zp_bytes);
        ovfcc::repack_weights(*desc, L, w, wt.data());
        ovfcc::repack_params(*desc, L, scales, zp, st.data(), zt.data());
        t_repacked = std::chrono::steady_clock::now();
        rc = upload(&W->d_w, wt.data(), wt.size());
        if (!rc)
            rc = upload(&W->d_scale, st.data(), st.size());
        if (!rc && L.zp_table)
            rc = upload(&W->d_zp, zt.data(), zt.size());
    } else {
        const bool four = desc->w_type == OVFCC_U4 || desc->w_type == OVFCC_I4;
        const size_t wb = four ? (size_t)(N * K + 1) / 2 : (size_t)N * K;
        rc = upload(&W->d_w, w, wb);
        if (!rc)
            rc = upload(&W->d_scale, scales, (size_t)N * ng * 2);
        if (!rc && desc->zp_type != OVFCC_NONE) {
            const size_t cnt = desc->zp_scalar ? 1 : (size_t)N * ng;
            rc = upload(&W->d_zp, zp, desc->zp_type == OVFCC_U4 ? (cnt + 1) / 2 : cnt);
        }
    }
    if (!rc && desc->bias_type != OVFCC_NONE) {
        if (L.tiled && L.glu) {  // bias follows the channel order of the tiles
            const uint16_t* b = static_cast<const uint16_t*>(bias);
            std::vector<uint16_t> bt((size_t)N);
            for (int64_t nt = 0; nt < L.n_tiles; ++nt)
                std::memcpy(&bt[(size_t)nt * ovfcc::kTileRows], b + L.source_tile(nt) * ovfcc::kTileRows,
                            ovfcc::kTileRows * 2);
            rc = upload(&W->d_bias, bt.data(), (size_t)N * 2);
        } else {
            rc = upload(&W->d_bias, bias, (size_t)N * 2);
        }
    }
    if (!rc)
        rc = finish_weights(W);
    if (rc) {
        ovfcc_weights_destroy(W);
        return rc;
    }
    if (ovfcc::env_int("OVFCC_VERBOSE", 0) >= 1) {
        using ms = std::chrono::duration<double, std::milli>;
        const auto t_end = std::chrono::steady_clock::now();
        std::fprintf(stderr, "ovfcc: weights N=%lld K=%lld group=%lld w_type=%d zp_type=%d%s: %s layout, %zu bytes on the "
                     "device, repack %.2f ms, upload %.2f ms\n", (long long)N, (long long)K, (long long)desc->group_size,
                     desc->w_type, desc->zp_type, desc->zp_scalar ? " (scalar)" : "", L.tiled ? "tiled" : "OpenVINO",
                     W->bytes, ms(t_repacked - t_start).count(), ms(t_end - t_repacked).count());
    }
    *out = W;
    return OVFCC_OK;
}

void ovfcc_weights_destroy(ovfcc_weights* w) {
    if (!w)
        return;
    ovfcc_weights_destroy(w->mlp_down);
    if (w->d_w) (void)hipFree(w->d_w);
    if (w->d_scale) (void)hipFree(w->d_scale);
    if (w->d_zp) (void)hipFree(w->d_zp);
    if (w->d_bias) (void)hipFree(w->d_bias);
    if (w->d_scale_cm) (void)hipFree(w->d_scale_cm);
    if (w->d_colsum) (void)hipFree(w->d_colsum);
    if (w->d_zp_cm) (void)hipFree(w->d_zp_cm);
    delete w;
}

int ovfcc_weights_clone(const ovfcc_weights* src, ovfcc_weights** out) {
    if (!src || !out)
        return fail(OVFCC_EINVAL, "null argument");
    *out = nullptr;
    HIP_TRY(hipSetDevice(src->ctx->device));
    ovfcc_weights* W = new ovfcc_weights();
    W->ctx = src->ctx;
    W->desc = src->desc;
    W->layout = src->layout;
    const ovfcc::Layout& L = src->layout;
    const int64_t N = src->desc.N, K = src->desc.K, ng = L.groups;
    const bool four = L.bits == 4;
    size_t wb, sb, zb = 0;
    if (L.tiled) {
        wb = L.w_bytes;
        sb = L.scale_bytes;
        zb = L.zp_bytes;
    } else {
        wb = four ? (size_t)(N * K + 1) / 2 : (size_t)N * K;
        sb = (size_t)N * ng * 2;
        if (src->desc.zp_type != OVFCC_NONE) {
            const size_t cnt = src->desc.zp_scalar ? 1 : (size_t)N * ng;
            zb = src->desc.zp_type == OVFCC_U4 ? (cnt + 1) / 2 : cnt;
        }
    }
    auto dup = [&](void** dst, const void* from, size_t bytes) -> int {
        if (!from || bytes == 0)
            return OVFCC_OK;
        HIP_TRY(hipMalloc(dst, bytes));
        HIP_TRY(hipMemcpy(*dst, from, bytes, hipMemcpyDeviceToDevice));
        W->bytes += bytes;
        return OVFCC_OK;
    };
    int rc = dup(&W->d_w, src->d_w, wb);
    if (!rc) rc = dup(&W->d_scale, src->d_scale, sb);
    if (!rc) rc = dup(&W->d_zp, src->d_zp, zb);
    if (!rc) rc = dup(&W->d_bias, src->d_bias, (size_t)N * 2);
    if (!rc)
        rc = finish_weights(W);
    if (!rc && src->mlp_down)
        rc = ovfcc_weights_clone(src->mlp_down, &W->mlp_down);
    if (rc) {
        ovfcc_weights_destroy(W);
        return rc;
    }
    *out = W;
    return OVFCC_OK;
}

static int create_from(ovfcc_ctx* ctx, ovfcc::FoldConstants& c, int extra_flags, ovfcc_weights** out) {
    c.desc.flags |= extra_flags;
    return ovfcc_weights_create(ctx, &c.desc, c.weights, c.scales.data(), c.zero_points.empty() ? nullptr : c.zero_points.data(),
                                c.bias.empty() ? nullptr : c.bias.data(), out);
}

int ovfcc_fold_weights_create(ovfcc_ctx* ctx, const ovfcc_gnode* nodes, int n_nodes, const ovfcc_fold* fold,
                              const void* const* constant_data, int extra_flags, ovfcc_weights** out) {
    if (!ctx || !fold || !out)
        return fail(OVFCC_EINVAL, "null argument");
    *out = nullptr;
    ovfcc::FoldConstants c;
    if (int rc = ovfcc::fold_constants(nodes, n_nodes, *fold, constant_data, c))
        return rc;
    return create_from(ctx, c, extra_flags, out);
}

int ovfcc_fold_expert_weights_create(ovfcc_ctx* ctx, const ovfcc_gnode* nodes, int n_nodes, const ovfcc_gather_fold* fold,
                                     int expert, const void* const* constant_data, int extra_flags, ovfcc_weights** out) {
    if (!ctx || !fold || !out)
        return fail(OVFCC_EINVAL, "null argument");
    *out = nullptr;
    ovfcc::FoldConstants c;
    if (int rc = ovfcc::fold_expert_constants(nodes, n_nodes, *fold, expert, constant_data, c))
        return rc;
    return create_from(ctx, c, extra_flags, out);
}

int ovfcc_weights_mlp(const ovfcc_weights* gate_up, const ovfcc_weights* down, ovfcc_weights** out) {
    if (!gate_up || !down || !out)
        return fail(OVFCC_EINVAL, "null argument");
    *out = nullptr;
    if (gate_up->ctx != down->ctx)
        return fail(OVFCC_EINVAL, "the two nodes belong to different contexts");
    if (gate_up->mlp_down || down->mlp_down)
        return fail(OVFCC_EINVAL, "an MLP node cannot be part of another");
    if (!gate_up->layout.glu)
        return fail(OVFCC_EINVAL, "the first node must carry a gated linear unit (ovfcc_weights_glu or OVFCC_GLU_* flags)");
    if (down->layout.glu)
        return fail(OVFCC_EINVAL, "the down projection must not carry a gated linear unit");
    if (gate_up->desc.out_type != OVFCC_F16)
        return fail(OVFCC_EUNSUPPORTED, "the intermediate activations are f16: the first node's output_type must be f16");
    if (out_channels(gate_up) != down->desc.K)
        return fail(OVFCC_EINVAL, "the down projection's K (" + std::to_string(down->desc.K) +
                                      ") is not the first node's output width (" +
                                      std::to_string(out_channels(gate_up)) + ")");
    ovfcc_weights* W = nullptr;
    int rc = ovfcc_weights_clone(gate_up, &W);
    if (rc)
        return rc;
    rc = ovfcc_weights_clone(down, &W->mlp_down);
    if (rc) {
        ovfcc_weights_destroy(W);
        return rc;
    }
    *out = W;
    return OVFCC_OK;
}

int ovfcc_weights_concat(const ovfcc_weights* const* parts, int n_parts, ovfcc_weights** out) {
    for (int i = 0; parts && i < n_parts; ++i)
        if (parts[i] && parts[i]->mlp_down)
            return fail(OVFCC_EINVAL, "an MLP node cannot be concatenated");
    if (!parts || n_parts <= 0 || !out)
        return fail(OVFCC_EINVAL, "null or empty part list");
    *out = nullptr;
    const ovfcc_weights* first = parts[0];
    if (!first)
        return fail(OVFCC_EINVAL, "part 0 is null");
    int64_t n_total = 0;
    for (int i = 0; i < n_parts; ++i) {
        const ovfcc_weights* p = parts[i];
        if (!p)
            return fail(OVFCC_EINVAL, "a part is null");
        if (!p->layout.tiled)
            return fail(OVFCC_EUNSUPPORTED, "only tiled nodes can be fused");
        if (p->layout.glu)
            return fail(OVFCC_EUNSUPPORTED, "a node with a gated-linear-unit epilogue cannot be a part");
        const bool same = p->ctx == first->ctx && p->desc.K == first->desc.K &&
                          p->desc.group_size == first->desc.group_size && p->desc.w_type == first->desc.w_type &&
                          p->desc.zp_type == first->desc.zp_type && p->desc.zp_scalar == first->desc.zp_scalar &&
                          p->desc.bias_type == first->desc.bias_type && p->desc.out_type == first->desc.out_type &&
                          p->layout.zp_const == first->layout.zp_const;
        if (!same)
            return fail(OVFCC_EUNSUPPORTED,
                        "parts differ in K, group size, types, scalar zero-point, bias or output type");
        n_total += p->desc.N;
    }
    HIP_TRY(hipSetDevice(first->ctx->device));
    ovfcc_weights* W = new ovfcc_weights();
    W->ctx = first->ctx;
    W->desc = first->desc;
    W->desc.N = n_total;
    W->layout = ovfcc::make_layout(W->desc);
    W->layout.zp_const = first->layout.zp_const;
    const ovfcc::Layout& L = W->layout;
    auto gather = [&](void** dst, size_t total, void* ovfcc_weights::*member, auto bytes_of) -> int {
        if (total == 0)
            return OVFCC_OK;
        HIP_TRY(hipMalloc(dst, total));
        W->bytes += total;
        size_t at = 0;
        for (int i = 0; i < n_parts; ++i) {
            const size_t b = bytes_of(parts[i]);
            HIP_TRY(hipMemcpy(static_cast<char*>(*dst) + at, parts[i]->*member, b, hipMemcpyDeviceToDevice));
            at += b;
        }
        return OVFCC_OK;
    };
    int rc = gather(&W->d_w, L.w_bytes, &ovfcc_weights::d_w, [](const ovfcc_weights* p) { return p->layout.w_bytes; });
    if (!rc)
        rc = gather(&W->d_scale, L.scale_bytes, &ovfcc_weights::d_scale,
                    [](const ovfcc_weights* p) { return p->layout.scale_bytes; });
    if (!rc)
        rc = gather(&W->d_zp, L.zp_bytes, &ovfcc_weights::d_zp, [](const ovfcc_weights* p) { return p->layout.zp_bytes; });
    if (!rc && W->desc.bias_type != OVFCC_NONE)
        rc = gather(&W->d_bias, (size_t)n_total * 2, &ovfcc_weights::d_bias,
                    [](const ovfcc_weights* p) { return (size_t)p->desc.N * 2; });
    if (!rc)
        rc = finish_weights(W);
    if (rc) {
        ovfcc_weights_destroy(W);
        return rc;
    }
    *out = W;
    return OVFCC_OK;
}

int ovfcc_weights_glu(const ovfcc_weights* gate, const ovfcc_weights* up, int glu_type, ovfcc_weights** out) {
    if ((gate && gate->mlp_down) || (up && up->mlp_down))
        return fail(OVFCC_EINVAL, "an MLP node cannot be one half of a gated linear unit");
    if (!gate || !up || !out)
        return fail(OVFCC_EINVAL, "null argument");
    *out = nullptr;
    if (glu_type != OVFCC_GLU_SWISH && glu_type != OVFCC_GLU_GELU && glu_type != OVFCC_GLU_GELU_TANH)
        return fail(OVFCC_EINVAL, "unknown gated-linear-unit type");
    if (!gate->layout.tiled || !up->layout.tiled)
        return fail(OVFCC_EUNSUPPORTED, "only tiled nodes can be fused");
    if (gate->layout.glu || up->layout.glu)
        return fail(OVFCC_EUNSUPPORTED, "a node with a gated-linear-unit epilogue cannot be a part");
    ovfcc_fc_desc want = gate->desc;
    if (std::memcmp(&want, &up->desc, sizeof(want)) != 0 || gate->ctx != up->ctx ||
        gate->layout.zp_const != up->layout.zp_const)
        return fail(OVFCC_EUNSUPPORTED, "gate and up projection differ in shape, types, bias or output type");
    HIP_TRY(hipSetDevice(gate->ctx->device));
    ovfcc_weights* W = new ovfcc_weights();
    W->ctx = gate->ctx;
    W->desc = gate->desc;
    W->desc.N = 2 * gate->desc.N;
    W->desc.flags = glu_type;
    W->layout = ovfcc::make_layout(W->desc);
    W->layout.zp_const = gate->layout.zp_const;
    const ovfcc::Layout& L = W->layout;
    const size_t tiles = (size_t)gate->layout.n_tiles;
    // rows of one tile in each array; gate tiles land on even rows of the fused arrays, up tiles on odd rows
    auto weave = [&](void** dst, const void* g, const void* u, size_t row) -> int {
        if (!g || row == 0)
            return OVFCC_OK;
        HIP_TRY(hipMalloc(dst, 2 * tiles * row));
        W->bytes += 2 * tiles * row;
        HIP_TRY(hipMemcpy2D(*dst, 2 * row, g, row, row, tiles, hipMemcpyDeviceToDevice));
        HIP_TRY(hipMemcpy2D(static_cast<char*>(*dst) + row, 2 * row, u, row, row, tiles, hipMemcpyDeviceToDevice));
        return OVFCC_OK;
    };
    int rc = weave(&W->d_w, gate->d_w, up->d_w, gate->layout.w_bytes / tiles);
    if (!rc)
        rc = weave(&W->d_scale, gate->d_scale, up->d_scale, gate->layout.scale_bytes / tiles);
    if (!rc && L.zp_table)
        rc = weave(&W->d_zp, gate->d_zp, up->d_zp, gate->layout.zp_bytes / tiles);
    if (!rc && W->desc.bias_type != OVFCC_NONE)
        rc = weave(&W->d_bias, gate->d_bias, up->d_bias, (size_t)ovfcc::kTileRows * 2);
    if (!rc)
        rc = finish_weights(W);
    if (rc) {
        ovfcc_weights_destroy(W);
        return rc;
    }
    *out = W;
    return OVFCC_OK;
}

int64_t ovfcc_weights_device_bytes(const ovfcc_weights* w) {
    return w ? (int64_t)w->bytes + ovfcc_weights_device_bytes(w->mlp_down) : 0;
}

int ovfcc_weights_is_tiled(const ovfcc_weights* w) {
    return w && w->layout.tiled ? 1 : 0;
}

namespace {

// Blob of one node: header, then the device arrays in this order, each padded to 16 bytes.
struct BlobHeader {
    char magic[8];        // "OVFCCW\0\0"
    uint32_t version;     // layout version of blob and tiles
    uint32_t header_bytes;
    ovfcc_fc_desc desc;
    int32_t zp_const;
    int32_t tiled;        // kBlobTiled | kBlobHasDown
    uint64_t w_bytes, scale_bytes, zp_bytes, bias_bytes;
};
constexpr uint32_t kBlobVersion = 2;
constexpr int32_t kBlobTiled = 1, kBlobHasDown = 2;  // bits of BlobHeader::tiled; HasDown: another node's blob follows
const char kBlobMagic[8] = {'O', 'V', 'F', 'C', 'C', 'W', 0, 0};

size_t pad16(size_t n) {
    return (n + 15) & ~(size_t)15;
}

// sizes of the four device arrays of a node
void device_sizes(const ovfcc_fc_desc& d, const ovfcc::Layout& L, uint64_t out[4]) {
    const int64_t N = d.N, K = d.K, ng = L.groups;
    if (L.tiled) {
        out[0] = L.w_bytes, out[1] = L.scale_bytes, out[2] = L.zp_bytes;
    } else {
        out[0] = L.bits == 4 ? (uint64_t)(N * K + 1) / 2 : (uint64_t)N * K;
        out[1] = (uint64_t)N * ng * 2;
        out[2] = 0;
        if (d.zp_type != OVFCC_NONE) {
            const uint64_t cnt = d.zp_scalar ? 1 : (uint64_t)N * ng;
            out[2] = d.zp_type == OVFCC_U4 ? (cnt + 1) / 2 : cnt;
        }
    }
    out[3] = d.bias_type != OVFCC_NONE ? (uint64_t)N * 2 : 0;
}

}  // namespace

// one node's own part of a blob (an MLP node's blob is its first node's part followed by its down projection's)
static size_t own_blob_bytes(const ovfcc_weights* w) {
    uint64_t sz[4];
    device_sizes(w->desc, w->layout, sz);
    return pad16(sizeof(BlobHeader)) + pad16(sz[0]) + pad16(sz[1]) + pad16(sz[2]) + pad16(sz[3]);
}

int ovfcc_weights_export_size(const ovfcc_weights* w, size_t* bytes) {
    if (!w || !bytes)
        return fail(OVFCC_EINVAL, "null argument");
    *bytes = own_blob_bytes(w) + (w->mlp_down ? own_blob_bytes(w->mlp_down) : 0);
    return OVFCC_OK;
}

int ovfcc_weights_export(const ovfcc_weights* w, void* blob, size_t bytes) {
    size_t total = 0;
    int rc = ovfcc_weights_export_size(w, &total);
    if (rc)
        return rc;
    if (!blob || bytes < total)
        return fail(OVFCC_EINVAL, "blob buffer is null or too small");
    const size_t need = own_blob_bytes(w);
    if (w->mlp_down) {
        rc = ovfcc_weights_export(w->mlp_down, static_cast<char*>(blob) + need, bytes - need);
        if (rc)
            return rc;
    }
    HIP_TRY(hipSetDevice(w->ctx->device));
    uint64_t sz[4];
    device_sizes(w->desc, w->layout, sz);
    BlobHeader h{};
    std::memcpy(h.magic, kBlobMagic, 8);
    h.version = kBlobVersion;
    h.header_bytes = (uint32_t)sizeof(BlobHeader);
    h.desc = w->desc;
    h.zp_const = w->layout.zp_const;
    h.tiled = (w->layout.tiled ? kBlobTiled : 0) | (w->mlp_down ? kBlobHasDown : 0);
    h.w_bytes = sz[0], h.scale_bytes = sz[1], h.zp_bytes = sz[2], h.bias_bytes = sz[3];
    char* at = static_cast<char*>(blob);
    std::memset(at, 0, need);
    std::memcpy(at, &h, sizeof(h));
    at += pad16(sizeof(BlobHeader));
    const void* src[4] = {w->d_w, w->d_scale, w->d_zp, w->d_bias};
    for (int i = 0; i < 4; ++i) {
        if (sz[i] && src[i])
            HIP_TRY(hipMemcpy(at, src[i], sz[i], hipMemcpyDeviceToHost));
        at += pad16(sz[i]);
    }
    return OVFCC_OK;
}

int ovfcc_weights_import(ovfcc_ctx* ctx, const void* blob, size_t bytes, ovfcc_weights** out) {
    if (!ctx || !blob || !out)
        return fail(OVFCC_EINVAL, "null argument");
    *out = nullptr;
    if (bytes < pad16(sizeof(BlobHeader)))
        return fail(OVFCC_EINVAL, "blob is shorter than its header");
    BlobHeader h;
    std::memcpy(&h, blob, sizeof(h));
    if (std::memcmp(h.magic, kBlobMagic, 8) != 0 || h.version != kBlobVersion || h.header_bytes != sizeof(BlobHeader))
        return fail(OVFCC_EINVAL, "not a weight blob of this library version");
    int rc = ovfcc::validate_desc(&h.desc);
    if (rc)
        return rc;
    ovfcc::Layout L = ovfcc::make_layout(h.desc);
    uint64_t sz[4];
    device_sizes(h.desc, L, sz);
    // a scalar zero-point lives in zp_const; everything else must be exactly what the descriptor implies
    const int zp_lo = L.zp_offset, zp_hi = L.zp_offset + 255;
    const size_t need = pad16(sizeof(BlobHeader)) + pad16(sz[0]) + pad16(sz[1]) + pad16(sz[2]) + pad16(sz[3]);
    if ((h.tiled & ~(kBlobTiled | kBlobHasDown)) != 0 || ((h.tiled & kBlobTiled) != 0) != L.tiled || h.w_bytes != sz[0] || h.scale_bytes != sz[1] || h.zp_bytes != sz[2] ||
        h.bias_bytes != sz[3] || h.zp_const < zp_lo || h.zp_const > zp_hi ||
        bytes < need)
        return fail(OVFCC_EINVAL, "blob sizes do not match its descriptor");
    L.zp_const = h.zp_const;
    HIP_TRY(hipSetDevice(ctx->device));
    ovfcc_weights* W = new ovfcc_weights();
    W->ctx = ctx;
    W->desc = h.desc;
    W->layout = L;
    const char* at = static_cast<const char*>(blob) + pad16(sizeof(BlobHeader));
    void** dst[4] = {&W->d_w, &W->d_scale, &W->d_zp, &W->d_bias};
    for (int i = 0; i < 4 && !rc; ++i) {
        if (sz[i]) {
            hipError_t e = hipMalloc(dst[i], sz[i]);
            if (e == hipSuccess)
                e = hipMemcpy(*dst[i], at, sz[i], hipMemcpyHostToDevice);
            if (e != hipSuccess)
                rc = hip_fail(e, "weight blob upload");
            W->bytes += sz[i];
        }
        at += pad16(sz[i]);
    }
    if (!rc)
        rc = finish_weights(W);
    if (!rc && (h.tiled & kBlobHasDown)) {
        // an MLP node: the down projection's blob follows; the pair must fit as ovfcc_weights_mlp demands
        ovfcc_weights* down = nullptr;
        rc = ovfcc_weights_import(ctx, static_cast<const char*>(blob) + need, bytes - need, &down);
        if (!rc && (down->mlp_down || !W->layout.glu || down->layout.glu || W->desc.out_type != OVFCC_F16 ||
                    out_channels(W) != down->desc.K))
            rc = fail(OVFCC_EINVAL, "the two nodes of an MLP blob do not fit each other");
        if (rc)
            ovfcc_weights_destroy(down);
        else
            W->mlp_down = down;
    }
    if (rc) {
        ovfcc_weights_destroy(W);
        return rc;
    }
    *out = W;
    return OVFCC_OK;
}

int ovfcc_request_create(ovfcc_ctx* ctx, ovfcc_request** out) {
    if (!ctx || !out)
        return fail(OVFCC_EINVAL, "ctx or out is null");
    *out = nullptr;
    HIP_TRY(hipSetDevice(ctx->device));
    ovfcc_request* r = new ovfcc_request();
    r->ctx = ctx;
    hipError_t e = hipStreamCreateWithFlags(&r->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete r;
        return hip_fail(e, "hipStreamCreateWithFlags");
    }
    *out = r;
    return OVFCC_OK;
}

void ovfcc_request_destroy(ovfcc_request* r) {
    if (!r)
        return;
    if (r->stream) {
        (void)hipStreamSynchronize(r->stream);
        (void)hipStreamDestroy(r->stream);
    }
    if (r->d_x) (void)hipFree(r->d_x);
    if (r->d_y) (void)hipFree(r->d_y);
    if (r->workspace) (void)hipFree(r->workspace);
    if (r->counters) (void)hipFree(r->counters);
    if (r->d_gather) (void)hipFree(r->d_gather);
    if (r->d_quant) (void)hipFree(r->d_quant);
    if (r->d_mid) (void)hipFree(r->d_mid);
    if (r->d_sync) (void)hipFree(r->d_sync);
    if (r->h_error) (void)hipHostFree(r->h_error);
    if (r->h_maps) (void)hipHostFree(r->h_maps);
    if (r->h_stage) (void)hipHostFree(r->h_stage);
    if (r->maps_uploaded) (void)hipEventDestroy(r->maps_uploaded);
    delete r;
}

int ovfcc_request_force_kernel(ovfcc_request* r, int kernel, int split_k) {
    if (!r)
        return fail(OVFCC_EINVAL, "request is null");
    if (kernel < OVFCC_KERNEL_AUTO || kernel > OVFCC_KERNEL_PREFILL || split_k < 0)
        return fail(OVFCC_EINVAL, "unknown kernel or negative split");
    r->force_kernel = kernel;
    r->force_split = split_k;
    return OVFCC_OK;
}

int ovfcc_last_kernel_info(const ovfcc_request* r, ovfcc_kernel_info* info) {
    if (!r || !info)
        return fail(OVFCC_EINVAL, "null argument");
    *info = r->last;
    return OVFCC_OK;
}

int ovfcc_fc_run_device(ovfcc_request* r, const ovfcc_weights* w, const void* x_dev, void* y_dev, int64_t M) {
    if (!r || !w)
        return fail(OVFCC_EINVAL, "request or weights is null");
    if (M < 0)
        return fail(OVFCC_EINVAL, "M is negative");
    if (M > 0 && (!x_dev || !y_dev))
        return fail(OVFCC_EINVAL, "x or y is null");
    if (w->ctx != r->ctx)
        return fail(OVFCC_EINVAL, "weights and request belong to different contexts");
    if (M > ((int64_t)1 << 24))
        return fail(OVFCC_EUNSUPPORTED, "M is limited to 2^24");
    HIP_TRY(hipSetDevice(r->ctx->device));
    VerboseTimer timer(r, w, M);
    return enqueue(r, w, x_dev, y_dev, M);
}

int ovfcc_fc_run_device_static(ovfcc_request* r, const ovfcc_weights* w, const void* x_dev, void* y_dev, int64_t M) {
    if (!r || !w)
        return fail(OVFCC_EINVAL, "request or weights is null");
    if (M < 0)
        return fail(OVFCC_EINVAL, "M is negative");
    if (M > 0 && (!x_dev || !y_dev))
        return fail(OVFCC_EINVAL, "x or y is null");
    if (w->ctx != r->ctx)
        return fail(OVFCC_EINVAL, "weights and request belong to different contexts");
    if (M > ((int64_t)1 << 24))
        return fail(OVFCC_EUNSUPPORTED, "M is limited to 2^24");
    HIP_TRY(hipSetDevice(r->ctx->device));
    return enqueue(r, w, x_dev, y_dev, M, true);
}

int ovfcc_fc_run_grouped_device(ovfcc_request* r, const ovfcc_group_item* items, int n_items) {
    if (!r || (!items && n_items > 0) || n_items < 0)
        return fail(OVFCC_EINVAL, "bad grouped-run arguments");
    if (n_items == 0)
        return OVFCC_OK;
    HIP_TRY(hipSetDevice(r->ctx->device));
    const ovfcc_weights* w0 = items[0].weights;
    if (!w0)
        return fail(OVFCC_EINVAL, "an item has no weights");
    bool same = true;
    for (int i = 0; i < n_items && same; ++i) {
        const ovfcc_weights* w = items[i].weights;
        if (!w || w->ctx != r->ctx)
            return fail(OVFCC_EINVAL, "an item's weights are null or belong to another context");
        if (items[i].M < 0 || (items[i].M > 0 && (!items[i].x_dev || !items[i].y_dev)))
            return fail(OVFCC_EINVAL, "an item has a negative row count or a null buffer");
        // (a scalar zero-point lives in the layout, not in the descriptor, and the grouped kernels take one for all)
        same = std::memcmp(&w->desc, &w0->desc, sizeof(ovfcc_fc_desc)) == 0 &&
               (w->d_bias != nullptr) == (w0->d_bias != nullptr) && w->layout.zp_const == w0->layout.zp_const;
    }
    // one launch needs a common shape and format, the tiled layout and no forced kernel; otherwise item by item
    bool grouped = same && w0->layout.tiled && r->force_kernel == OVFCC_KERNEL_AUTO;
    int64_t rows_max = 0;
    for (int i = 0; i < n_items; ++i)
        rows_max = std::max<int64_t>(rows_max, items[i].M);
    if (rows_max == 0)
        return OVFCC_OK;
    // Few rows everywhere: the small-batch decode kernel; otherwise the prefill kernel, one tile of 64 or 128 rows
    // per slice, whichever makes the cheaper launch: a 64-row tile costs about 0.7 of a 128-row tile
    // (OVFCC_PREFILL_ROWS overrides).
    const bool decode = rows_max <= ovfcc::kDecodeMaxRows;
    int64_t rows_cap = ovfcc::kDecodeMaxRows;
    if (!decode) {
        std::vector<int64_t> rows(n_items);
        for (int i = 0; i < n_items; ++i)
            rows[i] = items[i].M;
        rows_cap = ovfcc::rows_cap_for(rows.data(), n_items, w0->layout.groups_per_kblock == 1);
    }
    ovfcc::FcDeviceArgs a;
    std::vector<ovfcc::BatchGroupItem> work;
    std::vector<const ovfcc_weights*> work_w;  // the node of every slice, for slices that end up running one by one
    if (grouped) {
        // cut every item into equal slices of at most rows_cap rows
        const size_t out_bytes = w0->desc.out_type == OVFCC_F32 ? 4 : 2;
        rows_max = 0;
        for (int i = 0; i < n_items; ++i) {
            const int64_t M = items[i].M;
            if (M == 0)
                continue;
            const int64_t slices = (M + rows_cap - 1) / rows_cap;
            const int64_t step = (M + slices - 1) / slices;
            const ovfcc_weights* w = items[i].weights;
            for (int64_t m0 = 0; m0 < M; m0 += step) {
                ovfcc::BatchGroupItem it{};
                it.w = w->d_w, it.scale = w->d_scale, it.zp = w->d_zp, it.bias = w->d_bias;
                it.x = static_cast<const char*>(items[i].x_dev) + (size_t)m0 * w->desc.K * 2;
                it.y = static_cast<char*>(items[i].y_dev) + (size_t)m0 * out_channels(w) * out_bytes;
                it.M = (int)std::min(M - m0, step);
                rows_max = std::max<int64_t>(rows_max, it.M);
                work.push_back(it);
                work_w.push_back(w);
            }
        }
    }
    for (size_t first = 0; grouped && first < work.size(); first += ovfcc::kMaxGroupItems) {
        const int n = (int)std::min<size_t>(ovfcc::kMaxGroupItems, work.size() - first);
        ovfcc::BatchGroupTable tab{};
        for (int i = 0; i < n; ++i)
            tab.item[i] = work[first + i];
        ovfcc::LaunchPlan p;
        int rc;
        if (decode) {
            // planned for one slice; the other slices fill the chip, so K is split only as far as LDS demands
            // unless the slices together still leave compute units idle
            fill_args(w0, work[0].x, work[0].y, rows_max, &a);
            int split = r->force_split;
            if (split <= 0) {
                const int64_t per_slice = (w0->layout.n_tiles + 7) / 8;
                const int kb = (int)w0->layout.k_blocks;
                split = 1;
                while (per_slice * n * split < r->ctx->n_cus && split < 8 && kb / (split * 2) >= 2)
                    split *= 2;
            }
            rc = ovfcc::plan_launch(a, OVFCC_KERNEL_DECODE, split, r->ctx->n_cus, &p);
            // (small nodes with few rows plan the streaming kernel; the grouped kernel has no gated-linear-unit form)
            grouped = !rc && p.batch && p.tiles_per_group == 1 && !w0->layout.glu;
        } else {
            // planned as one node whose row tiles are the slices: tile counts and split-K come out right
            fill_args(w0, work[0].x, work[0].y, (int64_t)n * rows_cap, &a);
            a.tile_rows = (int)rows_cap;
            rc = ovfcc::plan_launch(a, OVFCC_KERNEL_PREFILL, r->force_split, r->ctx->n_cus, &p);
            grouped = !rc && p.async_dma && p.tiles_y == n;
        }
        if (!grouped) {
            if (first == 0)
                break;
            // A later, smaller batch of slices for which no grouped kernel applies (a short tail of a long list):
            // its slices run one by one, with the same results.
            for (size_t j = first; j < work.size(); ++j) {
                rc = enqueue(r, work_w[j], work[j].x, work[j].y, work[j].M);
                if (rc)
                    return rc;
            }
            return OVFCC_OK;
        }
        ovfcc::LaunchPlan all = p;  // split-K buffers for n slices
        if (decode) {
            all.workspace_bytes = p.workspace_bytes * n;
            all.counter_count = p.counter_count * n;
        }
        rc = ensure_split_buffers(r, all);
        if (rc)
            return rc;
        a.workspace = r->workspace;
        a.counters = r->counters;
        const int e = decode ? ovfcc::launch_batch_grouped(tab, n, a, p, r->stream)
                             : ovfcc::launch_prefill_async_grouped(tab, n, a, p, r->stream);
        if (e)
            return hip_fail((hipError_t)e, "grouped kernel launch");
        ovfcc::LaunchPlan shown = p;
        if (decode)
            shown.grid[2] = (unsigned)n;
        shown.name = decode ? (w0->layout.bits == 4 ? "fcc_batch_grouped_w4" : "fcc_batch_grouped_w8")
                            : "fcc_prefill_async_grouped_w4";
        record(r, shown);
    }
    if (!grouped) {
        for (int i = 0; i < n_items; ++i) {
            int rc = enqueue(r, items[i].weights, items[i].x_dev, items[i].y_dev, items[i].M);
            if (rc)
                return rc;
        }
    }
    return OVFCC_OK;
}

namespace {
// argument checks shared by the two forms of the gather-matmul entry point; *same_zp: the experts' scalar
// zero-points agree (a grouped launch carries one)
int check_gather_matmul(ovfcc_request* r, const ovfcc_weights* const* experts, int n_experts, const void* a_dev,
                        int a_batches, const void* indices, int64_t M, int top_k, void* y_dev, bool* same_zp) {
    if (!r || !experts || n_experts <= 0 || !indices || M < 0 || top_k <= 0)
        return fail(OVFCC_EINVAL, "bad gather-matmul arguments");
    if (a_batches != 1 && a_batches != top_k)
        return fail(OVFCC_EINVAL, "A must have one batch or one batch per selected expert");
    if (top_k > n_experts)
        return fail(OVFCC_EINVAL, "more selected experts per row than experts");
    if (M > 0 && (!a_dev || !y_dev))
        return fail(OVFCC_EINVAL, "A or Y is null");
    if (M * top_k > ((int64_t)1 << 24))
        return fail(OVFCC_EUNSUPPORTED, "M * top_k is limited to 2^24");
    if (!experts[0])
        return fail(OVFCC_EINVAL, "an expert's weights are null or belong to another context");
    int rc = experts_agree(r, experts, n_experts, same_zp);
    if (rc)
        return rc;
    const ovfcc_weights* w0 = experts[0];
    const size_t out_bytes = w0->desc.out_type == OVFCC_F32 ? 4 : 2;
    if ((w0->desc.K * 2) % 16 != 0 || (out_channels(w0) * out_bytes) % 16 != 0)
        return fail(OVFCC_EUNSUPPORTED, "rows of A and Y must be multiples of 16 bytes");
    return OVFCC_OK;
}
}  // namespace

int ovfcc_gather_matmul_routed_device(ovfcc_request* r, const ovfcc_weights* const* experts, int n_experts,
                                      const void* a_dev, int a_batches, const int32_t* indices_dev, int64_t M, int top_k,
                                      void* y_dev) {
    bool same_zp = true, ran = false;
    int rc = check_gather_matmul(r, experts, n_experts, a_dev, a_batches, indices_dev, M, top_k, y_dev, &same_zp);
    if (rc || M == 0)
        return rc;
    HIP_TRY(hipSetDevice(r->ctx->device));
    if (same_zp)
        rc = gather_matmul_routed(r, experts, n_experts, a_dev, a_batches, indices_dev, nullptr, M, top_k, y_dev, &ran);
    if (rc)
        return rc;
    if (!ran)
        return fail(OVFCC_EUNSUPPORTED,
                    "routing on the device needs tiled 4-bit experts of one scalar zero-point that the grouped prefill "
                    "kernel runs (N % 256 == 0), at most 64 of them; pass the indices in host memory instead");
    return OVFCC_OK;
}

int ovfcc_gather_matmul_device(ovfcc_request* r, const ovfcc_weights* const* experts, int n_experts, const void* a_dev,
                               int a_batches, const int32_t* indices, int64_t M, int top_k, void* y_dev) {
    bool same_zp = true, ran = false;
    int rc = check_gather_matmul(r, experts, n_experts, a_dev, a_batches, indices, M, top_k, y_dev, &same_zp);
    if (rc || M == 0)
        return rc;
    const ovfcc_weights* w0 = experts[0];
    const int64_t K = w0->desc.K, N_out = out_channels(w0);
    const size_t out_bytes = w0->desc.out_type == OVFCC_F32 ? 4 : 2;
    HIP_TRY(hipSetDevice(r->ctx->device));
    // the routed form wherever it fits: the indices are copied to the device and bucketed there, and the call does
    // not depend on what the host threads were doing; otherwise the rows are bucketed here
    if (same_zp && ovfcc::env_int("OVFCC_MOE_HOST_ROUTING", 0) == 0) {
        rc = gather_matmul_routed(r, experts, n_experts, a_dev, a_batches, nullptr, indices, M, top_k, y_dev, &ran);
        if (rc || ran)
            return rc;
    }

    const int64_t R = M * top_k;
    std::vector<int> count, start;
    rc = bucket_rows(r, indices, M, top_k, n_experts, a_batches, false, &count, &start);
    if (rc)
        return rc;
    const size_t map_bytes = (size_t)2 * R * sizeof(int);

    // one scratch allocation: gathered rows | results | row maps
    const size_t x_bytes = (size_t)R * K * 2, y_bytes = (size_t)R * N_out * out_bytes;
    const size_t x_off = 0, y_off = (x_bytes + 255) & ~(size_t)255, m_off = (y_off + y_bytes + 255) & ~(size_t)255;
    if (m_off + map_bytes > r->gather_cap)
        HIP_TRY(hipStreamSynchronize(r->stream));
    rc = grow(&r->d_gather, &r->gather_cap, m_off + map_bytes);
    if (rc)
        return rc;
    char* base = static_cast<char*>(r->d_gather);
    int* d_maps = reinterpret_cast<int*>(base + m_off);
    HIP_TRY(hipMemcpyAsync(d_maps, r->h_maps, map_bytes, hipMemcpyHostToDevice, r->stream));
    HIP_TRY(hipEventRecord(r->maps_uploaded, r->stream));
    int e1 = ovfcc::launch_rows(base + x_off, a_dev, d_maps, nullptr, (int)R, (int)(K * 2), r->stream);
    if (e1)
        return hip_fail((hipError_t)e1, "row gather launch");
    std::vector<ovfcc_group_item> items;
    for (int e = 0; e < n_experts; ++e)
        if (count[e])
            items.push_back({experts[e], base + x_off + (size_t)start[e] * K * 2,
                             base + y_off + (size_t)start[e] * N_out * out_bytes, (int64_t)count[e]});
    rc = ovfcc_fc_run_grouped_device(r, items.data(), (int)items.size());
    if (rc)
        return rc;
    e1 = ovfcc::launch_rows(y_dev, base + y_off, nullptr, d_maps + R, (int)R, (int)(N_out * out_bytes), r->stream);
    if (e1)
        return hip_fail((hipError_t)e1, "row scatter launch");
    return OVFCC_OK;
}

int ovfcc_grouped_matmul_device(ovfcc_request* r, const ovfcc_weights* const* groups, int n_groups, const void* a_dev,
                                const int32_t* offsets, int64_t rows, void* y_dev) {
    if (!r || !groups || n_groups <= 0 || rows < 0)
        return fail(OVFCC_EINVAL, "bad grouped-matmul arguments");
    if (!groups[0])
        return fail(OVFCC_EINVAL, "a group's weights are null or belong to another context");
    bool same_zp = true;
    int rc = experts_agree(r, groups, n_groups, &same_zp);
    if (rc)
        return rc;
    const ovfcc_weights* w0 = groups[0];
    const int64_t K = w0->desc.K, N_out = out_channels(w0);
    const size_t out_bytes = w0->desc.out_type == OVFCC_F32 ? 4 : 2;
    if (offsets) {
        int64_t before = 0;
        for (int g = 0; g < n_groups; ++g) {
            if (offsets[g] < before || offsets[g] > rows)
                return fail(OVFCC_EINVAL, "offsets must not decrease and must not exceed the rows of A");
            before = offsets[g];
        }
    }
    if (rows == 0)
        return OVFCC_OK;
    if (!a_dev || !y_dev)
        return fail(OVFCC_EINVAL, "A or Y is null");
    if ((N_out * out_bytes) % 4 != 0)
        return fail(OVFCC_EUNSUPPORTED, "rows of Y must be multiples of 4 bytes");
    HIP_TRY(hipSetDevice(r->ctx->device));
    const char* a = static_cast<const char*>(a_dev);
    char* y = static_cast<char*>(y_dev);
    std::vector<ovfcc_group_item> items;
    items.reserve((size_t)n_groups);
    if (offsets) {
        int64_t start = 0;
        for (int g = 0; g < n_groups; ++g) {
            const int64_t end = offsets[g];
            if (end > start)
                items.push_back({groups[g], a + (size_t)start * K * 2, y + (size_t)start * N_out * out_bytes, end - start});
            start = end;
        }
        if (start < rows) {  // rows that belong to no group: zeros
            int e = ovfcc::launch_zero_u32(reinterpret_cast<unsigned*>(y + (size_t)start * N_out * out_bytes),
                                           (size_t)(rows - start) * N_out * out_bytes / 4, r->stream);
            if (e)
                return hip_fail((hipError_t)e, "zero fill launch");
        }
    } else {
        for (int g = 0; g < n_groups; ++g)
            items.push_back({groups[g], a + (size_t)g * rows * K * 2, y + (size_t)g * rows * N_out * out_bytes, rows});
    }
    return ovfcc_fc_run_grouped_device(r, items.data(), (int)items.size());
}

int ovfcc_grouped_matmul_offsets_device(ovfcc_request* r, const ovfcc_weights* const* groups, int n_groups,
                                        const void* a_dev, const int32_t* offsets_dev, int64_t rows, void* y_dev) {
    if (!r || !groups || n_groups <= 0 || rows < 0 || !offsets_dev)
        return fail(OVFCC_EINVAL, "bad grouped-matmul arguments");
    if (!groups[0])
        return fail(OVFCC_EINVAL, "a group's weights are null or belong to another context");
    bool same_zp = true;
    int rc = experts_agree(r, groups, n_groups, &same_zp);
    if (rc || rows == 0)
        return rc;
    if (!a_dev || !y_dev)
        return fail(OVFCC_EINVAL, "A or Y is null");
    const ovfcc_weights* w0 = groups[0];
    const int64_t K = w0->desc.K, N_out = out_channels(w0);
    const size_t out_bytes = w0->desc.out_type == OVFCC_F32 ? 4 : 2;
    HIP_TRY(hipSetDevice(r->ctx->device));
    RoutedLaunch L;
    if (!same_zp || (K * 2) % 16 != 0 || (N_out * out_bytes) % 16 != 0 || !plan_routed(r, w0, rows, n_groups, &L))
        return fail(OVFCC_EUNSUPPORTED,
                    "offsets in device memory need tiled 4-bit groups of one scalar zero-point that the grouped prefill "
                    "kernel runs (N % 256 == 0), at most 64 of them; pass the offsets in host memory instead");
    const size_t need = sizeof(ovfcc::RoutedHeader) + (size_t)L.n_slices * sizeof(ovfcc::BatchGroupItem) + 256;
    if (need > r->gather_cap)
        HIP_TRY(hipStreamSynchronize(r->stream));
    rc = grow(&r->d_gather, &r->gather_cap, need);
    if (rc)
        return rc;
    char* base = static_cast<char*>(r->d_gather);
    int* d_tail = reinterpret_cast<int*>(base);  // the header starts 256 bytes in
    auto* d_header = reinterpret_cast<ovfcc::RoutedHeader*>(base + 256);
    ovfcc::ExpertPointers ptrs{};
    for (int g = 0; g < n_groups; ++g)
        ptrs.w[g] = groups[g]->d_w, ptrs.scale[g] = groups[g]->d_scale, ptrs.zp[g] = groups[g]->d_zp,
        ptrs.bias[g] = groups[g]->d_bias;
    const int e = ovfcc::launch_offsets_table(offsets_dev, n_groups, rows, L.cap, ptrs, a_dev, (size_t)K * 2, y_dev,
                                              (size_t)N_out * out_bytes,
                                              reinterpret_cast<ovfcc::BatchGroupItem*>(d_header + 1), L.n_slices, d_header,
                                              d_tail, L.plan.tiles_x, (int)w0->layout.k_blocks, L.plan.n_cus, r->stream);
    if (e)
        return hip_fail((hipError_t)e, "offsets kernel launch");
    return launch_routed(r, L, d_header);
}

namespace {
int check_moe(ovfcc_request* r, const ovfcc_weights* const* gate_up, const ovfcc_weights* const* down, int n_experts,
              const void* x_dev, const void* routing_dev, const void* indices, int64_t M, int top_k, void* y_dev,
              bool* same_zp) {
    if (!r || !gate_up || !down || n_experts <= 0 || !indices || M < 0 || top_k <= 0)
        return fail(OVFCC_EINVAL, "bad mixture-of-experts arguments");
    if (top_k > n_experts)
        return fail(OVFCC_EINVAL, "more selected experts per row than experts");
    if (M > 0 && (!x_dev || !routing_dev || !y_dev))
        return fail(OVFCC_EINVAL, "hidden states, routing weights or output is null");
    if (M * top_k > ((int64_t)1 << 24))
        return fail(OVFCC_EUNSUPPORTED, "M * top_k is limited to 2^24");
    if (!gate_up[0] || !down[0])
        return fail(OVFCC_EINVAL, "an expert's weights are null or belong to another context");
    bool zg = true, zd = true;
    int rc = experts_agree(r, gate_up, n_experts, &zg);
    if (!rc)
        rc = experts_agree(r, down, n_experts, &zd);
    if (rc)
        return rc;
    *same_zp = zg && zd;
    const ovfcc_weights *g0 = gate_up[0], *d0 = down[0];
    // gate/up: [2 I, H] with a gated linear unit, f16 out (it feeds the down projection); down: [H, I], no unit
    const int64_t H = g0->desc.K, I = out_channels(g0);
    if (!g0->layout.glu || g0->desc.out_type != OVFCC_F16)
        return fail(OVFCC_EINVAL, "the gate/up nodes must carry a gated linear unit and write f16");
    if (d0->layout.glu || d0->desc.K != I || d0->desc.N != H)
        return fail(OVFCC_EINVAL, "the down nodes must map the gate/up output back to the hidden size, without a unit");
    if ((H * 2) % 16 != 0 || (I * 2) % 16 != 0)
        return fail(OVFCC_EUNSUPPORTED, "hidden and intermediate rows must be multiples of 16 bytes");
    return OVFCC_OK;
}
}  // namespace

int ovfcc_moe_routed_device(ovfcc_request* r, const ovfcc_weights* const* gate_up, const ovfcc_weights* const* down,
                            int n_experts, const void* x_dev, const void* routing_dev, const int32_t* indices_dev,
                            int64_t M, int top_k, void* y_dev) {
    bool same_zp = true, ran = false;
    int rc = check_moe(r, gate_up, down, n_experts, x_dev, routing_dev, indices_dev, M, top_k, y_dev, &same_zp);
    if (rc || M == 0)
        return rc;
    HIP_TRY(hipSetDevice(r->ctx->device));
    if (same_zp)
        rc = moe_routed(r, gate_up, down, n_experts, x_dev, routing_dev, indices_dev, nullptr, M, top_k, y_dev, &ran);
    if (rc)
        return rc;
    if (!ran)
        return fail(OVFCC_EUNSUPPORTED,
                    "routing on the device needs tiled 4-bit experts of one scalar zero-point that the grouped prefill "
                    "kernel runs (N % 256 == 0), at most 64 of them; pass the indices in host memory instead");
    return OVFCC_OK;
}

int ovfcc_moe_device(ovfcc_request* r, const ovfcc_weights* const* gate_up, const ovfcc_weights* const* down,
                     int n_experts, const void* x_dev, const void* routing_dev, const int32_t* indices, int64_t M,
                     int top_k, void* y_dev) {
    bool same_zp = true, ran = false;
    int rc = check_moe(r, gate_up, down, n_experts, x_dev, routing_dev, indices, M, top_k, y_dev, &same_zp);
    if (rc || M == 0)
        return rc;
    const ovfcc_weights *g0 = gate_up[0], *d0 = down[0];
    const int64_t H = g0->desc.K, I = out_channels(g0);
    const int d_f32 = d0->desc.out_type == OVFCC_F32 ? 1 : 0;
    HIP_TRY(hipSetDevice(r->ctx->device));
    if (same_zp && ovfcc::env_int("OVFCC_MOE_HOST_ROUTING", 0) == 0) {
        rc = moe_routed(r, gate_up, down, n_experts, x_dev, routing_dev, nullptr, indices, M, top_k, y_dev, &ran);
        if (rc || ran)
            return rc;
    }

    const int64_t R = M * top_k;
    std::vector<int> count, start;
    rc = bucket_rows(r, indices, M, top_k, n_experts, 1, true, &count, &start);
    if (rc)
        return rc;
    const size_t map_bytes = (size_t)2 * R * sizeof(int);

    // one scratch allocation: gathered rows | gate/up results | down results | row maps
    auto up256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t x_bytes = (size_t)R * H * 2, h_bytes = (size_t)R * I * 2, d_bytes = (size_t)R * H * (d_f32 ? 4 : 2);
    const size_t h_off = up256(x_bytes), d_off = up256(h_off + h_bytes), m_off = up256(d_off + d_bytes);
    if (m_off + map_bytes > r->gather_cap)
        HIP_TRY(hipStreamSynchronize(r->stream));
    rc = grow(&r->d_gather, &r->gather_cap, m_off + map_bytes);
    if (rc)
        return rc;
    char* base = static_cast<char*>(r->d_gather);
    int* d_maps = reinterpret_cast<int*>(base + m_off);
    HIP_TRY(hipMemcpyAsync(d_maps, r->h_maps, map_bytes, hipMemcpyHostToDevice, r->stream));
    HIP_TRY(hipEventRecord(r->maps_uploaded, r->stream));
    int e1 = ovfcc::launch_rows(base, x_dev, d_maps, nullptr, (int)R, (int)(H * 2), r->stream);
    if (e1)
        return hip_fail((hipError_t)e1, "row gather launch");
    std::vector<ovfcc_group_item> items;
    for (int e = 0; e < n_experts; ++e)
        if (count[e])
            items.push_back({gate_up[e], base + (size_t)start[e] * H * 2, base + h_off + (size_t)start[e] * I * 2,
                             (int64_t)count[e]});
    rc = ovfcc_fc_run_grouped_device(r, items.data(), (int)items.size());
    if (rc)
        return rc;
    items.clear();
    for (int e = 0; e < n_experts; ++e)
        if (count[e])
            items.push_back({down[e], base + h_off + (size_t)start[e] * I * 2,
                             base + d_off + (size_t)start[e] * H * (d_f32 ? 4 : 2), (int64_t)count[e]});
    rc = ovfcc_fc_run_grouped_device(r, items.data(), (int)items.size());
    if (rc)
        return rc;
    e1 = ovfcc::launch_moe_combine(y_dev, base + d_off, routing_dev, d_maps + R, (int)M, top_k, (int)H, d_f32, d_f32,
                                   r->stream);
    if (e1)
        return hip_fail((hipError_t)e1, "expert combine launch");
    return OVFCC_OK;
}

int ovfcc_request_sync(ovfcc_request* r) {
    if (!r)
        return fail(OVFCC_EINVAL, "request is null");
    HIP_TRY(hipStreamSynchronize(r->stream));
    if (r->h_error && *r->h_error) {
        // a one-launch MLP kernel gave up waiting for its workgroups: its output is not valid
        HIP_TRY(hipMemset(r->d_sync, 0, ovfcc::mlp_sync_bytes(r->ctx->n_cus)));
        *r->h_error = 0;
        return fail(OVFCC_EDEVICE, "an MLP launch on this request gave up waiting for its workgroups; its output is invalid");
    }
    return OVFCC_OK;
}

int ovfcc_fc_run(ovfcc_request* r, const ovfcc_weights* w, const void* x_host, void* y_host, int64_t M) {
    if (!r || !w)
        return fail(OVFCC_EINVAL, "request or weights is null");
    if (M < 0)
        return fail(OVFCC_EINVAL, "M is negative");
    if (M == 0)
        return OVFCC_OK;
    if (!x_host || !y_host)
        return fail(OVFCC_EINVAL, "x or y is null");
    HIP_TRY(hipSetDevice(r->ctx->device));
    const size_t xb = (size_t)M * w->desc.K * 2;
    const ovfcc_weights* last = output_node(w);
    const size_t yb = (size_t)M * out_channels(last) * (last->desc.out_type == OVFCC_F32 ? 4 : 2);
    if (xb > r->x_cap || yb > r->y_cap)
        HIP_TRY(hipStreamSynchronize(r->stream));
    int rc = grow(&r->d_x, &r->x_cap, xb);
    if (rc)
        return rc;
    rc = grow(&r->d_y, &r->y_cap, yb);
    if (rc)
        return rc;
    // Small transfers go through pinned memory of the request: a copy from or to pageable memory makes the runtime
    // stage, pin and synchronise per call, which at decode sizes costs more than the copy and the kernel together.
    // (The request is idle here: the previous call ended with a synchronisation.)  Large ones go directly.
    const size_t y_off = (xb + 255) & ~(size_t)255;
    const bool staged = y_off + yb <= kHostStageMax;
    if (staged && y_off + yb > r->h_stage_cap) {
        if (r->h_stage)
            HIP_TRY(hipHostFree(r->h_stage));
        r->h_stage = nullptr, r->h_stage_cap = 0;
        const size_t cap = std::max<size_t>(y_off + yb, 64 << 10);
        HIP_TRY(hipHostMalloc(&r->h_stage, cap, hipHostMallocDefault));
        r->h_stage_cap = cap;
    }
    char* hs = static_cast<char*>(r->h_stage);
    if (staged)
        std::memcpy(hs, x_host, xb);
    HIP_TRY(hipMemcpyAsync(r->d_x, staged ? hs : x_host, xb, hipMemcpyHostToDevice, r->stream));
    // ... and the kernel writes its (write-once) output straight into the pinned memory, which is mapped into the
    // device's address space: one copy operation less.  The activations are copied: every workgroup reads them.
    rc = ovfcc_fc_run_device(r, w, r->d_x, staged ? static_cast<void*>(hs + y_off) : r->d_y, M);
    if (rc)
        return rc;
    if (!staged)
        HIP_TRY(hipMemcpyAsync(y_host, r->d_y, yb, hipMemcpyDeviceToHost, r->stream));
    rc = ovfcc_request_sync(r);  // (also reports an MLP launch that gave up its wait)
    if (rc)
        return rc;
    if (staged)
        std::memcpy(y_host, hs + y_off, yb);
    return OVFCC_OK;
}

int ovfcc_device_malloc(ovfcc_ctx* ctx, size_t bytes, void** out) {
    if (!ctx || !out)
        return fail(OVFCC_EINVAL, "null argument");
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipMalloc(out, bytes ? bytes : 1));
    return OVFCC_OK;
}

int ovfcc_device_free(ovfcc_ctx* ctx, void* ptr) {
    if (!ctx)
        return fail(OVFCC_EINVAL, "null argument");
    if (ptr)
        HIP_TRY(hipFree(ptr));
    return OVFCC_OK;
}

int ovfcc_memcpy_h2d(ovfcc_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes) {
    if (!ctx || ((!dst_dev || !src_host) && bytes))
        return fail(OVFCC_EINVAL, "null argument");
    if (bytes)
        HIP_TRY(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
    return OVFCC_OK;
}

int ovfcc_memcpy_d2h(ovfcc_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes) {
    if (!ctx || ((!dst_host || !src_dev) && bytes))
        return fail(OVFCC_EINVAL, "null argument");
    if (bytes)
        HIP_TRY(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
    return OVFCC_OK;
}

int ovfcc_memcpy_d2d(ovfcc_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes) {
    if (!ctx || ((!dst_dev || !src_dev) && bytes))
        return fail(OVFCC_EINVAL, "null argument");
    if (bytes)
        HIP_TRY(hipMemcpy(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice));
    return OVFCC_OK;
}

}  // extern "C"
