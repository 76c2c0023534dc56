// Timing helpers of the benchmark driver (include/ovfcc_bench.h), built into their own library beside the product
// library: event-bracketed launches on a request's stream, the copy yardstick, launch-floor and matrix-core probes.
#include <hip/hip_runtime.h>

#include <string>
#include <vector>

#include "api_types.h"
#include "bench_probe.h"
#include "ovfcc_bench.h"
#include "ovfcc_internal.h"

namespace {

using ovfcc::fail;

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

// HIP objects of one benchmark call, released on every way out of it
struct Held {
    hipStream_t stream = nullptr;
    hipStream_t borrowed = nullptr;  // a stream of the caller's that may still run the graph: drained before the release
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    void* mem = nullptr;
    ~Held() {
        if (borrowed && (exec || graph)) (void)hipStreamSynchronize(borrowed);
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        if (mem) (void)hipFree(mem);
        if (stream) (void)hipStreamDestroy(stream);
    }
};

}  // namespace

extern "C" {

int ovfcc_bench_layers(ovfcc_request* r, const ovfcc_weights* const* layers, int n_layers, const void* x_dev,
                       void* y_dev, int64_t M, int warmup, int iters, int use_graph, float* elapsed_ms) {
    if (!r || !layers || n_layers <= 0 || !elapsed_ms || iters <= 0 || warmup < 0)
        return fail(OVFCC_EINVAL, "bad benchmark arguments");
    HIP_TRY(hipSetDevice(r->ctx->device));
    // one eager pass first: sizes the split-K buffers so that nothing allocates inside a capture
    for (int i = 0; i < n_layers; ++i) {
        int rc = ovfcc_fc_run_device(r, layers[i], x_dev, y_dev, M);
        if (rc)
            return rc;
    }
    HIP_TRY(hipStreamSynchronize(r->stream));

    Held h;  // graph, executable graph and events: released on every way out, error paths included
    h.borrowed = r->stream;
    if (use_graph) {
        HIP_TRY(hipStreamBeginCapture(r->stream, hipStreamCaptureModeThreadLocal));
        int rc = OVFCC_OK;
        for (int i = 0; i < n_layers && !rc; ++i)
            rc = ovfcc_fc_run_device(r, layers[i], x_dev, y_dev, M);
        // the capture is always ended, so that the stream leaves capture mode whatever a launch returned
        hipError_t e = hipStreamEndCapture(r->stream, &h.graph);
        if (rc)
            return rc;
        if (e != hipSuccess)
            return hip_fail(e, "hipStreamEndCapture");
        HIP_TRY(hipGraphInstantiate(&h.exec, h.graph, nullptr, nullptr, 0));
    }
    auto one_pass = [&]() -> int {
        if (use_graph) {
            HIP_TRY(hipGraphLaunch(h.exec, r->stream));
            return OVFCC_OK;
        }
        for (int i = 0; i < n_layers; ++i) {
            int rc = ovfcc_fc_run_device(r, layers[i], x_dev, y_dev, M);
            if (rc)
                return rc;
        }
        return OVFCC_OK;
    };
    for (int i = 0; i < warmup; ++i) {
        int rc = one_pass();
        if (rc)
            return rc;
    }
    HIP_TRY(hipEventCreate(&h.t0));
    HIP_TRY(hipEventCreate(&h.t1));
    HIP_TRY(hipStreamSynchronize(r->stream));
    HIP_TRY(hipEventRecord(h.t0, r->stream));
    int rc = OVFCC_OK;
    for (int i = 0; i < iters && !rc; ++i)
        rc = one_pass();
    HIP_TRY(hipEventRecord(h.t1, r->stream));
    HIP_TRY(hipEventSynchronize(h.t1));
    HIP_TRY(hipEventElapsedTime(elapsed_ms, h.t0, h.t1));
    return rc;
}

int ovfcc_bench_grouped(ovfcc_request* r, const ovfcc_group_item* items, int n_items, int warmup, int iters,
                        float* elapsed_ms) {
    if (!r || !items || n_items <= 0 || !elapsed_ms || iters <= 0 || warmup < 0)
        return fail(OVFCC_EINVAL, "bad benchmark arguments");
    HIP_TRY(hipSetDevice(r->ctx->device));
    int rc = OVFCC_OK;
    for (int i = 0; i < warmup + 1 && !rc; ++i)
        rc = ovfcc_fc_run_grouped_device(r, items, n_items);
    if (rc)
        return rc;
    Held h;
    HIP_TRY(hipEventCreate(&h.t0));
    HIP_TRY(hipEventCreate(&h.t1));
    HIP_TRY(hipStreamSynchronize(r->stream));
    HIP_TRY(hipEventRecord(h.t0, r->stream));
    for (int i = 0; i < iters && !rc; ++i)
        rc = ovfcc_fc_run_grouped_device(r, items, n_items);
    HIP_TRY(hipEventRecord(h.t1, r->stream));
    HIP_TRY(hipEventSynchronize(h.t1));
    HIP_TRY(hipEventElapsedTime(elapsed_ms, h.t0, h.t1));
    return rc;
}

int ovfcc_bench_copy(ovfcc_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes, int iters, float* elapsed_ms) {
    if (!ctx || !dst_dev || !src_dev || !elapsed_ms || iters <= 0 || bytes % 16)
        return fail(OVFCC_EINVAL, "bad copy benchmark arguments");
    HIP_TRY(hipSetDevice(ctx->device));
    Held h;
    HIP_TRY(hipStreamCreateWithFlags(&h.stream, hipStreamNonBlocking));
    HIP_TRY(hipEventCreate(&h.t0));
    HIP_TRY(hipEventCreate(&h.t1));
    int e = ovfcc::launch_copy(dst_dev, src_dev, bytes, h.stream);  // warm-up
    HIP_TRY(hipStreamSynchronize(h.stream));
    HIP_TRY(hipEventRecord(h.t0, h.stream));
    for (int i = 0; i < iters && !e; ++i)
        e = ovfcc::launch_copy(dst_dev, src_dev, bytes, h.stream);
    HIP_TRY(hipEventRecord(h.t1, h.stream));
    HIP_TRY(hipEventSynchronize(h.t1));
    HIP_TRY(hipEventElapsedTime(elapsed_ms, h.t0, h.t1));
    if (e)
        return hip_fail((hipError_t)e, "copy kernel launch");
    return OVFCC_OK;
}

int ovfcc_bench_mfma(ovfcc_ctx* ctx, int waves, int valu, int shape, int rounds, float* elapsed_ms, double* flops) {
    if (!ctx || !elapsed_ms || !flops || rounds <= 0 || (waves != 4 && waves != 8) || valu < 0 || valu > 4 ||
        shape < 0 || shape > 4 || (shape >= 2 && valu != 0))
        return fail(OVFCC_EINVAL, "bad matrix-core benchmark arguments");
    HIP_TRY(hipSetDevice(ctx->device));
    Held h;
    HIP_TRY(hipStreamCreateWithFlags(&h.stream, hipStreamNonBlocking));
    const int workgroups = ctx->n_cus;
    HIP_TRY(hipMalloc(&h.mem, (size_t)workgroups * 64 * waves * sizeof(float)));
    float* sink = static_cast<float*>(h.mem);
    HIP_TRY(hipEventCreate(&h.t0));
    HIP_TRY(hipEventCreate(&h.t1));
    int e = ovfcc::launch_mfma_probe(sink, workgroups, waves, valu, shape, 16, h.stream);  // warm-up
    HIP_TRY(hipStreamSynchronize(h.stream));
    HIP_TRY(hipEventRecord(h.t0, h.stream));
    if (!e)
        e = ovfcc::launch_mfma_probe(sink, workgroups, waves, valu, shape, rounds, h.stream);
    HIP_TRY(hipEventRecord(h.t1, h.stream));
    HIP_TRY(hipEventSynchronize(h.t1));
    HIP_TRY(hipEventElapsedTime(elapsed_ms, h.t0, h.t1));
    if (e)
        return hip_fail((hipError_t)e, "matrix-core probe launch");
    *flops = 2.0 * 16 * 16 * 32 * 8.0 * rounds * waves * workgroups;  // either shape: 2^17 multiply-adds per round
    return OVFCC_OK;
}

int ovfcc_bench_issue(ovfcc_ctx* ctx, int workgroups, int waves, int mode, int valu, int rounds, double* cycles_per_mfma,
                      double* ns_per_mfma) {
    if (!ctx || !cycles_per_mfma || !ns_per_mfma || rounds <= 0 || workgroups < 1 || workgroups > 4096 ||
        (waves != 4 && waves != 8))
        return fail(OVFCC_EINVAL, "bad issue benchmark arguments");
    HIP_TRY(hipSetDevice(ctx->device));
    Held h;
    HIP_TRY(hipStreamCreateWithFlags(&h.stream, hipStreamNonBlocking));
    const size_t sink_bytes = (size_t)workgroups * 64 * waves * sizeof(float);
    HIP_TRY(hipMalloc(&h.mem, sink_bytes + (size_t)workgroups * 2 * sizeof(long long)));
    float* sink = static_cast<float*>(h.mem);
    long long* ticks = reinterpret_cast<long long*>(static_cast<char*>(h.mem) + sink_bytes);
    int e = ovfcc::launch_issue_probe(sink, ticks, workgroups, waves, mode, valu, 64, h.stream);  // warm-up
    if (!e)
        e = ovfcc::launch_issue_probe(sink, ticks, workgroups, waves, mode, valu, rounds, h.stream);
    if (e)
        return hip_fail((hipError_t)e, "issue probe launch (mode and vector instruction count must be a built pair)");
    HIP_TRY(hipStreamSynchronize(h.stream));
    std::vector<long long> host((size_t)workgroups * 2);
    HIP_TRY(hipMemcpy(host.data(), ticks, host.size() * sizeof(long long), hipMemcpyDeviceToHost));
    double shader = 0.0, wall = 0.0;
    for (int g = 0; g < workgroups; ++g)
        shader += (double)host[2 * (size_t)g], wall += (double)host[2 * (size_t)g + 1];
    const double mfmas_per_simd = 8.0 * rounds * (waves / 4);
    *cycles_per_mfma = shader / workgroups / mfmas_per_simd;
    *ns_per_mfma = wall / workgroups * 10.0 / mfmas_per_simd;  // the wall clock counts at 100 MHz
    return OVFCC_OK;
}

// One graph of n_nodes probe launches, replayed `iters` times after three warm-up replays.
int ovfcc_bench_floor(ovfcc_ctx* ctx, const void* arena_dev, size_t arena_bytes, size_t node_bytes, int n_nodes, int waves,
                      int kib_per_wave, int iters, float* elapsed_ms) {
    if (!ctx || !elapsed_ms || n_nodes <= 0 || iters <= 0 || (node_bytes && (!arena_dev || arena_bytes < node_bytes)))
        return fail(OVFCC_EINVAL, "bad floor benchmark arguments");
    HIP_TRY(hipSetDevice(ctx->device));
    Held h;
    HIP_TRY(hipStreamCreateWithFlags(&h.stream, hipStreamNonBlocking));
    HIP_TRY(hipMalloc(&h.mem, 256));
    unsigned* out = static_cast<unsigned*>(h.mem);
    int e = 0;
    HIP_TRY(hipStreamBeginCapture(h.stream, hipStreamCaptureModeThreadLocal));
    const size_t slices = node_bytes ? arena_bytes / node_bytes : 1;
    for (int i = 0; i < n_nodes && !e; ++i)
        e = node_bytes ? ovfcc::launch_stream_probe(static_cast<const char*>(arena_dev) + (size_t)(i % slices) * node_bytes,
                                                    node_bytes, waves, kib_per_wave, out, h.stream)
                       : ovfcc::launch_empty(out, h.stream);
    hipError_t ce = hipStreamEndCapture(h.stream, &h.graph);
    if (e || ce != hipSuccess)
        return e ? hip_fail((hipError_t)e, "probe launch") : hip_fail(ce, "graph capture");
    HIP_TRY(hipGraphInstantiate(&h.exec, h.graph, nullptr, nullptr, 0));
    HIP_TRY(hipEventCreate(&h.t0));
    HIP_TRY(hipEventCreate(&h.t1));
    for (int i = 0; i < 3; ++i)
        HIP_TRY(hipGraphLaunch(h.exec, h.stream));
    HIP_TRY(hipStreamSynchronize(h.stream));
    HIP_TRY(hipEventRecord(h.t0, h.stream));
    for (int i = 0; i < iters; ++i)
        HIP_TRY(hipGraphLaunch(h.exec, h.stream));
    HIP_TRY(hipEventRecord(h.t1, h.stream));
    HIP_TRY(hipEventSynchronize(h.t1));
    HIP_TRY(hipEventElapsedTime(elapsed_ms, h.t0, h.t1));
    return OVFCC_OK;
}

}  // extern "C"
