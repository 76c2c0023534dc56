// The objects behind the C ABI's opaque handles.  Private to the library and to the benchmark library that is
// built from the same tree (it brackets launches with events on a request's own stream).
#pragma once

#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

#include "ovfcc.h"
#include "ovfcc_internal.h"

struct ovfcc_ctx {
    int device = 0;
    int n_cus = 256;
    std::string arch;
    // Launches whose workgroups wait for each other (the one-launch MLP) must not share the chip with another of
    // their kind: each waits, on its stream, for the event recorded behind the one before it.
    std::mutex coop_mu;
    hipEvent_t coop_done = nullptr;
};

struct ovfcc_weights {
    ovfcc_ctx* ctx = nullptr;
    ovfcc_fc_desc desc{};
    ovfcc::Layout layout;
    void* d_w = nullptr;
    void* d_scale = nullptr;
    void* d_zp = nullptr;
    void* d_bias = nullptr;
    ovfcc_weights* mlp_down = nullptr;  // ovfcc_weights_mlp: this node is gate / up, that one (owned) the down projection
    void* d_scale_cm = nullptr;  // channel-major copies of the group parameters for the matrix-vector kernel
    void* d_zp_cm = nullptr;
    int* d_colsum = nullptr;     // 8-bit per-channel node with OVFCC_DYNQUANT_ASYM: sum_k (w - zp) per channel, tiled order
    size_t bytes = 0;
    // Launch plans of recent calls, keyed by what a plan depends on besides the node itself.  Shared by every
    // request that runs the node, hence the lock; eight entries, replaced in turn.
    struct PlanEntry {
        int64_t M = -1;
        int force_kernel = 0, force_split = 0, n_cus = 0;
        unsigned env_generation = 0;
        ovfcc::LaunchPlan plan;
    };
    mutable std::mutex plan_mu;
    mutable PlanEntry plans[8];
    mutable unsigned plan_next = 0;
};

struct ovfcc_request {
    ovfcc_ctx* ctx = nullptr;
    hipStream_t stream = nullptr;
    void* d_x = nullptr;
    void* d_y = nullptr;
    size_t x_cap = 0, y_cap = 0;
    void* h_stage = nullptr;   // pinned host memory that small host transfers of ovfcc_fc_run go through: x | y
    size_t h_stage_cap = 0;
    float* workspace = nullptr;
    size_t ws_cap = 0;
    unsigned* counters = nullptr;
    size_t counter_cap = 0;
    void* d_gather = nullptr;  // gather-matmul: gathered rows, results before the scatter, row maps
    size_t gather_cap = 0;
    void* d_quant = nullptr;   // dynamic quantisation: int8 activations, inverse scales, sums
    size_t quant_cap = 0;
    void* d_mid = nullptr;     // MLP node: the intermediate row block [M, I] f16
    size_t mid_cap = 0;
    unsigned* d_sync = nullptr;   // ... the two counters of its one-launch kernel (zero between launches)
    unsigned* h_error = nullptr;  // ... and the pinned word that kernel sets when its wait ran out
    int* h_maps = nullptr;     // ... and the pinned host copy of the row maps, reused once its upload has finished
    size_t h_maps_cap = 0;
    hipEvent_t maps_uploaded = nullptr;
    int force_kernel = OVFCC_KERNEL_AUTO;
    int force_split = 0;
    ovfcc_kernel_info last{};
};
