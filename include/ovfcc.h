/*
 * ovfcc -- MI355X (gfx950) implementation of OpenVINO's weight-compressed FullyConnected,
 * ov::op::internal::FullyConnectedCompressed, behind a plain C ABI.
 *
 *   Y[m,n] = sum_k X[m,k] * ((W[n,k] - ZP[n,k/G]) * S[n,k/G]) (+ bias[n])
 *
 * All entry points return OVFCC_OK (0) or a negative OVFCC_E* code; the reason is kept in a
 * thread-local string readable with ovfcc_last_error().  No exceptions, no C++ or HIP types.
 * Host pointers hold OpenVINO's constant layout: weights row-major [N,K] (MatMul with
 * transpose_b = true), 4-bit types two per byte with the even element in the low nibble.
 *
 * Each declaration names the piece of the OpenVINO source tree it stands in for
 * (paths relative to the OpenVINO repository root).
 */
#ifndef OVFCC_H
#define OVFCC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OVFCC_OK 0
#define OVFCC_EINVAL (-1)       /* bad argument (null pointer, shape, type tag) */
#define OVFCC_EUNSUPPORTED (-2) /* valid OpenVINO configuration this library does not run */
#define OVFCC_EDEVICE (-3)      /* HIP runtime error (no device, launch failure, ...) */
#define OVFCC_ENOMEM (-4)       /* host or device allocation failed */

/* element type tags; the subset of ov::element::Type_t this path uses
 * (src/core/include/openvino/core/type/element_type.hpp) */
enum ovfcc_type {
    OVFCC_NONE = 0,
    OVFCC_U4 = 1,
    OVFCC_I4 = 2,
    OVFCC_U8 = 3,
    OVFCC_I8 = 4,
    OVFCC_F16 = 5,
    OVFCC_F32 = 6
};

/* One FullyConnectedCompressed node: the five inputs X, W, bias, weight_scales,
 * weight_zero_points of src/common/transformations/include/ov_ops/fully_connected_compressed.hpp:15-37
 * after ConvertFullyConnectedToFullyConnectedCompressed has re-viewed the constants as
 * W [N,K], S/ZP [N,K/G] (src/common/transformations/src/transformations/op_conversions/
 * convert_fc_to_compressed.cpp:42-78).  An absent input (the reference's
 * Constant(dynamic, Shape{0})) is type OVFCC_NONE with a null pointer. */
typedef struct ovfcc_fc_desc {
    int64_t N;          /* output channels (OC) */
    int64_t K;          /* input channels (IC) */
    int64_t group_size; /* G along K; K for per-output-channel scale/zp */
    int32_t w_type;     /* OVFCC_U4 | OVFCC_I4 | OVFCC_U8 | OVFCC_I8 */
    int32_t scale_type; /* OVFCC_F16 */
    int32_t zp_type;    /* OVFCC_NONE | OVFCC_U4 | OVFCC_U8 */
    int32_t zp_scalar;  /* non-zero: zp holds one element (Shape{} / Shape{1}) used for every (n, group) */
    int32_t bias_type;  /* OVFCC_NONE | OVFCC_F16, [N] */
    int32_t act_type;   /* OVFCC_F16 */
    int32_t out_type;   /* OVFCC_F16 | OVFCC_F32 (FullyConnected's output_type; default = activation type) */
    int32_t flags;      /* 0, or OVFCC_GLU_* [| OVFCC_GLU_GATE_SECOND] | OVFCC_DYNQUANT_I8 [| OVFCC_DYNQUANT_PER_GROUP | OVFCC_DYNQUANT_ASYM] | OVFCC_W_INPUT_MAJOR */
} ovfcc_fc_desc;

/* Gated linear unit fused into the node (flags).  The reference fuses ov::op::internal::GLU
 * (src/common/transformations/include/ov_ops/glu.hpp:16-40: axis = -1, split_lengths = N/2, glu_type,
 * split_to_glu_idx) into the FullyConnected that produces its input when gate and up projection were fused
 * horizontally (src/plugins/intel_gpu/src/kernel_selector/kernels/fully_connected/
 * fully_connected_kernel_bf_tiled.cpp:223-236,661-666; epilogue cl_kernels/fully_connected_gpu_bf_tiled.cl:764-780;
 * stand-alone formula cl_kernels/swiglu_gpu_ref.cl:66-85).  With Y = X W^T (+ bias) of shape [M, N], L = N / 2:
 *     out[m, f] = act(Y[m, g + f]) * Y[m, u + f],  f in [0, L)
 * where (g, u) = (0, L), or (L, 0) with OVFCC_GLU_GATE_SECOND (split_to_glu_idx = 1), and act is
 * Swish x / (1 + exp(-x)), Gelu x (1 + erf(x / sqrt 2)) / 2 or Gelu_Tanh
 * x (1 + tanh(sqrt(2 / pi) x (1 + 0.044715 x^2))) / 2, evaluated in f32 on the f32 sums.  The node's output is
 * [M, L] in out_type; N, W, scales, zero-points and bias keep their [N, ...] shapes.  N must be even; the fast
 * (tiled) kernels also need N % 32 == 0. */
#define OVFCC_GLU_NONE 0
#define OVFCC_GLU_SWISH 1
#define OVFCC_GLU_GELU 2
#define OVFCC_GLU_GELU_TANH 3
#define OVFCC_GLU_TYPE_MASK 3
#define OVFCC_GLU_GATE_SECOND 4

/* Dynamic quantisation of the activations (flags), the counterpart of ov::hint::dynamic_quantization_group_size
 * with per-token groups: the reference's plugins quantise FullyConnected activations to int8 on the fly
 * (ov::op::internal::DynamicQuantize, src/common/transformations/include/ov_ops/dynamic_quantize.hpp:16-60; Intel
 * GPU: cl_kernels/dynamic_quantize_gpu_ref.cl:100-250 and the integer path of
 * cl_kernels/fully_connected_gpu_bf_tiled.cl:1257-1291, for batches above a threshold only).  The flag is a
 * permission, not a request for a specific kernel: it takes effect for 8-bit weights with one scale per output
 * channel, N % 256 == 0, K % 128 == 0 and more than 48 rows (a gated linear unit, if any, is applied to the
 * results as usual); every other call of the node
 * computes in f16 as without the flag.  Where it takes effect,
 *     q[m, k] = rte(half(x[m, k] * half(127 / max(0.003, max_k |x[m, k]|)))),
 *     y[m, n] = (sum_k q[m, k] W[n, k] - ZP[n] sum_k q[m, k]) * (S[n] * half(1 / scale_m)) + bias[n],
 * integers exact, which differs from the f16 result by the quantisation noise (about 1e-2 relative; the
 * reference tests such nodes with absolute tolerances of 0.1-0.2). */
#define OVFCC_DYNQUANT_I8 8

/* With OVFCC_DYNQUANT_I8, for 4-bit weights with one scale (and zero-point) per group of 128 inputs (W4A8): the
 * reference quantises the source of such a node too -- the CPU plugin in groups of
 * ov::hint::dynamic_quantization_group_size inputs (src/plugins/intel_cpu/src/nodes/executors/dnnl/
 * dnnl_fullyconnected_primitive.cpp:161-241,284-298), the GPU plugin per token on matrix-engine hardware and per
 * group elsewhere (src/plugins/intel_gpu/src/plugin/transformations/dynamic_quantize_fully_connected.cpp:24-140,
 * src/plugins/intel_gpu/src/runtime/execution_config.cpp:348-354).  OVFCC_DYNQUANT_I8 alone quantises per token;
 * with OVFCC_DYNQUANT_PER_GROUP every group of 128 inputs of a row has its own scale (group size = the weights'
 * group).  Takes effect for u4 / i4 weights, G = 128, zero-points none, scalar or a u4 table, N % 256 == 0 and more
 * than 48 rows:
 *     y[m, n] = sum_g ( sum_{k in g} q[m, k] (W[n, k] - ZP[n, g]) ) * S[n, g] * inv_scale[m (, g)]  + bias[n],
 * q and inv_scale as above over a row or a group, the integer sums exact, the sum over groups in f32. */
#define OVFCC_DYNQUANT_PER_GROUP 32

/* With OVFCC_DYNQUANT_I8, per token only: the reference's asymmetric form of the same quantisation -- unsigned 8-bit
 * activations with a zero-point per token (ov::op::internal::DynamicQuantize with QuantizationType::Asymmetric,
 * quantization_dt = zp_dt = u8: src/common/transformations/include/ov_ops/dynamic_quantize.hpp:16-60, chosen by
 * src/plugins/intel_gpu/src/plugin/transformations/dynamic_quantize_fully_connected.cpp:109-117; arithmetic of
 * cl_kernels/dynamic_quantize_gpu_ref.cl:100-250 with ASYMMETRIC_QUANTIZATION and UNSIGNED_OUTPUT; consumed as the
 * source zero-point of the matrix product, src/plugins/intel_gpu/src/graph/impls/onednn/fully_connected_onednn.cpp:
 * 83-88,325-329).  Takes effect where OVFCC_DYNQUANT_I8 does for 8-bit weights with one scale per channel, and
 * K <= 32768 (the sums below must fit 32 bits; a longer K keeps the symmetric form):
 *     d = max_k x - min_k x in half (0.003 if the two are equal), scale = half(255 / d), zp = half(-min * (255 / d)),
 *     q[m, k] = sat_u8(rte(half(x[m, k] * scale) + zp)),  za[m] = sat_u8(rte(zp)),
 *     y[m, n] = sum_k (q[m, k] - za[m]) (W[n, k] - ZP[n]) * (S[n] * half(1 / scale)) + bias[n],
 * integers exact.  The conversions saturate where the reference's are undefined (a row whose values all lie on one
 * side of zero has a zero-point outside 0..255; such a row is shifted by the clamped zero-point, as it would be on
 * hardware whose conversion saturates). */
#define OVFCC_DYNQUANT_ASYM 64

/* Input-major constants (flags): W is given as [K, N] (grouped: [K/G, G, N]) and scales / zero-points as
 * [K/G, N], each packed over its own flattened index -- the form in which a MatMul with transpose_b = false holds
 * its weights.  The reference brings such a node to [N, K] by a constant-folded Transpose that
 * ConvertMatMulToFC inserts (src/plugins/intel_cpu/src/transformations/cpu_opset/common/pass/
 * convert_matmul_to_fc.cpp:47-270) and ConvertFullyConnectedToFullyConnectedCompressed replays on scales and
 * zero-points (convert_fc_to_compressed.cpp:170-225); here ovfcc_weights_create (and ovfcc_repack_host) do that
 * transposition once on the host.  The node that results is the [N, K] node: ovfcc_weights_export never carries
 * the flag.  A scalar zero-point and the bias [N] are not affected. */
#define OVFCC_W_INPUT_MAJOR 16

typedef struct ovfcc_ctx ovfcc_ctx;         /* one device + its kernels */
typedef struct ovfcc_weights ovfcc_weights; /* repacked, device-resident W/S/ZP/bias of one node */
typedef struct ovfcc_request ovfcc_request; /* one HIP stream + staging + split-K workspace */

/* kernel families, as reported by ovfcc_last_kernel_info and accepted by ovfcc_request_force_kernel */
enum ovfcc_kernel {
    OVFCC_KERNEL_AUTO = 0,
    OVFCC_KERNEL_PLAIN = 1,  /* any shape, OpenVINO layout, one wave per output channel */
    OVFCC_KERNEL_DECODE = 2, /* M <= 48: the streaming and the small-batch kernel over the tiled layout */
    OVFCC_KERNEL_PREFILL = 3 /* more rows: MFMA tile kernels over the tiled layout (N % 128 == 0) */
};

typedef struct ovfcc_kernel_info {
    int32_t kernel;     /* enum ovfcc_kernel actually launched */
    int32_t grid[3];
    int32_t block;
    int32_t split_k;
    int32_t tile_m, tile_n;
    char name[64];
} ovfcc_kernel_info;

/* ---- life cycle ---------------------------------------------------------------------------- */

/* Plugin creation for one device: stands in for the device-side part of
 * ov::IPlugin construction (src/inference/dev_api/openvino/runtime/iplugin.hpp:74-255;
 * template: src/plugins/template/src/plugin.cpp:36-60).  Fails with OVFCC_EDEVICE when no
 * gfx950 device is visible. */
int ovfcc_init(int device, ovfcc_ctx** out);
void ovfcc_destroy(ovfcc_ctx* ctx);

/* Number of visible HIP devices (0 on a host without a GPU); never fails. */
int ovfcc_device_count(void);

/* Compile-time weight preparation: what DnnlFCPrimitive::createShapeAgnosticData +
 * utils::prepareWeightsMemory do once per node on the CPU plugin
 * (src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_fullyconnected_primitive.cpp:421-484,
 * src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_utils.cpp:49-122) and
 * reorder_weights_int4.cl does on the Intel GPU plugin.  Validates the descriptor with this
 * library's analogue of FullyConnected::isSupportedCompressedOperation
 * (src/plugins/intel_cpu/src/nodes/fullyconnected.cpp:143-218), repacks on the host into
 * wave64 tiles and uploads.  Host buffers may be released on return. */
int ovfcc_weights_create(ovfcc_ctx* ctx, const ovfcc_fc_desc* desc, const void* w, const void* scales,
                         const void* zp, const void* bias, ovfcc_weights** out);
void ovfcc_weights_destroy(ovfcc_weights* w);
/* A second device copy of an existing node (same bytes at distinct addresses, no host work):
 * what sharing one compressed constant between several FullyConnected nodes needs when each node
 * must own its buffer (shared weights: src/tests/functional/plugin/shared/src/subgraph/
 * shared_matmul_weights_decompression.cpp); the benchmark uses it to build a rotating weight set. */
int ovfcc_weights_clone(const ovfcc_weights* src, ovfcc_weights** out);
/* Horizontal fusion of FullyConnected nodes that read the same activations (Q/K/V, gate/up): one node whose
 * output channels are the parts' channels in order, N = sum N_i, so that one launch serves them all and the
 * caller splits Y [M, N] by columns.  What FullyConnectedHorizontalFusion does on the Intel GPU plugin
 * (src/plugins/intel_gpu/src/plugin/transformations/fc_horizontal_fusion.cpp: Concat of weights, scales and
 * zero-points along the output-channel axis, VariadicSplit of the result).  Parts must be tiled nodes with
 * equal K, group size, weight type, zero-point kind, bias presence and output type; the copy is made on the
 * device and the parts stay valid. */
int ovfcc_weights_concat(const ovfcc_weights* const* parts, int n_parts, ovfcc_weights** out);
/* Gate and up projection of a gated linear unit as one node: out[m, f] = act(gate(x)[m, f]) * up(x)[m, f]
 * (see OVFCC_GLU_*; gate first).  The device-side counterpart of creating the node from concatenated constants
 * with desc.flags = glu_type: both parts must be tiled nodes equal in shape, types, bias presence and output type;
 * they stay valid.  The result reports N = 2 * N_part and produces [M, N_part]. */
int ovfcc_weights_glu(const ovfcc_weights* gate, const ovfcc_weights* up, int glu_type, ovfcc_weights** out);

/* The gated MLP of a decoder block as one node: gate / up projection with its gated linear unit (a node created
 * with OVFCC_GLU_* flags or by ovfcc_weights_glu, f16 output), then the down projection, whose K is the first
 * node's output width.  The counterpart of the CPU plugin's LLMMLP node (src/plugins/intel_cpu/src/nodes/llm_mlp.cpp:
 * 495-526; the pattern: cpu_opset/x64/pass/mlp_fusion.cpp:48-120).  ovfcc_fc_run[_device] on it takes X [M, K of
 * the first node] and writes Y [M, N of the down projection] in the down projection's output_type; the
 * intermediate activations live in a buffer of the request, rounded to f16 as between two separate nodes.  The
 * node runs as two launches on the request's stream.  With OVFCC_MLP_FUSED=1 in the environment, one to four rows
 * of 4-bit nodes with groups of 128 run as one kernel launch whose workgroups wait for each other in the middle (a
 * bounded wait: if it runs out, ovfcc_request_sync / ovfcc_fc_run return OVFCC_EDEVICE); it gives the same bits and,
 * as measured, is the slower of the two.  The new node owns copies of both; the arguments stay the caller's. */
int ovfcc_weights_mlp(const ovfcc_weights* gate_up, const ovfcc_weights* down, ovfcc_weights** out);
/* device bytes held by the repacked node */
int64_t ovfcc_weights_device_bytes(const ovfcc_weights* w);
/* 1 when the node uses the tiled layout (fast kernels), 0 for the OpenVINO-layout fallback */
int ovfcc_weights_is_tiled(const ovfcc_weights* w);

/* The node in its device form as one relocatable host blob, and back: what ICompiledModel::export_model /
 * IPlugin::import_model (src/inference/dev_api/openvino/runtime/icompiled_model.hpp:105, iplugin.hpp:173-208; the
 * template plugin's pair: src/plugins/template/src/compiled_model.cpp:173-192, plugin.cpp:230-311) store per node so
 * that a cached model skips the repack (ov::cache_dir, src/inference/src/dev/core_impl.cpp:858-897).
 * ovfcc_weights_export_size gives the blob's size; ovfcc_weights_export fills a host buffer of at least that size;
 * ovfcc_weights_import rebuilds the node on ctx's device.  A blob is valid for this library version only: import
 * checks magic, version, descriptor and every size against what the descriptor implies and fails with
 * OVFCC_EINVAL otherwise. */
int ovfcc_weights_export_size(const ovfcc_weights* w, size_t* bytes);
int ovfcc_weights_export(const ovfcc_weights* w, void* blob, size_t bytes);
int ovfcc_weights_import(ovfcc_ctx* ctx, const void* blob, size_t bytes, ovfcc_weights** out);

/* One infer request: ov::ISyncInferRequest
 * (src/inference/dev_api/openvino/runtime/isync_infer_request.hpp:30-175).  Different requests
 * may run concurrently from different threads; one request is used by one thread at a time. */
int ovfcc_request_create(ovfcc_ctx* ctx, ovfcc_request** out);
void ovfcc_request_destroy(ovfcc_request* req);

/* ---- execution ----------------------------------------------------------------------------- */

/* ISyncInferRequest::infer for one node with host tensors: copies X [M,K] f16 to the device,
 * runs the kernel, copies Y [M,N] (out_type) back and waits.  The CPU plugin's equivalent is
 * FullyConnected::execute -> DnnlFCPrimitive::execute
 * (src/plugins/intel_cpu/src/nodes/fullyconnected.cpp:427-433,
 * .../dnnl_fullyconnected_primitive.cpp:518-520).  M may be 0. */
int ovfcc_fc_run(ovfcc_request* req, const ovfcc_weights* w, const void* x_host, void* y_host, int64_t M);

/* Same with device-resident X and Y (a remote tensor in OpenVINO terms,
 * src/inference/dev_api/openvino/runtime/iremote_tensor.hpp): enqueues on the request's
 * stream and returns without waiting. */
int ovfcc_fc_run_device(ovfcc_request* req, const ovfcc_weights* w, const void* x_dev, void* y_dev, int64_t M);

/* ovfcc_fc_run_device for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the OpenVINO sources.  Same arguments, same
 * kernels and bit-identical results, but the call allocates nothing: launches that split K take their partial
 * tiles and arrival counters from a fixed scratch array in device memory (32 MiB of partial tiles, 16384
 * counters, held by every GPU the library runs on until the process ends) instead of buffers of the request,
 * and clear the counters they use with a small fill kernel first.  A launch that needs more than the array holds,
 * and a node whose activations would be quantised to int8 (OVFCC_DYNQUANT_I8 taking effect), is
 * OVFCC_EUNSUPPORTED.  All requests of a GPU share that GPU's array.  The library orders the launches that use it:
 * each waits, on its own stream, for an event recorded behind the one before it (the event is created by
 * ovfcc_init, not here), so calls from different requests and host threads are safe and simply do not overlap.  The
 * exception is a stream under graph capture, which cannot wait for an event from outside its capture: replays of
 * graphs that hold such launches, and anything else that uses the array at the same time, are the caller's to keep
 * apart. */
int ovfcc_fc_run_device_static(ovfcc_request* req, const ovfcc_weights* w, const void* x_dev, void* y_dev, int64_t M);

/* Several independent nodes of one shape and weight format in one launch: the experts of a
 * mixture-of-experts layer, each with its own gathered rows.  Stands in for the grouped forms of the op,
 * ov::op::internal::GatherMatmulCompressed (src/common/transformations/include/ov_ops/
 * gather_matmul_compressed.hpp:17-33; shape contract src/common/transformations/src/ov_ops/gather_matmul.cpp:38-110:
 * B = [n_experts, N, K], one row set per expert) and GroupedMatMulCompressed
 * (include/ov_ops/grouped_matmul_compressed.hpp), with the gather already done by the caller: item i multiplies its
 * M_i rows x_dev [M_i, K] with its own weights into y_dev [M_i, N].  Device pointers, no copies, enqueued on the
 * request's stream.  Items with M = 0 are skipped; items that differ in shape or format, untiled nodes and small
 * nodes with few rows run one by one, with the same results. */
typedef struct ovfcc_group_item {
    const ovfcc_weights* weights;
    const void* x_dev;
    void* y_dev;
    int64_t M;
} ovfcc_group_item;
int ovfcc_fc_run_grouped_device(ovfcc_request* req, const ovfcc_group_item* items, int n_items);

/* GroupedMatMulCompressed (src/common/transformations/include/ov_ops/grouped_matmul_compressed.hpp:17-66, the
 * compressed form of ov::op::v17::GroupedMatMul, src/core/include/openvino/op/grouped_matmul.hpp:26-50; arithmetic
 * src/core/reference/include/openvino/reference/grouped_matmul.hpp:36-88): groups[g] is group g's node (B[g] of the
 * op's [G, N, K] constant, all of one shape and format).
 *   2-D x 3-D form (offsets != NULL): a_dev is A [rows, K] f16, offsets [n_groups] int32 in host memory are the
 *   cumulative row ends -- group g multiplies rows [offsets[g-1], offsets[g]) (offsets[-1] = 0; a group may be
 *   empty) -- and y_dev receives [rows, N_out]; rows from offsets[n_groups-1] on come out as zeros, as in the
 *   reference.  Offsets that decrease or exceed `rows` are OVFCC_EINVAL.
 *   3-D x 3-D form (offsets == NULL): a_dev is A [n_groups, rows, K], y_dev receives [n_groups, rows, N_out].
 * One grouped launch (ovfcc_fc_run_grouped_device) on the request's stream; no copies, no waiting. */
int ovfcc_grouped_matmul_device(ovfcc_request* req, const ovfcc_weights* const* groups, int n_groups, const void* a_dev,
                                const int32_t* offsets, int64_t rows, void* y_dev);

/* The 2-D x 3-D form with the offsets in device memory, where the kernel that sorted the rows by group leaves them:
 * the slices of the grouped launch are cut by a kernel on the request's stream and the call never waits for it.
 * Needs tiled 4-bit groups of one scalar zero-point that the grouped prefill kernel runs (N % 256 == 0), at most 64
 * of them; otherwise OVFCC_EUNSUPPORTED (pass the offsets in host memory).  The host cannot check what it does not
 * read: an offset below its predecessor or above `rows` is taken as that bound (the group loses rows, nothing is
 * read or written outside A and Y). */
int ovfcc_grouped_matmul_offsets_device(ovfcc_request* req, const ovfcc_weights* const* groups, int n_groups,
                                        const void* a_dev, const int32_t* offsets_dev, int64_t rows, void* y_dev);

/* GatherMatmulCompressed (src/common/transformations/include/ov_ops/gather_matmul.hpp:17-41,
 * gather_matmul_compressed.hpp:17-33; shapes src/common/transformations/src/ov_ops/gather_matmul.cpp:38-130; CPU
 * executor src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_gathermatmul_executor.cpp:470-600): the expert
 * matrices of a mixture-of-experts layer applied to routed rows.  experts[e] is expert e's node (B[e] of the op's
 * [n_experts, N, K] constant, all of one shape and format); a_dev is A [a_batches, M, K] f16 in device memory with
 * a_batches = 1 (every selected expert reads the same row) or top_k; indices [M, top_k] int32 in host memory names
 * the experts of each row; y_dev receives [top_k, M, N_out]:
 *     Y[i, m, :] = experts[indices[m, i]](A[a_batches == 1 ? 0 : i, m, :]).
 * Rows are gathered per expert on the device, all experts run as one grouped launch
 * (ovfcc_fc_run_grouped_device) and the results are scattered back; everything is enqueued on the request's
 * stream.  An index outside [0, n_experts) is OVFCC_EINVAL. */
int ovfcc_gather_matmul_device(ovfcc_request* req, const ovfcc_weights* const* experts, int n_experts,
                               const void* a_dev, int a_batches, const int32_t* indices, int64_t M, int top_k,
                               void* y_dev);

/* The same with the indices in device memory, where a router's TopK leaves them: the (row, selection) pairs are
 * bucketed per expert by a kernel on the request's stream (one workgroup per expert; the reference's GPU plugin builds
 * its expert masks on the device as well, src/plugins/intel_gpu/src/graph/impls/ocl_v2/moe_mask_gen.cl), the grouped
 * launch reads its slice table from device memory, and the call neither waits for the stream nor depends on the row
 * counts.  Indices in device memory cannot be checked without waiting for them, so where the host-index form
 * returns OVFCC_EINVAL this one goes on: an index outside [0, n_experts) selects nothing and its row Y[i, m, :] is
 * written as zeros; every other row is what it would be without that pair.  Needs tiled 4-bit
 * experts with N % 256 == 0 and one scalar zero-point (what the grouped prefill kernel runs) and at most 64 experts;
 * otherwise OVFCC_EUNSUPPORTED.  ovfcc_gather_matmul_device takes this path itself wherever it fits, after copying
 * its indices to the device (OVFCC_MOE_HOST_ROUTING=1 in the environment keeps the bucketing on the host). */
int ovfcc_gather_matmul_routed_device(ovfcc_request* req, const ovfcc_weights* const* experts, int n_experts,
                                      const void* a_dev, int a_batches, const int32_t* indices_dev, int64_t M, int top_k,
                                      void* y_dev);

/* The expert block of a mixture-of-experts layer as one call: ov::op::internal::MOECompressed with
 * Expert_type::GEMM3_SWIGLU (src/common/transformations/include/ov_ops/moe_compressed.hpp:15-75,
 * src/core/dev_api/openvino/op/moe.hpp:17-45), the node that MoE op fusion folds three GatherMatmulCompressed, the
 * gate activation, the Multiply by the routing weights and the ReduceSum over the selected experts into
 * (src/common/transformations/src/transformations/common_optimizations/moe_op_fusion.cpp:55-105):
 *     y[m, :] = sum_{j < top_k} routing[m, j] * down_e( act(gate_e(x[m, :])) * up_e(x[m, :]) ),  e = indices[m, j].
 * gate_up[e] is expert e's gate and up projection as one node with a gated linear unit (W [2 I, H] created with
 * OVFCC_GLU_*, or ovfcc_weights_glu of the op's w0 and w1 slices; f16 output), down[e] its down projection
 * (w2: [H, I]); the experts agree in shape and format.  x_dev is [M, H] f16 and routing_dev [M, top_k] f16 in device
 * memory, indices [M, top_k] int32 in host memory; y_dev receives [M, H] in the down nodes' output type.  Rows are
 * bucketed per expert as in ovfcc_gather_matmul_device, every projection runs as one grouped launch over all
 * experts, the intermediate activations stay f16 in device memory, and the weighted sum over a row's experts is
 * taken in f32 in the order j = 0, 1, ....  Everything is enqueued on the request's stream. */
int ovfcc_moe_device(ovfcc_request* req, const ovfcc_weights* const* gate_up, const ovfcc_weights* const* down,
                     int n_experts, const void* x_dev, const void* routing_dev, const int32_t* indices_host, int64_t M,
                     int top_k, void* y_dev);

/* ovfcc_moe_device with indices_dev [M, top_k] int32 in device memory (see ovfcc_gather_matmul_routed_device): the
 * routing kernel runs once per projection, nothing in the call waits for the stream.  Where ovfcc_moe_device returns
 * OVFCC_EINVAL for an index outside [0, n_experts), this form cannot look: such a pair contributes nothing to its
 * row's sum (a row whose pairs all name no expert is written as zeros), every other row is unaffected. */
int ovfcc_moe_routed_device(ovfcc_request* req, const ovfcc_weights* const* gate_up, const ovfcc_weights* const* down,
                            int n_experts, const void* x_dev, const void* routing_dev, const int32_t* indices_dev,
                            int64_t M, int top_k, void* y_dev);

/* Wait for everything enqueued on the request (IAsyncInferRequest::wait). */
int ovfcc_request_sync(ovfcc_request* req);

/* Kernel choice override for tests and profiling (enum ovfcc_kernel; AUTO restores the policy),
 * and split-K override (0 = heuristic). */
int ovfcc_request_force_kernel(ovfcc_request* req, int kernel, int split_k);

/* What the last ovfcc_fc_run* on this request launched: the data behind
 * ICompiledModel::get_runtime_model's primitiveType / IInferRequest::get_profiling_info
 * (src/inference/dev_api/openvino/runtime/exec_model_info.hpp:31-73). */
int ovfcc_last_kernel_info(const ovfcc_request* req, ovfcc_kernel_info* info);

/* ---- device memory helpers (plain pointers; for hosts that do not link HIP themselves) ------ */
int ovfcc_device_malloc(ovfcc_ctx* ctx, size_t bytes, void** out);
/* Free and total memory of the context's device in bytes: the figures behind ov::intel_gpu::device_total_mem_size
 * and ov::intel_gpu::memory_statistics (src/inference/include/openvino/runtime/intel_gpu/properties.hpp:33, :64). */
int ovfcc_device_mem_info(ovfcc_ctx* ctx, size_t* free_bytes, size_t* total_bytes);
int ovfcc_device_free(ovfcc_ctx* ctx, void* ptr);
int ovfcc_memcpy_h2d(ovfcc_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes);
int ovfcc_memcpy_d2h(ovfcc_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes);
int ovfcc_memcpy_d2d(ovfcc_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes);

/* The OVFCC_* variables of the process environment (tuning overrides for experiments, and OVFCC_VERBOSE = 1: one
 * line per launch and per created node on stderr -- kernel, grid, tile, split-K; layout, bytes, repack and upload
 * time; = 2: every ovfcc_fc_run_device call is also timed with events and waited for, and its time, GB/s and
 * TFLOP/s are printed; the counterpart of OV_CPU_VERBOSE / the oneDNN verbose mode) are read once, at the first
 * ovfcc_init.  A process that changes them afterwards calls this to have them read again; launch plans cached
 * under the old values are dropped. */
void ovfcc_env_reload(void);

/* ---- host-only pieces (no device needed) ----------------------------------------------------- */

/* Validation alone: OVFCC_OK, OVFCC_EINVAL or OVFCC_EUNSUPPORTED, as ovfcc_weights_create would. */
int ovfcc_desc_validate(const ovfcc_fc_desc* desc);

/* Sizes of the tiled layout for a descriptor; all zero when the descriptor falls back to the
 * OpenVINO layout.  w_bytes: 1 KiB tiles of 16 channels x 128 (4-bit) or 64 (8-bit) inputs;
 * scale_bytes: f16 [N/16][groups][16]; zp_bytes: u8 [N/16][groups][16] (0 without zero-points).
 * With 4-bit weights and groups of 32 or 64 inputs both tables are [N/16][K/128][16][128/group_size]. */
int ovfcc_tiled_sizes(const ovfcc_fc_desc* desc, size_t* w_bytes, size_t* scale_bytes, size_t* zp_bytes);

/* The repacker itself, host to host (what ovfcc_weights_create uploads), and its inverse, which
 * restores OpenVINO's layout bit for bit.  i4 weights are stored as u4 = i4 xor 8 with the
 * zero-point raised by 8 (the transformation the CPU plugin applies for its unsigned kernels,
 * src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_utils.cpp:70-97); i8 likewise xor 0x80. */
int ovfcc_repack_host(const ovfcc_fc_desc* desc, const void* w, const void* scales, const void* zp,
                      void* w_tiled, void* scale_tiled, void* zp_tiled);
int ovfcc_unrepack_host(const ovfcc_fc_desc* desc, const void* w_tiled, const void* scale_tiled,
                        const void* zp_tiled, void* w, void* scales, void* zp);

/* 4-bit element access in OpenVINO order
 * (src/core/dev_api/openvino/core/type/element_iterator.hpp:76,161-176,248-259). */
int ovfcc_unpack_u4(const void* src, size_t n, uint8_t* dst);
int ovfcc_unpack_i4(const void* src, size_t n, int8_t* dst);

/* Last error text of the calling thread ("" when none). */
const char* ovfcc_last_error(void);
const char* ovfcc_version(void);

#ifdef __cplusplus
}
#endif
#endif /* OVFCC_H */
