/*
 * ovfcc_graph -- the graph-side half of the weight-compressed FullyConnected path, free of OpenVINO types.
 *
 * A host (the ov::IPlugin shim, a test) describes the relevant part of a model as an array of plain nodes;
 * the functions here decide what OpenVINO's transformation passes decide on the real graph and return
 * descriptors for ovfcc_weights_create / ovfcc_weights_concat / ovfcc_weights_glu:
 *
 *   ovfcc_fold_match   MatMul (or internal FullyConnected) over a weight-decompression subgraph
 *                      -> one FullyConnectedCompressed node: the roles of pattern::op::CompressedWeightsBlock
 *                      (src/common/transformations/src/transformations/pattern_blocks/compressed_weights_block.cpp:31-84),
 *                      ConvertMatMulToFC (src/plugins/intel_cpu/src/transformations/cpu_opset/common/pass/
 *                      convert_matmul_to_fc.cpp:47-270), ConvertFullyConnectedToFullyConnectedCompressed with its
 *                      combine_groups shape algebra (src/common/transformations/src/transformations/op_conversions/
 *                      convert_fc_to_compressed.cpp:32-225) and FullyConnectedBiasFusion
 *                      (src/plugins/intel_cpu/src/transformations/cpu_opset/common/pass/fc_bias_fusion.cpp:32-93).
 *   ovfcc_fold_model   all such nodes of a model, plus which of them share a launch: horizontal fusion of
 *                      siblings that read the same activations (src/plugins/intel_gpu/src/plugin/transformations/
 *                      fc_horizontal_fusion.cpp:30-140) and the gated linear unit act(gate(x)) * up(x)
 *                      (src/common/transformations/include/ov_ops/glu.hpp:16-40; kernel-side fusion
 *                      src/plugins/intel_gpu/src/kernel_selector/kernels/fully_connected/
 *                      fully_connected_kernel_bf_tiled.cpp:223-236).
 *
 * The matchers touch neither constant data nor a device: shapes, element types and small integer attributes in,
 * decisions out.  Return codes and ovfcc_last_error() as in ovfcc.h; "this subgraph is not a compressed
 * FullyConnected" is OVFCC_EUNSUPPORTED with the reason in the error string.
 *
 *   ovfcc_fold_weights_create / ovfcc_fold_expert_weights_create
 *                      the data half of the same passes: from a matched node and the bytes of its Constants to an
 *                      ovfcc_weights, so that a host's compile step is a loop over library calls.
 */
#ifndef OVFCC_GRAPH_H
#define OVFCC_GRAPH_H

#include "ovfcc.h"

#ifdef __cplusplus
extern "C" {
#endif

/* operations the matchers look at (openvino/op/*.hpp, ov_ops/fully_connected.hpp); everything else is OTHER */
enum ovfcc_op {
    OVFCC_OP_OTHER = 0,
    OVFCC_OP_PARAMETER = 1,
    OVFCC_OP_CONSTANT = 2,
    OVFCC_OP_CONVERT = 3,
    OVFCC_OP_SUBTRACT = 4,
    OVFCC_OP_MULTIPLY = 5,
    OVFCC_OP_RESHAPE = 6,
    OVFCC_OP_TRANSPOSE = 7,
    OVFCC_OP_MATMUL = 8,          /* v0::MatMul: inputs (A, B), attributes transpose_a / transpose_b */
    OVFCC_OP_FULLY_CONNECTED = 9, /* internal::FullyConnected: inputs (A, W [N, K], bias or -1) */
    OVFCC_OP_ADD = 10,
    OVFCC_OP_SWISH = 11,          /* v4::Swish with beta = 1 (one input) */
    OVFCC_OP_GELU = 12,           /* v7::Gelu; attr = 0 erf, 1 tanh */
    OVFCC_OP_RESULT = 13,
    OVFCC_OP_GATHER_MATMUL = 14,            /* internal::GatherMatmul: inputs (A, B, indices, bias) */
    OVFCC_OP_GATHER_MATMUL_COMPRESSED = 15, /* internal::GatherMatmulCompressed: (A, B, indices, bias, scale, zp) */
    OVFCC_OP_UNSQUEEZE = 16,
    OVFCC_OP_SLICE = 17,
    OVFCC_OP_REDUCE_SUM = 18,               /* v1::ReduceSum; attr = keep_dims */
    OVFCC_OP_GROUPED_MATMUL = 19,           /* v17::GroupedMatMul: inputs (A, B) or (A, B, offsets) */
    OVFCC_OP_GROUPED_MATMUL_COMPRESSED = 20 /* internal::GroupedMatMulCompressed: (A, B, [offsets,] scale[, zp]) */
};

/* element types beyond enum ovfcc_type that a graph may carry (bf16, i32 shape constants, ...) */
#define OVFCC_TYPE_OTHER 7
#define OVFCC_MAX_RANK 6
#define OVFCC_MAX_INPUTS 6

/* One node, described by its first output. */
typedef struct ovfcc_gnode {
    int32_t op;                    /* enum ovfcc_op */
    int32_t type;                  /* enum ovfcc_type or OVFCC_TYPE_OTHER */
    int32_t rank;                  /* rank of the output shape, -1 when dynamic */
    int64_t dims[OVFCC_MAX_RANK];  /* -1 = dynamic dimension */
    int32_t n_inputs;
    int32_t inputs[OVFCC_MAX_INPUTS]; /* indices into the node array; -1 = absent (FullyConnected without bias) */
    int32_t transpose_a, transpose_b; /* MatMul */
    int32_t attr;                  /* Gelu: 1 = tanh approximation; ReduceSum: keep_dims */
    int32_t consumers;             /* how many node inputs read this output */
    int32_t n_ints;                /* integer Constant of at most OVFCC_MAX_RANK elements: its values (a Transpose */
    int64_t ints[OVFCC_MAX_RANK];  /* order, a Reshape pattern); n_ints = -1 when not supplied */
} ovfcc_gnode;

/* A matched FullyConnectedCompressed node. */
typedef struct ovfcc_fold {
    ovfcc_fc_desc desc;       /* for ovfcc_weights_create; flags carry OVFCC_W_INPUT_MAJOR where the constants are [K, N] */
    int32_t root;             /* node whose output the fused node produces: the MatMul / FullyConnected, or the bias Add */
    int32_t matmul;           /* the MatMul / FullyConnected itself */
    int32_t activations;      /* producer of X */
    int32_t weights, scales, zero_points, bias; /* Constant nodes; -1 = absent */
    int32_t scale_broadcast;  /* the scale Constant holds one value for the whole node: replicate it N * K/G times */
    int32_t zp_from_real;     /* the zero-point Constant is f16 / f32: its values must be integers in 0..255 and become u8 */
    int32_t activations_f32;  /* X is f32: the host converts to f16 */
    /* The constants re-viewed without touching bytes (combine_groups): W as [N, K] (input-major: [K, N]), scales
     * and zero-point table as [N, K/G] (input-major: [K/G, N]); all zero for an absent or one-element constant. */
    int64_t w_view[2], scale_view[2], zp_view[2];
    int32_t n_chain;          /* nodes between the weights Constant and the root that the fused node absorbs */
    int32_t chain[16];
} ovfcc_fold;

/* Matches the subgraph that ends in `root` (a MatMul, a FullyConnected, or an Add of one of them with a Constant). */
int ovfcc_fold_match(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_fold* out);

/* Creates the node a fold describes from the bytes of its Constants -- what
 * ConvertFullyConnectedToFullyConnectedCompressed does with the Constants it re-views and converts
 * (src/common/transformations/src/transformations/op_conversions/convert_fc_to_compressed.cpp:127-225).
 * constant_data has n_nodes entries; entry i points at the data of node i in OpenVINO's packing (4-bit types two per
 * byte, low nibble first) where node i is one of fold->weights / scales / zero_points / bias, and is not read
 * otherwise (null is fine).  Weights and integer zero-points are taken as they are; f32 scales and bias are rounded
 * to f16 (nearest even), a scale Constant of one element is replicated (scale_broadcast), a real-typed zero-point
 * (zp_from_real) must hold integers in 0..255 and becomes u8 -- OVFCC_EUNSUPPORTED otherwise.  Every Constant's
 * element type and count are checked against the fold's descriptor (OVFCC_EINVAL).  extra_flags is or-ed into
 * desc.flags (OVFCC_W_DYN_QUANT, ...). */
int ovfcc_fold_weights_create(ovfcc_ctx* ctx, const ovfcc_gnode* nodes, int n_nodes, const ovfcc_fold* fold,
                              const void* const* constant_data, int extra_flags, ovfcc_weights** out);

/* How matched nodes share launches. */
enum ovfcc_fused_kind {
    OVFCC_FUSED_SINGLE = 0, /* one node of its own */
    OVFCC_FUSED_CONCAT = 1, /* siblings reading the same activations, concatenated along N (ovfcc_weights_concat);
                               part i owns the next parts[i].N output columns */
    OVFCC_FUSED_GLU = 2,    /* parts[0] = gate, parts[1] = up, glu_type applied (ovfcc_weights_glu); root = the Multiply */
    OVFCC_FUSED_MLP = 3     /* a gated unit read by nothing but one more compressed MatMul: parts[0] = gate, parts[1] = up,
                               parts[2] = down (ovfcc_weights_glu, then ovfcc_weights_mlp with the down node); root = the
                               down projection's root.  The subgraph MLPFusionPass folds into LLMMLP
                               (src/plugins/intel_cpu/src/transformations/cpu_opset/x64/pass/mlp_fusion.cpp:48-120),
                               here over compressed weights of any supported type; the gated unit's output must be f16 */
};
typedef struct ovfcc_fused {
    int32_t kind;
    int32_t n_parts;
    int32_t parts[4];  /* indices into the folds array */
    int32_t glu_type;  /* OVFCC_GLU_SWISH | OVFCC_GLU_GELU | OVFCC_GLU_GELU_TANH */
    int32_t root;      /* GLU: the Multiply node that the fused node's output replaces; MLP: the down projection's
                          root; otherwise -1 */
} ovfcc_fused;

/* Every compressed FullyConnected of the node array (bias Adds folded in where the reference's rule allows) in
 * folds[0 .. *n_folds), and their grouping into launches in fused[0 .. *n_fused).  Every fold appears in exactly one
 * group.  OVFCC_EINVAL when an output array is too small. */
int ovfcc_fold_model(const ovfcc_gnode* nodes, int n_nodes, ovfcc_fold* folds, int max_folds, int* n_folds,
                     ovfcc_fused* fused, int max_fused, int* n_fused);

/* ---- mixture-of-experts layers ---------------------------------------------------------------------------- */

/* A matched GatherMatmulCompressed node: the expert matrices of a mixture-of-experts layer applied to routed rows
 * (src/common/transformations/include/ov_ops/gather_matmul.hpp:17-41, gather_matmul_compressed.hpp:17-33; shapes
 * src/common/transformations/src/ov_ops/gather_matmul.cpp:38-130).  Either an internal::GatherMatmul whose B input is
 * the weight-decompression subgraph over a batched Constant -- [E, N, K], or grouped [E, N, K/G, G] behind a Reshape to
 * three dimensions -- the role of ConvertGatherMatmulToGatherMatmulCompressed
 * (src/common/transformations/src/transformations/op_conversions/convert_gather_matmul_to_compressed.cpp:27-92), or an
 * internal::GatherMatmulCompressed as that pass leaves it.  desc describes ONE expert: expert e's node is created
 * with ovfcc_weights_create from slice e of every constant (the views are [E, N, K] and [E, N, K/G]: slice e
 * starts at element e N K, resp. e N K/G, of the flattened constant -- for 4-bit types with an odd element count per
 * expert that is in the middle of a byte and the host re-packs the slice), and the E nodes go to
 * ovfcc_gather_matmul_device / ovfcc_gather_matmul_routed_device. */
typedef struct ovfcc_gather_fold {
    ovfcc_fc_desc desc;
    int32_t n_experts;
    int32_t root;         /* the GatherMatmul / GatherMatmulCompressed node */
    int32_t activations;  /* A [1 or top_k, M, K] */
    int32_t indices;      /* [M, top_k] */
    int32_t top_k;        /* -1 when dynamic */
    int32_t weights, scales, zero_points, bias; /* Constant nodes; -1 = absent */
    int32_t scale_broadcast;  /* one scale value for the whole layer */
    int32_t zp_from_real;     /* as in ovfcc_fold */
    int32_t bias_per_expert;  /* the bias Constant holds E x N values (else N, shared by the experts) */
    int32_t activations_f32;
    int64_t w_view[3], scale_view[3], zp_view[3];
    int32_t n_chain;
    int32_t chain[16];
} ovfcc_gather_fold;

int ovfcc_fold_gather_matmul(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_gather_fold* out);

/* Expert (or group) `expert` of a gather / grouped fold as a node of its own: slice `expert` of every batched
 * Constant (convert_gather_matmul_to_compressed.cpp:27-92 re-views the same Constants as [E, N, K], [E, N, K/G]).  A
 * 4-bit slice that begins or ends in the middle of a byte is re-packed; a one-element scale or zero-point serves
 * every expert; the bias Constant holds N values shared by the experts or E x N (bias_per_expert).  Otherwise as
 * ovfcc_fold_weights_create. */
int ovfcc_fold_expert_weights_create(ovfcc_ctx* ctx, const ovfcc_gnode* nodes, int n_nodes, const ovfcc_gather_fold* fold,
                                     int expert, const void* const* constant_data, int extra_flags, ovfcc_weights** out);

/* A matched GroupedMatMulCompressed node (src/common/transformations/include/ov_ops/grouped_matmul_compressed.hpp:
 * 17-66): either a v17::GroupedMatMul (src/core/include/openvino/op/grouped_matmul.hpp:26-50) whose B input is the
 * weight-decompression subgraph over a batched Constant [G, N, K] (or [G, N, K/g, g] behind a Reshape) -- the role
 * of ConvertGroupedMatMulToGroupedMatMulCompressed (src/common/transformations/src/transformations/op_conversions/
 * convert_grouped_matmul_to_compressed.cpp:25-118) -- or an internal::GroupedMatMulCompressed as that pass leaves
 * it.  The result uses ovfcc_gather_fold with this reading: n_experts = the number of groups G, activations = A
 * ([rows, K] with offsets, [G, M, K] without), indices = the offsets node ([G], int32 or int64 cumulative row ends)
 * or -1 for the 3-D x 3-D form, top_k = -1, bias = -1 (the op has none).  Group g's node is created from slice g of
 * every constant, as for ovfcc_fold_gather_matmul, and the G nodes go to ovfcc_grouped_matmul_device.  Weights
 * behind a Transpose ([G, K, N] constants) are OVFCC_EUNSUPPORTED. */
int ovfcc_fold_grouped_matmul(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_gather_fold* out);

/* A matched expert block: three GatherMatmul[Compressed] nodes, the gate activation, the Multiply by the routing
 * weights and the ReduceSum over the selected experts -- what Convert3GatherMatmulMoeBlockToMoeOp
 * (src/common/transformations/src/transformations/common_optimizations/moe_op_fusion.cpp:55-232) folds into
 * MOE / MOECompressed with Expert_type::GEMM3_SWIGLU (src/common/transformations/include/ov_ops/moe_compressed.hpp:15-75):
 *     Reshape( ReduceSum( down(act(gate(u)) * up(u)) * Unsqueeze(Transpose([Slice](routing))) ) ),
 *     u = Unsqueeze([Reshape](hidden_states)), all three over the same indices.
 * gate[e] and up[e] become one node with a gated linear unit (ovfcc_weights_glu, glu_type), down[e] another, and the
 * block is one ovfcc_moe_device / ovfcc_moe_routed_device call with x = hidden_states as [M, H], routing = the
 * tensor that enters the Transpose ([M, top_k]) and the indices. */
typedef struct ovfcc_moe_fold {
    ovfcc_gather_fold gate, up, down;
    int32_t glu_type;       /* OVFCC_GLU_SWISH | OVFCC_GLU_GELU | OVFCC_GLU_GELU_TANH */
    int32_t root;           /* the closing Reshape: the node whose output the block produces */
    int32_t hidden_states;
    int32_t routing;        /* producer of the [M, top_k] routing weights (the Slice, where there is one) */
    int32_t indices;
    int32_t n_chain;        /* nodes between the inputs and the root that the block absorbs, the three folds' own aside */
    int32_t chain[16];
} ovfcc_moe_fold;

/* root: the closing Reshape (or the ReduceSum under it). */
int ovfcc_fold_moe(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_moe_fold* out);

#ifdef __cplusplus
}
#endif
#endif /* OVFCC_GRAPH_H */
