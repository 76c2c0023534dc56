// Graph-side decisions of the weight-compressed FullyConnected path on plain node arrays (include/ovfcc_graph.h):
// which subgraphs are one FullyConnectedCompressed node, how their constants are re-viewed, which bias Adds fold
// in, and which nodes share a launch.  Host only; no constant data, no device.
#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

#include "ovfcc_graph.h"
#include "ovfcc_internal.h"

namespace {

using ovfcc::fail;

struct Graph {
    const ovfcc_gnode* nodes;
    int count;
    bool has(int i) const {
        return i >= 0 && i < count;
    }
    const ovfcc_gnode& at(int i) const {
        return nodes[i];
    }
    int input(int node, int k) const {
        const ovfcc_gnode& n = nodes[node];
        return k < n.n_inputs && k < OVFCC_MAX_INPUTS && has(n.inputs[k]) ? n.inputs[k] : -1;
    }
};

// number of elements of a static shape; -1 when the rank or a dimension is dynamic
int64_t element_count(const ovfcc_gnode& n) {
    if (n.rank < 0 || n.rank > OVFCC_MAX_RANK)
        return -1;
    int64_t c = 1;
    for (int i = 0; i < n.rank; ++i) {
        if (n.dims[i] < 0)
            return -1;
        c *= n.dims[i];
    }
    return c;
}

bool is_weight_type(int t) {
    return t == OVFCC_U4 || t == OVFCC_I4 || t == OVFCC_U8 || t == OVFCC_I8;
}
bool is_real(int t) {
    return t == OVFCC_F16 || t == OVFCC_F32;
}

struct Chain {
    ovfcc_fold* f;
    void add(int node) {
        if (node < 0)
            return;
        for (int i = 0; i < f->n_chain; ++i)
            if (f->chain[i] == node)
                return;
        if (f->n_chain < 16)
            f->chain[f->n_chain++] = node;
    }
};

// a Constant, directly or behind one Convert (mul_const | Convert(mul_const), sub_const | Convert(sub_const)).
// A Reshape of such a constant (the reference's builders squeeze the constant and reshape it back,
// weights_decompression_builders.cpp:118-165; constant folding removes it before the reference's matcher runs) is
// looked through: *shaped receives the node whose shape is the constant's effective shape.
int constant_behind_convert(const Graph& g, int node, Chain& chain, int* shaped = nullptr) {
    if (!g.has(node))
        return -1;
    if (shaped)
        *shaped = -1;
    if (shaped && g.at(node).op == OVFCC_OP_RESHAPE) {
        const int pattern = g.input(node, 1);
        if (pattern < 0 || g.at(pattern).op != OVFCC_OP_CONSTANT)
            return -1;
        *shaped = node;
        chain.add(node);
        chain.add(pattern);
        node = g.input(node, 0);
        if (node < 0)
            return -1;
    }
    int c = node;
    if (g.at(c).op == OVFCC_OP_CONVERT) {
        c = g.input(c, 0);
        if (c < 0 || g.at(c).op != OVFCC_OP_CONSTANT)
            return -1;
        chain.add(node);
    }
    if (g.at(c).op != OVFCC_OP_CONSTANT)
        return -1;
    chain.add(c);
    if (shaped && *shaped < 0)
        *shaped = c;
    return c;
}

// Does a scale / zero-point Constant of this shape broadcast against the weights Constant as one value per (output
// channel, group)?  `expected` is the weights' shape with the contracted axis (K, or G of [.., K/G, G, ..]) set to 1;
// the constant must equal it under right-aligned broadcasting (missing leading axes must be 1 in `expected`).
bool broadcasts_per_group(const ovfcc_gnode& c, const int64_t* expected, int expected_rank) {
    if (c.rank < 0 || c.rank > expected_rank)
        return false;
    for (int i = 0; i < expected_rank; ++i) {
        const int ci = i - (expected_rank - c.rank);
        const int64_t have = ci >= 0 ? c.dims[ci] : 1;
        if (have != expected[i])
            return false;
    }
    return true;
}

int match_impl(const Graph& g, int root, ovfcc_fold* out) {
    ovfcc_fold f;
    std::memset(&f, 0, sizeof(f));
    f.root = root;
    f.matmul = f.activations = f.weights = f.scales = f.zero_points = f.bias = -1;
    Chain chain{&f};
    if (!g.has(root))
        return fail(OVFCC_EINVAL, "root is not a node of the graph");

    // ---- a bias Add on top (FullyConnectedBiasFusion) ----
    int mm = root;
    int bias_add = -1, bias_const = -1;
    if (g.at(root).op == OVFCC_OP_ADD) {
        for (int side = 0; side < 2; ++side) {
            const int a = g.input(root, side), b = g.input(root, 1 - side);
            if (a >= 0 && b >= 0 && (g.at(a).op == OVFCC_OP_MATMUL || g.at(a).op == OVFCC_OP_FULLY_CONNECTED) &&
                g.at(b).op == OVFCC_OP_CONSTANT) {
                mm = a, bias_add = root, bias_const = b;
                break;
            }
        }
        if (bias_add < 0)
            return fail(OVFCC_EUNSUPPORTED, "Add does not join a MatMul / FullyConnected with a Constant");
        if (g.at(mm).consumers != 1)
            return fail(OVFCC_EUNSUPPORTED, "the MatMul under a bias Add must have the Add as its only consumer");
    }
    const ovfcc_gnode& m = g.at(mm);
    if (m.op != OVFCC_OP_MATMUL && m.op != OVFCC_OP_FULLY_CONNECTED)
        return fail(OVFCC_EUNSUPPORTED, "root is neither a MatMul nor a FullyConnected");
    if (m.n_inputs < 2)
        return fail(OVFCC_EINVAL, "MatMul with fewer than two inputs");
    const bool is_fc = m.op == OVFCC_OP_FULLY_CONNECTED;
    if (!is_fc && m.transpose_a)
        return fail(OVFCC_EUNSUPPORTED, "MatMul must have transpose_a = false");
    f.matmul = mm;
    f.activations = g.input(mm, 0);
    if (f.activations < 0)
        return fail(OVFCC_EINVAL, "MatMul without an activation input");

    // ---- the weight path, from the MatMul upwards: [Convert] <- [Transpose] <- [Reshape] <- Multiply ----
    int w = g.input(mm, 1);
    if (w < 0)
        return fail(OVFCC_EINVAL, "MatMul without a weight input");
    if (g.at(w).op == OVFCC_OP_CONVERT) {
        chain.add(w);
        w = g.input(w, 0);
    }
    bool transposed_in_graph = false;
    if (w >= 0 && g.at(w).op == OVFCC_OP_TRANSPOSE) {
        const int order = g.input(w, 1);
        if (order < 0 || g.at(order).op != OVFCC_OP_CONSTANT || g.at(order).n_ints != 2 || g.at(order).ints[0] != 1 ||
            g.at(order).ints[1] != 0)
            return fail(OVFCC_EUNSUPPORTED, "a Transpose on the weight path must swap the two axes of a 2-D tensor");
        transposed_in_graph = true;
        chain.add(w);
        chain.add(order);
        w = g.input(w, 0);
        // (the reference's test builders convert to the data precision ahead of the Transpose,
        // weights_decompression_builders.cpp:176-194)
        if (w >= 0 && g.at(w).op == OVFCC_OP_CONVERT) {
            chain.add(w);
            w = g.input(w, 0);
        }
    }
    int reshape = -1;
    if (w >= 0 && g.at(w).op == OVFCC_OP_RESHAPE) {
        reshape = w;
        chain.add(w);
        chain.add(g.input(w, 1));
        w = g.input(w, 0);
    }
    if (w < 0 || g.at(w).op != OVFCC_OP_MULTIPLY)
        return fail(OVFCC_EUNSUPPORTED, "no Multiply(scale) on the weight path");
    const int mul = w;
    chain.add(mul);

    // Multiply is commutative: one side is the scale (a real Constant, possibly behind a Convert), the other
    // Convert(W) or Subtract(Convert(W), zero-point)
    int scale = -1, body = -1, scale_shape = -1, zp_shape = -1;
    for (int side = 0; side < 2 && scale < 0; ++side) {
        ovfcc_fold probe = f;
        Chain pc{&probe};
        int shaped = -1;
        const int c = constant_behind_convert(g, g.input(mul, side), pc, &shaped);
        if (c >= 0 && is_real(g.at(c).type)) {
            scale = c;
            scale_shape = shaped;
            body = g.input(mul, 1 - side);
            f = probe;
        }
    }
    if (scale < 0)
        return fail(OVFCC_EUNSUPPORTED, "scale is not an f16 / f32 Constant");
    int zp = -1;
    if (body >= 0 && g.at(body).op == OVFCC_OP_SUBTRACT) {
        chain.add(body);
        zp = constant_behind_convert(g, g.input(body, 1), chain, &zp_shape);
        if (zp < 0)
            return fail(OVFCC_EUNSUPPORTED, "zero-point is not a Constant");
        body = g.input(body, 0);
    }
    if (body < 0 || g.at(body).op != OVFCC_OP_CONVERT)
        return fail(OVFCC_EUNSUPPORTED, "weights do not enter through a Convert");
    chain.add(body);
    const int wc = g.input(body, 0);
    if (wc < 0 || g.at(wc).op != OVFCC_OP_CONSTANT || !is_weight_type(g.at(wc).type))
        return fail(OVFCC_EUNSUPPORTED, "weights are not a u4 / i4 / u8 / i8 Constant");
    chain.add(wc);

    // ---- orientation and shapes ----
    // The constants are output-major ([N, K], what FullyConnected wants) when exactly one of transpose_b and a
    // Transpose node turns them; otherwise they are input-major and the library transposes them once at creation.
    const bool transpose_b = is_fc ? true : m.transpose_b != 0;
    const bool input_major = transpose_b == transposed_in_graph;
    const ovfcc_gnode& W = g.at(wc);
    if (element_count(W) <= 0)
        return fail(OVFCC_EUNSUPPORTED, "weights need a static, non-empty shape");
    int64_t N, K, G, expected[3];
    int expected_rank;
    if (W.rank == 2) {
        if (reshape >= 0)
            return fail(OVFCC_EUNSUPPORTED, "a Reshape on the weight path must merge [.., K/G, G] into K");
        N = W.dims[input_major ? 1 : 0];
        K = W.dims[input_major ? 0 : 1];
        G = K;
        expected_rank = 2;
        expected[0] = input_major ? 1 : N;
        expected[1] = input_major ? N : 1;
    } else if (W.rank == 3) {
        if (reshape < 0 || g.at(reshape).rank != 2)
            return fail(OVFCC_EUNSUPPORTED, "grouped weights [.., K/G, G] need a Reshape to two dimensions");
        expected_rank = 3;
        if (!input_major) {  // [N, K/G, G]
            N = W.dims[0], K = W.dims[1] * W.dims[2], G = W.dims[2];
            expected[0] = N, expected[1] = W.dims[1], expected[2] = 1;
        } else {  // [K/G, G, N]
            N = W.dims[2], K = W.dims[0] * W.dims[1], G = W.dims[1];
            expected[0] = W.dims[0], expected[1] = 1, expected[2] = N;
        }
        const ovfcc_gnode& R = g.at(reshape);
        if (R.dims[0] != (input_major ? K : N) || R.dims[1] != (input_major ? N : K))
            return fail(OVFCC_EUNSUPPORTED, "the Reshape on the weight path does not produce [N, K] (or [K, N])");
    } else {
        return fail(OVFCC_EUNSUPPORTED,
                    "weights must be [N, K] or [N, K/G, G] (or [K, N], [K/G, G, N] where the MatMul does not transpose them)");
    }
    if (N <= 0 || K <= 0 || G <= 0)
        return fail(OVFCC_EUNSUPPORTED, "empty weight dimension");
    const int64_t ng = K / G;

    const ovfcc_gnode& S = g.at(scale_shape);
    const int64_t scale_count = element_count(g.at(scale));
    if (scale_count != element_count(S))
        return fail(OVFCC_EUNSUPPORTED, "the Reshape above the scale changes its element count");
    if (scale_count == 1 && N * ng != 1)
        f.scale_broadcast = 1;
    else if (!broadcasts_per_group(S, expected, expected_rank))
        return fail(OVFCC_EUNSUPPORTED, "scale must hold one value, or one value per (output channel, group) in the weights' own axis order");
    f.desc.zp_type = OVFCC_NONE;
    if (zp >= 0) {
        const ovfcc_gnode& Z = g.at(zp_shape);
        const int64_t zc = element_count(g.at(zp));
        if (zc != element_count(Z))
            return fail(OVFCC_EUNSUPPORTED, "the Reshape above the zero-point changes its element count");
        if (zc == 1 && N * ng != 1)
            f.desc.zp_scalar = 1;
        else if (!broadcasts_per_group(Z, expected, expected_rank))
            return fail(OVFCC_EUNSUPPORTED, "zero-point must be scalar or hold one value per (output channel, group)");
        const int zp_type = g.at(zp).type;
        if (zp_type == OVFCC_U4 || zp_type == OVFCC_U8) {
            f.desc.zp_type = zp_type;
        } else if (is_real(zp_type)) {
            f.desc.zp_type = OVFCC_U8;  // the host checks that the values are integers in 0..255
            f.zp_from_real = 1;
        } else {
            return fail(OVFCC_EUNSUPPORTED, "zero-point must be u4, u8 or a real type holding integers");
        }
    }

    // ---- activations and output ----
    const ovfcc_gnode& X = g.at(f.activations);
    if (X.type == OVFCC_F32)
        f.activations_f32 = 1;
    else if (X.type != OVFCC_F16)
        return fail(OVFCC_EUNSUPPORTED, "activations must be f16 (or f32, converted by the host)");
    if (X.rank < 2 || X.rank > OVFCC_MAX_RANK || X.dims[X.rank - 1] != K)
        return fail(OVFCC_EUNSUPPORTED, "activations need a static rank of at least two and a last dimension equal to K");

    f.weights = wc, f.scales = scale, f.zero_points = zp;
    f.desc.N = N, f.desc.K = K, f.desc.group_size = G;
    f.desc.w_type = W.type;
    f.desc.scale_type = OVFCC_F16;
    f.desc.act_type = OVFCC_F16;
    f.desc.out_type = m.type == OVFCC_F32 ? OVFCC_F32 : OVFCC_F16;
    f.desc.flags = input_major ? OVFCC_W_INPUT_MAJOR : 0;
    f.desc.bias_type = OVFCC_NONE;
    f.w_view[0] = input_major ? K : N, f.w_view[1] = input_major ? N : K;
    if (!f.scale_broadcast)
        f.scale_view[0] = input_major ? ng : N, f.scale_view[1] = input_major ? N : ng;
    if (zp >= 0 && !f.desc.zp_scalar)
        f.zp_view[0] = input_major ? ng : N, f.zp_view[1] = input_major ? N : ng;

    // ---- bias: FullyConnected's own third input, or the Add above (last dimension N, every other 1) ----
    int bias = -1;
    if (is_fc && m.n_inputs >= 3 && g.has(m.inputs[2])) {
        const ovfcc_gnode& B = g.at(m.inputs[2]);
        const int64_t bc = element_count(B);
        if (bc != 0) {  // Constant(dynamic, Shape{0}) is the reference's "no bias"
            if (B.op != OVFCC_OP_CONSTANT || bc != N)
                return fail(OVFCC_EUNSUPPORTED, "FullyConnected bias must be a Constant of N elements");
            bias = m.inputs[2];
        }
    }
    if (bias_add >= 0) {
        const ovfcc_gnode& B = g.at(bias_const);
        if (bias >= 0)
            return fail(OVFCC_EUNSUPPORTED, "the node under the Add already has a bias");
        if (B.rank < 1 || B.rank > OVFCC_MAX_RANK || B.dims[B.rank - 1] != N || element_count(B) != N)
            return fail(OVFCC_EUNSUPPORTED, "a bias Constant needs N as its last dimension and 1 everywhere else");
        bias = bias_const;
        f.root = bias_add;
        chain.add(bias_const);
    } else {
        f.root = mm;
    }
    if (bias >= 0) {
        if (!is_real(g.at(bias).type))
            return fail(OVFCC_EUNSUPPORTED, "bias must be f16 or f32");
        f.bias = bias;
        f.desc.bias_type = OVFCC_F16;
    }
    int rc = ovfcc::validate_desc(&f.desc);
    if (rc != OVFCC_OK)
        return rc;
    *out = f;
    return OVFCC_OK;
}

bool same_format(const ovfcc_fc_desc& a, const ovfcc_fc_desc& b) {
    return a.K == b.K && a.group_size == b.group_size && a.w_type == b.w_type && a.zp_type == b.zp_type &&
           a.zp_scalar == b.zp_scalar && a.bias_type == b.bias_type && a.out_type == b.out_type && a.flags == b.flags;
}


// ---- mixture-of-experts layers --------------------------------------------------------------------------------

struct GatherChain {
    ovfcc_gather_fold* f;
    void add(int node) {
        if (node < 0)
            return;
        for (int i = 0; i < f->n_chain; ++i)
            if (f->chain[i] == node)
                return;
        if (f->n_chain < 16)
            f->chain[f->n_chain++] = node;
    }
};

// a Constant, directly or behind one Convert
int expert_constant(const Graph& g, int node, GatherChain& chain) {
    if (!g.has(node))
        return -1;
    int c = node;
    if (g.at(c).op == OVFCC_OP_CONVERT) {
        c = g.input(c, 0);
        if (c < 0)
            return -1;
        chain.add(node);
    }
    if (g.at(c).op != OVFCC_OP_CONSTANT)
        return -1;
    chain.add(c);
    return c;
}

// scale / zero-point of batched weights: one value per (expert, channel, group) in the weights' own axis order
// ([E, N, 1], or [E, N, K/G, 1] for grouped weights, leading ones allowed to be missing), or one value in all
bool per_expert_group(const ovfcc_gnode& c, int64_t E, int64_t N, int64_t ng, bool grouped) {
    const int64_t want3[3] = {E, N, 1}, want4[4] = {E, N, ng, 1};
    return grouped ? broadcasts_per_group(c, want4, 4) : (broadcasts_per_group(c, want3, 3) && ng == 1);
}

// grouped_op: the root is a GroupedMatMul[Compressed] (groups of consecutive rows, cut by offsets or by the first
// dimension of A) instead of a GatherMatmul[Compressed] (rows routed by indices); the weight side is the same
int gather_impl(const Graph& g, int root, ovfcc_gather_fold* out, bool grouped_op = false) {
    ovfcc_gather_fold f;
    std::memset(&f, 0, sizeof(f));
    f.root = root;
    f.activations = f.indices = f.weights = f.scales = f.zero_points = f.bias = -1;
    f.top_k = -1;
    GatherChain chain{&f};
    if (!g.has(root))
        return fail(OVFCC_EINVAL, "root is not a node of the graph");
    const ovfcc_gnode& m = g.at(root);
    const bool compressed =
        m.op == (grouped_op ? OVFCC_OP_GROUPED_MATMUL_COMPRESSED : OVFCC_OP_GATHER_MATMUL_COMPRESSED);
    if (m.op != (grouped_op ? OVFCC_OP_GROUPED_MATMUL : OVFCC_OP_GATHER_MATMUL) && !compressed)
        return fail(OVFCC_EUNSUPPORTED, grouped_op ? "root is neither a GroupedMatMul nor a GroupedMatMulCompressed"
                                                    : "root is neither a GatherMatmul nor a GatherMatmulCompressed");
    f.activations = g.input(root, 0);
    if (f.activations < 0)
        return fail(OVFCC_EINVAL, "no activations");
    // input slots: GatherMatmul (A, B, indices, bias[, scale, zp]); GroupedMatMul (A, B[, offsets]) and its
    // compressed form (A, B, [offsets,] scale[, zp]), where the rank of A tells whether there are offsets
    int scale_slot = 4, zp_slot = 5;
    if (grouped_op) {
        const bool with_offsets = g.at(f.activations).rank == 2;
        if (m.n_inputs < (compressed ? 3 : 2) + (with_offsets ? 1 : 0))
            return fail(OVFCC_EINVAL, "GroupedMatMul with too few inputs");
        f.indices = with_offsets ? g.input(root, 2) : -1;
        if (with_offsets && f.indices < 0)
            return fail(OVFCC_EINVAL, "GroupedMatMul over two-dimensional activations without offsets");
        scale_slot = with_offsets ? 3 : 2, zp_slot = scale_slot + 1;
    } else {
        if (m.n_inputs < (compressed ? 6 : 3))
            return fail(OVFCC_EINVAL, "GatherMatmul with too few inputs");
        f.indices = g.input(root, 2);
        if (f.indices < 0)
            return fail(OVFCC_EINVAL, "GatherMatmul without indices");
    }

    int wc = -1, scale = -1, zp = -1, reshape = -1;
    if (compressed) {
        // the node as the conversion pass leaves it: B, scale and zero-point are Constants of three dimensions (a
        // zero-point of no elements, or a missing one, stands for "none")
        wc = g.input(root, 1), scale = g.input(root, scale_slot), zp = zp_slot < m.n_inputs ? g.input(root, zp_slot) : -1;
        if (wc < 0 || g.at(wc).op != OVFCC_OP_CONSTANT || scale < 0 || g.at(scale).op != OVFCC_OP_CONSTANT)
            return fail(OVFCC_EUNSUPPORTED, "the compressed node needs Constant weights and scales");
        if (zp >= 0 && (g.at(zp).op != OVFCC_OP_CONSTANT || element_count(g.at(zp)) == 0))
            zp = -1;
        chain.add(wc), chain.add(scale), chain.add(zp);
    } else {
        // B = [Convert] <- [Reshape] <- Multiply(Subtract(Convert(W), zp) | Convert(W), scale)
        int w = g.input(root, 1);
        if (w >= 0 && g.at(w).op == OVFCC_OP_CONVERT) {
            chain.add(w);
            w = g.input(w, 0);
        }
        if (w >= 0 && g.at(w).op == OVFCC_OP_TRANSPOSE)
            return fail(OVFCC_EUNSUPPORTED, "expert weights behind a Transpose ([E, K, N]) are not supported");
        if (w >= 0 && g.at(w).op == OVFCC_OP_RESHAPE) {
            reshape = w;
            chain.add(w);
            chain.add(g.input(w, 1));
            w = g.input(w, 0);
        }
        if (w < 0 || g.at(w).op != OVFCC_OP_MULTIPLY)
            return fail(OVFCC_EUNSUPPORTED, "no Multiply(scale) on the weight path");
        chain.add(w);
        int body = -1;
        for (int side = 0; side < 2 && scale < 0; ++side) {
            ovfcc_gather_fold probe = f;
            GatherChain pc{&probe};
            const int c = expert_constant(g, g.input(w, side), pc);
            if (c >= 0 && is_real(g.at(c).type)) {
                scale = c;
                body = g.input(w, 1 - side);
                f = probe;
            }
        }
        if (scale < 0)
            return fail(OVFCC_EUNSUPPORTED, "scale is not an f16 / f32 Constant");
        if (body >= 0 && g.at(body).op == OVFCC_OP_SUBTRACT) {
            chain.add(body);
            zp = expert_constant(g, g.input(body, 1), chain);
            if (zp < 0)
                return fail(OVFCC_EUNSUPPORTED, "zero-point is not a Constant");
            body = g.input(body, 0);
        }
        if (body < 0 || g.at(body).op != OVFCC_OP_CONVERT)
            return fail(OVFCC_EUNSUPPORTED, "weights do not enter through a Convert");
        chain.add(body);
        wc = g.input(body, 0);
        if (wc < 0 || g.at(wc).op != OVFCC_OP_CONSTANT)
            return fail(OVFCC_EUNSUPPORTED, "weights are not a Constant");
        chain.add(wc);
    }
    const ovfcc_gnode& W = g.at(wc);
    if (!is_weight_type(W.type))
        return fail(OVFCC_EUNSUPPORTED, "weights are not a u4 / i4 / u8 / i8 Constant");
    if (element_count(W) <= 0)
        return fail(OVFCC_EUNSUPPORTED, "weights need a static, non-empty shape");
    int64_t E, N, K, G;
    bool grouped = false;
    if (W.rank == 3) {
        if (reshape >= 0)
            return fail(OVFCC_EUNSUPPORTED, "a Reshape on the weight path must merge [E, N, K/G, G] into [E, N, K]");
        E = W.dims[0], N = W.dims[1], K = W.dims[2], G = K;
        // GatherMatmulCompressed carries grouped scales as [E, N, K/G] beside [E, N, K] weights
        if (compressed && g.at(scale).rank == 3 && g.at(scale).dims[2] > 1) {
            if (K % g.at(scale).dims[2])
                return fail(OVFCC_EUNSUPPORTED, "the scales' group count does not divide K");
            G = K / g.at(scale).dims[2];
            grouped = true;
        }
    } else if (W.rank == 4) {
        E = W.dims[0], N = W.dims[1], K = W.dims[2] * W.dims[3], G = W.dims[3];
        grouped = true;
        if (!compressed) {
            if (reshape < 0 || g.at(reshape).rank != 3 || g.at(reshape).dims[0] != E || g.at(reshape).dims[1] != N ||
                g.at(reshape).dims[2] != K)
                return fail(OVFCC_EUNSUPPORTED, "grouped expert weights [E, N, K/G, G] need a Reshape to [E, N, K]");
        }
    } else {
        return fail(OVFCC_EUNSUPPORTED, "expert weights must be [E, N, K] or [E, N, K/G, G]");
    }
    const int64_t ng = K / G;
    auto shaped_ok = [&](const ovfcc_gnode& c) {
        if (compressed && W.rank == 3) {  // [E, N, K/G]
            const int64_t want[3] = {E, N, ng};
            return broadcasts_per_group(c, want, 3);
        }
        return per_expert_group(c, E, N, ng, grouped);
    };
    const int64_t sc = element_count(g.at(scale));
    if (sc == 1 && E * N * ng != 1)
        f.scale_broadcast = 1;
    else if (!shaped_ok(g.at(scale)))
        return fail(OVFCC_EUNSUPPORTED, "scale must hold one value, or one per (expert, output channel, group)");
    f.desc.zp_type = OVFCC_NONE;
    if (zp >= 0) {
        const int64_t zc = element_count(g.at(zp));
        if (zc == 1 && E * N * ng != 1)
            f.desc.zp_scalar = 1;
        else if (!shaped_ok(g.at(zp)))
            return fail(OVFCC_EUNSUPPORTED, "zero-point must be scalar or hold one value per (expert, output channel, group)");
        const int zt = g.at(zp).type;
        if (zt == OVFCC_U4 || zt == OVFCC_U8) {
            f.desc.zp_type = zt;
        } else if (is_real(zt)) {
            f.desc.zp_type = OVFCC_U8;
            f.zp_from_real = 1;
        } else {
            return fail(OVFCC_EUNSUPPORTED, "zero-point must be u4, u8 or a real type holding integers");
        }
    }

    const ovfcc_gnode& A = g.at(f.activations);
    if (A.type == OVFCC_F32)
        f.activations_f32 = 1;
    else if (A.type != OVFCC_F16)
        return fail(OVFCC_EUNSUPPORTED, "activations must be f16 (or f32, converted by the host)");
    if (grouped_op) {
        // ---- activations [rows, K] with offsets [G], or [G, M, K] ----
        if (f.indices >= 0) {
            const ovfcc_gnode& O = g.at(f.indices);
            if (A.rank != 2 || A.dims[1] != K)
                return fail(OVFCC_EUNSUPPORTED, "activations must be [rows, K]");
            if (O.rank != 1 || (O.dims[0] >= 0 && O.dims[0] != E))
                return fail(OVFCC_EUNSUPPORTED, "offsets must hold one cumulative row end per group");
        } else if (A.rank != 3 || A.dims[2] != K || (A.dims[0] >= 0 && A.dims[0] != E)) {
            return fail(OVFCC_EUNSUPPORTED, "activations must be [G, M, K]");
        }
    } else {
        // ---- activations [1 or top_k, M, K], indices [M, top_k] ----
        if (A.rank != 3 || A.dims[2] != K)
            return fail(OVFCC_EUNSUPPORTED, "activations must be [1 or top_k, M, K]");
        const ovfcc_gnode& I = g.at(f.indices);
        if (I.rank != 2)
            return fail(OVFCC_EUNSUPPORTED, "indices must be [M, top_k]");
        f.top_k = I.dims[1] >= 0 ? (int32_t)I.dims[1] : -1;
        if (f.top_k > 0 && A.dims[0] >= 0 && A.dims[0] != 1 && A.dims[0] != f.top_k)
            return fail(OVFCC_EUNSUPPORTED, "the first dimension of the activations must be 1 or top_k");
        if (f.top_k > E)
            return fail(OVFCC_EUNSUPPORTED, "more selections per row than experts");
    }

    // ---- bias (GatherMatmul only): Constant(dynamic, Shape{0}) = none; N values shared, or E x N ----
    const int bias = grouped_op ? -1 : g.input(root, 3);
    if (bias >= 0 && element_count(g.at(bias)) != 0) {
        const ovfcc_gnode& B = g.at(bias);
        const int64_t bc = element_count(B);
        if (B.op != OVFCC_OP_CONSTANT || !is_real(B.type) || (bc != N && bc != E * N) || B.rank < 1 ||
            B.dims[B.rank - 1] != N)
            return fail(OVFCC_EUNSUPPORTED, "bias must be an f16 / f32 Constant of N or E x N values with N innermost");
        f.bias = bias;
        f.bias_per_expert = bc == E * N && E > 1;
        f.desc.bias_type = OVFCC_F16;
        chain.add(bias);
    }
    f.n_experts = (int32_t)E;
    f.weights = wc, f.scales = scale, f.zero_points = zp;
    f.desc.N = N, f.desc.K = K, f.desc.group_size = G;
    f.desc.w_type = W.type;
    f.desc.scale_type = OVFCC_F16;
    f.desc.act_type = OVFCC_F16;
    f.desc.out_type = m.type == OVFCC_F32 ? OVFCC_F32 : OVFCC_F16;
    f.w_view[0] = E, f.w_view[1] = N, f.w_view[2] = K;
    if (!f.scale_broadcast)
        f.scale_view[0] = E, f.scale_view[1] = N, f.scale_view[2] = ng;
    if (zp >= 0 && !f.desc.zp_scalar)
        f.zp_view[0] = E, f.zp_view[1] = N, f.zp_view[2] = ng;
    if (E > ((int64_t)1 << 16))
        return fail(OVFCC_EUNSUPPORTED, "more than 65536 experts");
    int rc = ovfcc::validate_desc(&f.desc);
    if (rc != OVFCC_OK)
        return rc;
    *out = f;
    return OVFCC_OK;
}

bool is_gather(const ovfcc_gnode& n) {
    return n.op == OVFCC_OP_GATHER_MATMUL || n.op == OVFCC_OP_GATHER_MATMUL_COMPRESSED;
}

int moe_impl(const Graph& g, int root, ovfcc_moe_fold* out) {
    ovfcc_moe_fold f;
    std::memset(&f, 0, sizeof(f));
    f.root = root;
    f.hidden_states = f.routing = f.indices = -1;
    auto absorb = [&](int node) {
        if (node >= 0 && f.n_chain < 16)
            f.chain[f.n_chain++] = node;
    };
    if (!g.has(root))
        return fail(OVFCC_EINVAL, "root is not a node of the graph");
    int sum = root;
    if (g.at(root).op == OVFCC_OP_RESHAPE) {
        absorb(root);
        absorb(g.input(root, 1));
        sum = g.input(root, 0);
    }
    if (sum < 0 || g.at(sum).op != OVFCC_OP_REDUCE_SUM || g.at(sum).attr != 0)
        return fail(OVFCC_EUNSUPPORTED, "the block does not end in ReduceSum(keep_dims = false) [-> Reshape]");
    absorb(sum);
    absorb(g.input(sum, 1));
    const int mul = g.input(sum, 0);
    if (mul < 0 || g.at(mul).op != OVFCC_OP_MULTIPLY || g.at(mul).consumers != 1)
        return fail(OVFCC_EUNSUPPORTED, "ReduceSum must read a Multiply that nothing else reads");
    absorb(mul);
    // Multiply(down(..), Unsqueeze(Transpose([Slice](routing))))
    int down = -1, unsq = -1;
    for (int side = 0; side < 2; ++side) {
        const int a = g.input(mul, side), b = g.input(mul, 1 - side);
        if (a >= 0 && b >= 0 && is_gather(g.at(a)) && g.at(b).op == OVFCC_OP_UNSQUEEZE)
            down = a, unsq = b;
    }
    if (down < 0)
        return fail(OVFCC_EUNSUPPORTED, "no GatherMatmul multiplied by the unsqueezed routing weights");
    absorb(unsq);
    absorb(g.input(unsq, 1));
    const int tr = g.input(unsq, 0);
    if (tr < 0 || g.at(tr).op != OVFCC_OP_TRANSPOSE)
        return fail(OVFCC_EUNSUPPORTED, "the routing weights must pass a Transpose ([M, top_k] -> [top_k, M])");
    absorb(tr);
    absorb(g.input(tr, 1));
    f.routing = g.input(tr, 0);
    if (f.routing < 0)
        return fail(OVFCC_EINVAL, "Transpose without an input");
    // the expert projections
    const int glu_mul = g.input(down, 0);
    if (glu_mul < 0 || g.at(glu_mul).op != OVFCC_OP_MULTIPLY)
        return fail(OVFCC_EUNSUPPORTED, "the down projection must read Multiply(act(gate), up)");
    absorb(glu_mul);
    int gate = -1, up = -1, act = -1;
    for (int side = 0; side < 2; ++side) {
        const int a = g.input(glu_mul, side), b = g.input(glu_mul, 1 - side);
        if (a >= 0 && b >= 0 && (g.at(a).op == OVFCC_OP_SWISH || g.at(a).op == OVFCC_OP_GELU) && is_gather(g.at(b))) {
            const int gt = g.input(a, 0);
            if (gt >= 0 && is_gather(g.at(gt)))
                act = a, gate = gt, up = b;
        }
    }
    if (gate < 0)
        return fail(OVFCC_EUNSUPPORTED, "no Swish / Gelu of a GatherMatmul beside a second GatherMatmul");
    if (g.at(act).op == OVFCC_OP_SWISH && g.at(act).n_inputs != 1)
        return fail(OVFCC_EUNSUPPORTED, "Swish with a beta input");
    absorb(act);
    f.glu_type = g.at(act).op == OVFCC_OP_SWISH ? OVFCC_GLU_SWISH : (g.at(act).attr ? OVFCC_GLU_GELU_TANH : OVFCC_GLU_GELU);
    // the three nodes are all plain or all compressed (the reference bails out on a mix)
    if (g.at(gate).op != g.at(up).op || g.at(gate).op != g.at(down).op)
        return fail(OVFCC_EUNSUPPORTED, "the three projections mix GatherMatmul and GatherMatmulCompressed");
    int rc = gather_impl(g, gate, &f.gate);
    if (!rc)
        rc = gather_impl(g, up, &f.up);
    if (!rc)
        rc = gather_impl(g, down, &f.down);
    if (rc)
        return rc;
    if (f.gate.bias >= 0 || f.up.bias >= 0 || f.down.bias >= 0)
        return fail(OVFCC_EUNSUPPORTED, "the expert block has no place for biases");
    if (f.gate.indices != f.up.indices || f.gate.indices != f.down.indices)
        return fail(OVFCC_EUNSUPPORTED, "the three projections read different indices");
    f.indices = f.gate.indices;
    if (f.gate.activations != f.up.activations)
        return fail(OVFCC_EUNSUPPORTED, "gate and up read different activations");
    if (f.gate.n_experts != f.up.n_experts || f.gate.n_experts != f.down.n_experts)
        return fail(OVFCC_EUNSUPPORTED, "the projections differ in their number of experts");
    if (f.gate.desc.N != f.up.desc.N || f.gate.desc.K != f.up.desc.K || f.down.desc.K != f.gate.desc.N ||
        f.down.desc.N != f.gate.desc.K)
        return fail(OVFCC_EUNSUPPORTED, "the projections' shapes do not chain (gate, up: H -> I; down: I -> H)");
    if (!same_format(f.gate.desc, f.up.desc))
        return fail(OVFCC_EUNSUPPORTED, "gate and up differ in format");
    if (f.gate.desc.out_type != OVFCC_F16)
        return fail(OVFCC_EUNSUPPORTED, "the activations between the projections are f16");
    // u = Unsqueeze([Reshape](hidden_states))
    const int u = f.gate.activations;
    if (g.at(u).op != OVFCC_OP_UNSQUEEZE)
        return fail(OVFCC_EUNSUPPORTED, "gate and up must read Unsqueeze([Reshape](hidden states))");
    absorb(u);
    absorb(g.input(u, 1));
    int h = g.input(u, 0);
    if (h >= 0 && g.at(h).op == OVFCC_OP_RESHAPE) {
        absorb(h);
        absorb(g.input(h, 1));
        h = g.input(h, 0);
    }
    if (h < 0)
        return fail(OVFCC_EINVAL, "Unsqueeze without an input");
    f.hidden_states = h;
    const ovfcc_gnode& H = g.at(h);
    if (H.rank < 2 || H.dims[H.rank - 1] != f.gate.desc.K)
        return fail(OVFCC_EUNSUPPORTED, "the hidden states' last dimension is not the projections' input size");
    const ovfcc_gnode& R = g.at(f.routing);
    if (R.rank != 2 || (f.gate.top_k > 0 && R.dims[1] >= 0 && R.dims[1] != f.gate.top_k))
        return fail(OVFCC_EUNSUPPORTED, "the routing weights that enter the Transpose must be [M, top_k]");
    *out = f;
    return OVFCC_OK;
}

}  // namespace

extern "C" {

int ovfcc_fold_match(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_fold* out) {
    if (!nodes || n_nodes <= 0 || !out)
        return fail(OVFCC_EINVAL, "null graph or output");
    for (int i = 0; i < n_nodes; ++i)
        if (nodes[i].n_inputs < 0 || nodes[i].n_inputs > OVFCC_MAX_INPUTS || nodes[i].rank > OVFCC_MAX_RANK)
            return fail(OVFCC_EINVAL, "a node has more than OVFCC_MAX_INPUTS inputs or a rank above OVFCC_MAX_RANK");
    return match_impl(Graph{nodes, n_nodes}, root, out);
}

int ovfcc_fold_model(const ovfcc_gnode* nodes, int n_nodes, ovfcc_fold* folds, int max_folds, int* n_folds,
                     ovfcc_fused* fused, int max_fused, int* n_fused) {
    if (!nodes || n_nodes <= 0 || !folds || !n_folds || !fused || !n_fused || max_folds < 0 || max_fused < 0)
        return fail(OVFCC_EINVAL, "null graph or output");
    *n_folds = *n_fused = 0;
    const Graph g{nodes, n_nodes};
    // consumers of every node
    std::vector<std::vector<int>> users((size_t)n_nodes);
    for (int i = 0; i < n_nodes; ++i) {
        if (nodes[i].n_inputs < 0 || nodes[i].n_inputs > OVFCC_MAX_INPUTS || nodes[i].rank > OVFCC_MAX_RANK)
            return fail(OVFCC_EINVAL, "a node has more than OVFCC_MAX_INPUTS inputs or a rank above OVFCC_MAX_RANK");
        for (int k = 0; k < nodes[i].n_inputs; ++k)
            if (g.has(nodes[i].inputs[k]))
                users[(size_t)nodes[i].inputs[k]].push_back(i);
    }
    std::vector<ovfcc_fold> found;
    std::vector<int> fold_of_root((size_t)n_nodes, -1);
    for (int i = 0; i < n_nodes; ++i) {
        if (nodes[i].op != OVFCC_OP_MATMUL && nodes[i].op != OVFCC_OP_FULLY_CONNECTED)
            continue;
        ovfcc_fold f;
        if (match_impl(g, i, &f) != OVFCC_OK)
            continue;
        // the bias Add above it, where the reference's rule lets it fold in
        if (users[(size_t)i].size() == 1 && nodes[users[(size_t)i][0]].op == OVFCC_OP_ADD) {
            ovfcc_fold with_bias;
            if (match_impl(g, users[(size_t)i][0], &with_bias) == OVFCC_OK)
                f = with_bias;
        }
        fold_of_root[(size_t)f.root] = (int)found.size();
        found.push_back(f);
    }
    if ((int)found.size() > max_folds)
        return fail(OVFCC_EINVAL, "more compressed FullyConnected nodes than the folds array holds");
    std::vector<ovfcc_fused> groups;
    std::vector<char> taken(found.size(), 0);
    // gated linear unit: Multiply(act(gate(x)), up(x)), both projections of one shape over the same activations,
    // each read by nothing else
    for (int i = 0; i < n_nodes; ++i) {
        if (nodes[i].op != OVFCC_OP_MULTIPLY || nodes[i].n_inputs != 2)
            continue;
        for (int side = 0; side < 2; ++side) {
            const int act = g.input(i, side), up_root = g.input(i, 1 - side);
            if (act < 0 || up_root < 0 || (nodes[act].op != OVFCC_OP_SWISH && nodes[act].op != OVFCC_OP_GELU))
                continue;
            const int gate_root = g.input(act, 0);
            if (gate_root < 0 || fold_of_root[(size_t)gate_root] < 0 || fold_of_root[(size_t)up_root] < 0)
                continue;
            const int a = fold_of_root[(size_t)gate_root], b = fold_of_root[(size_t)up_root];
            if (a == b || taken[(size_t)a] || taken[(size_t)b])
                continue;
            const ovfcc_fold &fa = found[(size_t)a], &fb = found[(size_t)b];
            if (fa.activations != fb.activations || fa.desc.N != fb.desc.N || !same_format(fa.desc, fb.desc) ||
                users[(size_t)gate_root].size() != 1 || users[(size_t)up_root].size() != 1 ||
                users[(size_t)act].size() != 1 || (nodes[act].op == OVFCC_OP_SWISH && nodes[act].n_inputs != 1))
                continue;
            ovfcc_fused u{};
            u.kind = OVFCC_FUSED_GLU;
            u.n_parts = 2;
            u.parts[0] = a, u.parts[1] = b;
            u.glu_type = nodes[act].op == OVFCC_OP_SWISH ? OVFCC_GLU_SWISH
                                                         : (nodes[act].attr ? OVFCC_GLU_GELU_TANH : OVFCC_GLU_GELU);
            u.root = i;
            groups.push_back(u);
            taken[(size_t)a] = taken[(size_t)b] = 1;
            break;
        }
    }
    // MLP: a gated unit whose only reader is one more compressed MatMul (the down projection) becomes one node with
    // it, where the intermediate activations are f16 as between two nodes
    for (ovfcc_fused& u : groups) {
        const int mul = u.root;
        if (users[(size_t)mul].size() != 1)
            continue;
        const ovfcc_fold& gate = found[(size_t)u.parts[0]];
        for (size_t d = 0; d < found.size(); ++d) {
            const ovfcc_fold& down = found[d];
            if (taken[d] || down.activations != mul || down.matmul != users[(size_t)mul][0])
                continue;
            if (gate.desc.out_type != OVFCC_F16 || down.desc.K != gate.desc.N || down.activations_f32)
                continue;
            u.kind = OVFCC_FUSED_MLP;
            u.n_parts = 3;
            u.parts[2] = (int)d;
            u.root = down.root;
            taken[d] = 1;
            break;
        }
    }
    // horizontal fusion: two or three siblings of one format over the same activations share a launch
    for (size_t a = 0; a < found.size(); ++a) {
        if (taken[a])
            continue;
        std::vector<int> sib{(int)a};
        for (size_t b = a + 1; b < found.size(); ++b)
            if (!taken[b] && found[b].activations == found[a].activations && same_format(found[a].desc, found[b].desc))
                sib.push_back((int)b);
        ovfcc_fused u{};
        u.root = -1;
        if (sib.size() >= 2 && sib.size() <= 3) {
            u.kind = OVFCC_FUSED_CONCAT;
            u.n_parts = (int)sib.size();
            for (size_t k = 0; k < sib.size(); ++k) {
                u.parts[k] = sib[k];
                taken[(size_t)sib[k]] = 1;
            }
            groups.push_back(u);
            continue;
        }
        // alone, or more siblings than one fused node takes (the reference leaves such a fan-out alone): each on its own
        for (int k : sib) {
            ovfcc_fused one{};
            one.kind = OVFCC_FUSED_SINGLE;
            one.n_parts = 1;
            one.parts[0] = k;
            one.root = -1;
            taken[(size_t)k] = 1;
            groups.push_back(one);
        }
    }
    if ((int)groups.size() > max_fused)
        return fail(OVFCC_EINVAL, "more launch groups than the fused array holds");
    std::copy(found.begin(), found.end(), folds);
    std::copy(groups.begin(), groups.end(), fused);
    *n_folds = (int)found.size();
    *n_fused = (int)groups.size();
    return OVFCC_OK;
}

int ovfcc_fold_grouped_matmul(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_gather_fold* out) {
    if (!nodes || n_nodes <= 0 || !out)
        return fail(OVFCC_EINVAL, "null argument");
    return gather_impl(Graph{nodes, n_nodes}, root, out, true);
}

int ovfcc_fold_gather_matmul(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_gather_fold* out) {
    if (!nodes || n_nodes <= 0 || !out)
        return fail(OVFCC_EINVAL, "null graph or output");
    for (int i = 0; i < n_nodes; ++i)
        if (nodes[i].n_inputs < 0 || nodes[i].n_inputs > OVFCC_MAX_INPUTS || nodes[i].rank > OVFCC_MAX_RANK)
            return fail(OVFCC_EINVAL, "a node has more than OVFCC_MAX_INPUTS inputs or a rank above OVFCC_MAX_RANK");
    return gather_impl(Graph{nodes, n_nodes}, root, out);
}

int ovfcc_fold_moe(const ovfcc_gnode* nodes, int n_nodes, int root, ovfcc_moe_fold* out) {
    if (!nodes || n_nodes <= 0 || !out)
        return fail(OVFCC_EINVAL, "null graph or output");
    for (int i = 0; i < n_nodes; ++i)
        if (nodes[i].n_inputs < 0 || nodes[i].n_inputs > OVFCC_MAX_INPUTS || nodes[i].rank > OVFCC_MAX_RANK)
            return fail(OVFCC_EINVAL, "a node has more than OVFCC_MAX_INPUTS inputs or a rank above OVFCC_MAX_RANK");
    return moe_impl(Graph{nodes, n_nodes}, root, out);
}

}  // extern "C"
