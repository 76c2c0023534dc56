// From a matched node to the arrays ovfcc_weights_create takes: the constants of the weight-decompression
// subgraph are re-viewed without moving bytes where the descriptor allows it (weights, integer zero-points), and
// converted where the graph stores them in another element type (f32 scales and bias -> f16, real-typed zero-points
// -> u8) -- the data half of ConvertFullyConnectedToFullyConnectedCompressed
// (src/common/transformations/src/transformations/op_conversions/convert_fc_to_compressed.cpp:127-225, which reshapes
// the Constants and converts a real zero-point to the weights' type) and, for batched expert constants, of
// ConvertGatherMatmulToGatherMatmulCompressed (convert_gather_matmul_to_compressed.cpp:27-92).  Host code only.
#include <cmath>
#include <cstring>

#include "ovfcc_graph.h"
#include "ovfcc_internal.h"

namespace ovfcc {
namespace {

bool four_bit(int t) { return t == OVFCC_U4 || t == OVFCC_I4; }
bool real(int t) { return t == OVFCC_F16 || t == OVFCC_F32; }

float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 1023u;
    uint32_t bits;
    if (exp == 31u) {
        bits = sign | 0x7f800000u | (man << 13);
    } else if (exp != 0u) {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    } else if (man == 0u) {
        bits = sign;
    } else {  // subnormal half: man * 2^-24
        float v = std::ldexp((float)man, -24);
        std::memcpy(&bits, &v, 4);
        bits |= sign;
    }
    float out;
    std::memcpy(&out, &bits, 4);
    return out;
}

// round to nearest, ties to even; overflow to infinity: what ov::float16(float) does (src/core/src/type/float16.cpp)
uint16_t float_to_half(float v) {
    uint32_t bits;
    std::memcpy(&bits, &v, 4);
    const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    const uint32_t mag = bits & 0x7fffffffu;
    if (mag >= 0x7f800000u)  // infinity, NaN (kept quiet)
        return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u | ((mag >> 13) & 1023u) : 0u));
    if (mag >= 0x477ff000u)  // rounds to 65536 or more
        return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u)   // at most 2^-25: rounds to zero (the tie at 2^-25 goes to the even 0)
        return sign;
    const int exp = (int)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u;
    // the result keeps `keep` bits of the 24-bit significand: 11 for normal halves, fewer below 2^-14
    const int drop = exp >= -14 ? 13 : 13 + (-14 - exp);
    const uint32_t rest = man & ((1u << drop) - 1u), half = 1u << (drop - 1);
    man >>= drop;
    if (rest > half || (rest == half && (man & 1u)))
        ++man;
    // normal: man has its hidden bit at 1 << 10, adding the biased exponent minus one lets a carry ripple into it
    const uint32_t out = exp >= -14 ? ((uint32_t)(exp + 14) << 10) + man : man;
    return (uint16_t)(sign | out);
}

struct Roles {
    ovfcc_fc_desc desc;
    int weights, scales, zero_points, bias;
    bool scale_broadcast, zp_from_real, bias_per_expert;
    int64_t n_experts;  // 1 for a plain node
};

int64_t count_of(const ovfcc_gnode& n) {
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

struct Source {
    const ovfcc_gnode* node = nullptr;
    const uint8_t* bytes = nullptr;
    int64_t count = 0;
};

int source(const ovfcc_gnode* nodes, int n_nodes, const void* const* data, int id, const char* what, Source& out) {
    if (id < 0 || id >= n_nodes)
        return fail(OVFCC_EINVAL, std::string("the fold's ") + what + " is not a node of the graph");
    const ovfcc_gnode& n = nodes[id];
    if (n.op != OVFCC_OP_CONSTANT)
        return fail(OVFCC_EINVAL, std::string("the fold's ") + what + " is not a Constant");
    if (!data[id])
        return fail(OVFCC_EINVAL, std::string("no data given for the ") + what + " Constant (node " + std::to_string(id) + ")");
    out.node = &n;
    out.bytes = static_cast<const uint8_t*>(data[id]);
    out.count = count_of(n);
    if (out.count < 0)
        return fail(OVFCC_EINVAL, std::string("the ") + what + " Constant has no static shape");
    return OVFCC_OK;
}

// `count` elements from element `first` of a real-typed constant, as f16 bits (one value replicated when `broadcast`)
int reals_to_half(const Source& s, int64_t first, int64_t count, bool broadcast, const char* what, std::vector<uint16_t>& out) {
    if (!real(s.node->type))
        return fail(OVFCC_EUNSUPPORTED, std::string(what) + " must be an f16 or f32 Constant");
    if (broadcast ? s.count != 1 : first + count > s.count)
        return fail(OVFCC_EINVAL, std::string(what) + " Constant of " + std::to_string(s.count) + " elements, the node needs " +
                                      std::to_string(broadcast ? 1 : first + count));
    out.resize((size_t)count);
    for (int64_t i = 0; i < count; ++i) {
        const int64_t at = broadcast ? 0 : first + i;
        if (s.node->type == OVFCC_F16) {
            std::memcpy(&out[(size_t)i], s.bytes + 2 * at, 2);
        } else {
            float v;
            std::memcpy(&v, s.bytes + 4 * at, 4);
            out[(size_t)i] = float_to_half(v);
        }
    }
    return OVFCC_OK;
}

// `count` elements from element `first` of a packed constant (two 4-bit elements per byte, low nibble first), as a
// packed buffer of its own; a slice that starts in the middle of a byte is shifted down by one nibble
void packed_slice(const uint8_t* bytes, bool nibbles, int64_t first, int64_t count, std::vector<uint8_t>& out) {
    out.assign((size_t)(nibbles ? (count + 1) / 2 : count), 0);
    if (!nibbles) {
        std::memcpy(out.data(), bytes + first, (size_t)count);
    } else if ((first & 1) == 0) {
        std::memcpy(out.data(), bytes + first / 2, (size_t)(count / 2));
        if (count & 1)
            out[(size_t)(count / 2)] = bytes[(first + count) / 2] & 15;
    } else {
        for (int64_t i = 0; i < count; ++i) {
            const int64_t at = first + i;
            const uint8_t v = (at & 1) ? (uint8_t)(bytes[at >> 1] >> 4) : (uint8_t)(bytes[at >> 1] & 15);
            out[(size_t)(i >> 1)] |= (uint8_t)((i & 1) ? v << 4 : v);
        }
    }
}

int gather(const ovfcc_gnode* nodes, int n_nodes, const Roles& r, int64_t expert, const void* const* data, FoldConstants& out) {
    if (!nodes || !data || n_nodes <= 0)
        return fail(OVFCC_EINVAL, "null node array or constant table");
    if (expert < 0 || expert >= r.n_experts)
        return fail(OVFCC_EINVAL, "expert " + std::to_string(expert) + " of " + std::to_string(r.n_experts));
    const ovfcc_fc_desc& d = r.desc;
    if (d.N <= 0 || d.K <= 0 || d.group_size <= 0 || d.K % d.group_size)
        return fail(OVFCC_EINVAL, "the fold's descriptor has no valid N, K and group size");
    out = FoldConstants{};
    out.desc = d;
    const int64_t N = d.N, K = d.K, ng = K / d.group_size, per_node = N * ng;

    Source w;
    if (int rc = source(nodes, n_nodes, data, r.weights, "weights", w))
        return rc;
    if (w.node->type != d.w_type)
        return fail(OVFCC_EINVAL, "the weights Constant's element type differs from the descriptor's");
    if (w.count != r.n_experts * N * K)
        return fail(OVFCC_EINVAL, "weights Constant of " + std::to_string(w.count) + " elements for " +
                                      std::to_string(r.n_experts * N * K));
    const int64_t w_first = expert * N * K;
    if (!four_bit(d.w_type)) {
        out.weights = w.bytes + w_first;
    } else if ((w_first & 1) == 0) {
        out.weights = w.bytes + w_first / 2;
        if ((N * K) & 1) {  // the last byte is shared with the next expert: hand over a copy with a clean high nibble
            packed_slice(w.bytes, true, w_first, N * K, out.packed);
            out.weights = out.packed.data();
        }
    } else {
        packed_slice(w.bytes, true, w_first, N * K, out.packed);
        out.weights = out.packed.data();
    }

    Source s;
    if (int rc = source(nodes, n_nodes, data, r.scales, "scale", s))
        return rc;
    if (!r.scale_broadcast && s.count != r.n_experts * per_node)
        return fail(OVFCC_EINVAL, "scale Constant of " + std::to_string(s.count) + " elements for " +
                                      std::to_string(r.n_experts * per_node) + " groups");
    if (int rc = reals_to_half(s, expert * per_node, per_node, r.scale_broadcast, "scale", out.scales))
        return rc;

    if (r.zero_points >= 0) {
        if (d.zp_type == OVFCC_NONE)
            return fail(OVFCC_EINVAL, "the fold names a zero-point Constant but its descriptor has none");
        Source z;
        if (int rc = source(nodes, n_nodes, data, r.zero_points, "zero-point", z))
            return rc;
        const int64_t count = d.zp_scalar ? 1 : per_node, first = d.zp_scalar ? 0 : expert * per_node;
        if (d.zp_scalar ? z.count != 1 : z.count != r.n_experts * per_node)
            return fail(OVFCC_EINVAL, "zero-point Constant of " + std::to_string(z.count) + " elements");
        if (r.zp_from_real) {
            // real-typed zero-points (NNCF stores some so) must be integers in 0..255 and become u8
            if (!real(z.node->type) || d.zp_type != OVFCC_U8)
                return fail(OVFCC_EINVAL, "a zero-point marked real-typed must be an f16 / f32 Constant described as u8");
            out.zero_points.resize((size_t)count);
            for (int64_t i = 0; i < count; ++i) {
                float v;
                if (z.node->type == OVFCC_F16) {
                    uint16_t h;
                    std::memcpy(&h, z.bytes + 2 * (first + i), 2);
                    v = half_to_float(h);
                } else {
                    std::memcpy(&v, z.bytes + 4 * (first + i), 4);
                }
                if (!(v >= 0.0f && v <= 255.0f) || v != (float)(int)v)
                    return fail(OVFCC_EUNSUPPORTED, "zero-point values must be integers in 0..255");
                out.zero_points[(size_t)i] = (uint8_t)v;
            }
        } else {
            if (z.node->type != d.zp_type)
                return fail(OVFCC_EINVAL, "the zero-point Constant's element type differs from the descriptor's");
            packed_slice(z.bytes, d.zp_type == OVFCC_U4, first, count, out.zero_points);
        }
    } else if (d.zp_type != OVFCC_NONE) {
        return fail(OVFCC_EINVAL, "the descriptor has a zero-point but the fold names no Constant");
    }

    if (r.bias >= 0) {
        Source b;
        if (int rc = source(nodes, n_nodes, data, r.bias, "bias", b))
            return rc;
        if (b.count != (r.bias_per_expert ? r.n_experts * N : N))
            return fail(OVFCC_EINVAL, "bias Constant of " + std::to_string(b.count) + " elements for N = " + std::to_string(N));
        if (int rc = reals_to_half(b, r.bias_per_expert ? expert * N : 0, N, false, "bias", out.bias))
            return rc;
        out.desc.bias_type = OVFCC_F16;
    }
    return OVFCC_OK;
}

}  // namespace

int fold_constants(const ovfcc_gnode* nodes, int n_nodes, const ovfcc_fold& f, const void* const* data, FoldConstants& out) {
    const Roles r{f.desc, f.weights, f.scales, f.zero_points, f.bias, f.scale_broadcast != 0, f.zp_from_real != 0, false, 1};
    return gather(nodes, n_nodes, r, 0, data, out);
}

int fold_expert_constants(const ovfcc_gnode* nodes, int n_nodes, const ovfcc_gather_fold& f, int expert,
                          const void* const* data, FoldConstants& out) {
    if (f.n_experts <= 0)
        return fail(OVFCC_EINVAL, "the fold has no experts");
    const Roles r{f.desc, f.weights, f.scales, f.zero_points, f.bias, f.scale_broadcast != 0, f.zp_from_real != 0,
                  f.bias_per_expert != 0, f.n_experts};
    return gather(nodes, n_nodes, r, expert, data, out);
}

}  // namespace ovfcc
