"""Graphs of the reference's own tests and builders as plain-node arrays (tests/golden/fold_cases.json names the
sources), shared by the structural tests, the sanitizer run of the host code and the GPU tests that carry a graph
all the way to numbers; and seeded data for the Constants a fold names."""
import json
import math
import os

import numpy as np

from openvino_amd import _lib
from openvino_amd.graph import Graph, decompression_subgraph

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "fold_cases.json")) as fh:
    CASES = json.load(fh)

_TYPE = {v: k for k, v in _lib.TYPE.items()}
_NP = {"f16": np.float16, "f32": np.float32}


# ---- graphs ----------------------------------------------------------------------------------------------------

def convert_fc_graph(p, root_op):
    """A row of ConvertFCToCompressed: FullyConnected (or the MatMul with transpose_b it came from) over
    Constant -> Convert -> [Subtract(Convert(zp))] -> Multiply(scale) -> [Reshape]."""
    g = Graph()
    x = g.parameter("f32", p["in_shape"])
    wshape, sshape = p["wei_shape"], p["scale_zp_shape"]
    OC, IC = wshape[0], (wshape[1] * wshape[2] if p["grouped"] else wshape[1])
    chain = decompression_subgraph(g, p["type"], wshape, sshape, sshape if p["with_zp"] else None, p["type"],
                                   reshape_to=[OC, IC] if p["grouped"] else None)
    root = g.fully_connected(x, chain) if root_op == "fully_connected" else g.matmul(x, chain, transpose_b=True)
    return g, x, root


def transposed_graph(p):
    """[IC, OC] weights with rank-1 or rank-0 scale and zero-point and a Transpose([1, 0]) above the Multiply."""
    g = Graph()
    x = g.parameter("f32", p["in_shape"])
    chain = decompression_subgraph(g, p["type"], p["wei_shape"], p["scale_zp_shape"], p["scale_zp_shape"], p["type"],
                                   transpose=True)
    return g, x, g.fully_connected(x, chain)


def builder_graph(p, x_type="f16"):
    """A subgraph as initMatMulDecompressionSubgraph emits it: weights_shape = [IC, OC]; with transpose_weights the
    constants are stored [OC, IC] ([OC, IC/G, G], scales [OC, IC/G, 1]) and a Transpose node follows, without it they
    are [IC, OC] ([IC/G, G, OC], scales [IC/G, 1, OC]); the MatMul never transposes."""
    IC, OC = p["weights_shape"]
    G = p["group"] if p["group"] != -1 else IC
    grouped = p["group"] != -1
    tw = p["transpose_weights"]
    if tw:
        wshape = [OC, IC // G, G] if grouped else [OC, IC]
        sshape = [OC, IC // G, 1] if grouped else [OC, 1]
        reshape_to = [OC, IC] if grouped else None
    else:
        wshape = [IC // G, G, OC] if grouped else [IC, OC]
        sshape = [IC // G, 1, OC] if grouped else [1, OC]
        reshape_to = [IC, OC] if grouped else None
    zp_shape = None if p["zp"] == "empty" else (sshape if p["zp"] == "full" else [])
    squeezed = [d for d in sshape if d != 1] if p.get("reshape_on_decompression") else None
    g = Graph()
    x = g.parameter(x_type, [-1, -1, IC])
    chain = decompression_subgraph(g, p["type"], wshape, sshape, zp_shape, p["type"], scale_type="f16", compute_type="f16",
                                   reshape_to=reshape_to, transpose=tw, scale_const_shape=squeezed)
    return g, x, g.matmul(x, chain)


def simple_matmul(g, x, N=64, K=256, G=128, w_type="u4", zp=True, major="output", scale_type="f16", out=None,
                  zp_type=None, zp_shape=None):
    """One compressed MatMul in the grouped form of NNCF-compressed models, output-major ([N, K/G, G] behind a
    Reshape, transpose_b) or input-major ([K/G, G, N])."""
    ng = K // G
    if major == "output":
        zs = ([N, ng, 1] if zp_shape is None else zp_shape) if zp else None
        chain = decompression_subgraph(g, w_type, [N, ng, G], [N, ng, 1], zs, zp_type or w_type,
                                       scale_type=scale_type, compute_type="f16", reshape_to=[N, K])
        return g.matmul(x, chain, transpose_b=True, type_=out)
    zs = ([ng, 1, N] if zp_shape is None else zp_shape) if zp else None
    chain = decompression_subgraph(g, w_type, [ng, G, N], [ng, 1, N], zs, zp_type or w_type,
                                   scale_type=scale_type, compute_type="f16", reshape_to=[K, N])
    return g.matmul(x, chain, type_=out)


def expert_weights(g, type_, wei_shape, scale_zp_shape, grouped, with_zp=True, compute="f32"):
    """Constant -> Convert -> [Subtract] -> Multiply -> [Reshape to three dimensions], as the reference's test builds it."""
    w = g.convert(g.constant(type_, wei_shape), compute)
    if with_zp:
        w = g.subtract(w, g.convert(g.constant(type_, scale_zp_shape), compute))
    w = g.multiply(w, g.constant(compute, scale_zp_shape))
    if grouped:
        w = g.reshape(w, list(wei_shape[:-2]) + [wei_shape[-2] * wei_shape[-1]])
    return w


def moe_block(g, act, compressed, E, H, I, top_k, hidden_shape, wtype="u4", G=128, routing_slice=False):
    """build_3gemm_bgm_model with compressed experts: returns (root, hidden, routing producer, indices, nodes)."""
    hidden = g.parameter("f16", hidden_shape)
    flat = g.reshape(hidden, [-1, H]) if len(hidden_shape) != 2 else hidden
    u = g.unsqueeze(flat, 0)
    idx = g.parameter("i32", [-1, top_k])
    routing = g.parameter("f16", [-1, E if routing_slice else top_k])

    def bgm(x, N, K):
        if compressed:
            return g.gather_matmul_compressed(x, g.constant(wtype, [E, N, K]), idx, g.constant("f16", [E, N, K // G]),
                                              g.constant(wtype, [E, N, K // G]))
        return g.gather_matmul(x, expert_weights(g, wtype, [E, N, K // G, G], [E, N, K // G, 1], True, compute="f16"), idx)
    gate = bgm(u, I, H)
    a = g.swish(gate) if act == "swish" else g.gelu(gate, tanh=(act == "gelu_tanh"))
    up = bgm(u, I, H)
    down = bgm(g.multiply(a, up), H, I)
    r = g.slice(routing, [-1, top_k]) if routing_slice else routing
    final = g.multiply(down, g.unsqueeze(g.transpose(r, [1, 0]), -1))
    out = g.reshape(g.reduce_sum(final, 0), hidden_shape)
    return out, hidden, r, idx, (gate, up, down)


def grouped_matmul_graph(shape, wt, zp, group):
    """The graph of the reference's functional test of GroupedMatMulCompressed: GroupedMatMul over the decompression
    subgraph of a batched constant, with offsets (2-D activations) or without (3-D).  Returns (g, a, offsets, root)."""
    G_, N, K = shape["b_shape"]
    gs = K if group < 0 else group
    grouped = gs != K
    ng = K // gs
    g = Graph()
    a = g.parameter("f32", shape["a_shape"])
    offsets = g.parameter("i32", [G_]) if len(shape["a_shape"]) == 2 else None
    wshape = [G_, N, ng, gs] if grouped else [G_, N, K]
    szshape = [G_, N, ng, 1] if grouped else [G_, N, 1]
    w = g.convert(g.constant(wt, wshape), "f32")
    zp_type = "u8" if wt in ("u8", "i8") else "u4"
    if zp == "full":
        w = g.subtract(w, g.convert(g.constant(zp_type, szshape), "f32"))
    elif zp == "scalar":
        w = g.subtract(w, g.convert(g.constant(zp_type, []), "f32"))
    w = g.multiply(w, g.constant("f32", szshape))
    if grouped:
        w = g.reshape(w, [G_, N, K])
    return g, a, offsets, g.grouped_matmul(a, w, offsets)


VARIANTS = [
    # name, keyword arguments of simple_matmul, bias Constant (type, shape) or None
    ("bias_f16", dict(), ("f16", [64])),
    ("bias_f32_rank3", dict(N=96, K=512), ("f32", [1, 1, 96])),
    ("input_major_bias", dict(major="input", N=128), ("f16", [1, 128])),
    ("zp_real_f16", dict(zp_type="f16"), None),
    ("zp_real_f32_u8_weights", dict(w_type="u8", zp_type="f32", scale_type="f32"), None),
    ("zp_scalar", dict(zp_shape=[]), None),
    ("zp_scalar_real", dict(zp_shape=[], zp_type="f16", major="input"), None),
    ("i8_f32_out", dict(w_type="i8", zp=False, out="f32", N=80, K=384), None),
    ("i4_input_major", dict(w_type="i4", zp=False, major="input", N=48), None),
]


def variant_graph(kw, bias):
    g = Graph()
    x = g.parameter("f16", [-1, kw.get("K", 256)])
    root = simple_matmul(g, x, **kw)
    if bias is not None:
        root = g.add(root, g.constant(*bias))
    return g, x, root


def block_model(H=512, I=1024):
    """q / k / v reading the same activations (with bias Adds), gate and up with Swish and Multiply, and a down
    projection, each group on a Parameter of its own.  Returns (g, dict of named nodes)."""
    g = Graph()
    x = g.parameter("f16", [-1, H])
    q = g.add(simple_matmul(g, x, N=512, K=H, w_type="u4"), g.constant("f16", [512]))
    k = g.add(simple_matmul(g, x, N=128, K=H, w_type="u4"), g.constant("f16", [128]))
    v = g.add(simple_matmul(g, x, N=128, K=H, w_type="u4"), g.constant("f16", [128]))
    x2 = g.parameter("f16", [-1, H])
    gate = simple_matmul(g, x2, N=I, K=H, w_type="i4", zp=False)
    up = simple_matmul(g, x2, N=I, K=H, w_type="i4", zp=False)
    act = g.multiply(g.swish(gate), up)
    x3 = g.parameter("f16", [-1, I])
    down = simple_matmul(g, x3, N=H, K=I, w_type="i4", zp=False)
    for r in (q, k, v, act, down):
        g.result(r)
    return g, dict(x=x, x2=x2, x3=x3, q=q, k=k, v=v, gate=gate, up=up, act=act, down=down)


def mlp_model(H=512, I=1024, w_type="i4", zp=False, down_bias=True):
    """gate and up over one Parameter, Swish(gate) * up, and the down projection that alone reads it (with a bias
    Add): the subgraph the reference's MLPFusionPass matches.  Returns (g, x, root)."""
    g = Graph()
    x = g.parameter("f16", [-1, H])
    gate = simple_matmul(g, x, N=I, K=H, w_type=w_type, zp=zp)
    up = simple_matmul(g, x, N=I, K=H, w_type=w_type, zp=zp)
    down = simple_matmul(g, g.multiply(g.swish(gate), up), N=H, K=I, w_type=w_type, zp=zp)
    if down_bias:
        down = g.add(down, g.constant("f16", [H]))
    g.result(down)
    return g, x, down


def gather_graph(case, compressed=False, bias=None):
    """The reference's GatherMatmul test graph with the indices as a Parameter; bias: None, "shared" ([N]) or
    "per_expert" ([E, N]).  Returns (g, a, idx, root)."""
    g = Graph()
    a = g.parameter("f32", case["in_shape"])
    idx = g.parameter("i32", case["index_shape"])
    E, N = case["wei_shape"][0], case["wei_shape"][1]
    K = case["wei_shape"][2] * (case["wei_shape"][3] if case["grouped"] else 1)
    b_const = None if bias is None else g.constant("f32", [E, N] if bias == "per_expert" else [N])
    if compressed:
        sz = case["scale_zp_shape"][:-1] if case["grouped"] else case["scale_zp_shape"]
        root = g.gather_matmul_compressed(a, g.constant(case["type"], [E, N, K]), idx, g.constant("f32", sz),
                                          g.constant(case["type"], sz), bias=b_const)
    else:
        b = expert_weights(g, case["type"], case["wei_shape"], case["scale_zp_shape"], case["grouped"])
        root = g.gather_matmul(a, b, idx, bias=b_const)
    return g, a, idx, root


GATHER_FORMS = {"subgraph": (False, None), "compressed_per_expert_bias": (True, "per_expert"),
                "subgraph_shared_bias": (False, "shared")}


# ---- data ------------------------------------------------------------------------------------------------------

def _count(g, i):
    s = g.shape(i)
    return int(np.prod(s)) if len(s) else 1


def fill_constants(g, rng, K, weights, scales, zero_points=-1, bias=-1):
    """Seeded data for the Constants in these roles (node indices; -1 = absent), in OpenVINO's packing: weights any
    value of their type, scales sized so that outputs are of order one for unit-variance activations, zero-points
    inside the weights' range (integers also where the Constant is real-typed), bias of order one."""
    wt = _TYPE[g.nodes[weights].type]
    four = wt in ("u4", "i4")
    n = _count(g, weights)
    g.set_data(weights, rng.integers(0, 256, (n + 1) // 2 if four else n, dtype=np.uint8))
    st = _TYPE[g.nodes[scales].type]
    base = 3.5 / ((16 if four else 256) * math.sqrt(K))
    g.set_data(scales, (base * rng.uniform(0.5, 1.5, _count(g, scales))).astype(_NP[st]))
    if zero_points >= 0:
        zt = _TYPE[g.nodes[zero_points].type]
        zn = _count(g, zero_points)
        top = 16 if four else 256
        if zt == "u4":
            v = rng.integers(0, 16, zn + (zn & 1), dtype=np.uint8)
            packed = (v[0::2] | (v[1::2] << 4)).astype(np.uint8)
            if zn & 1:
                packed[-1] &= 15
            g.set_data(zero_points, packed)
        elif zt == "u8":
            g.set_data(zero_points, rng.integers(0, top, zn, dtype=np.uint8))
        else:
            g.set_data(zero_points, rng.integers(0, top, zn).astype(_NP[zt]))
    if bias >= 0:
        bt = _TYPE[g.nodes[bias].type]
        g.set_data(bias, rng.normal(0.0, 0.5, _count(g, bias)).astype(_NP[bt]))


def fill_fold(g, f, rng):
    """f: a Fold or a GatherFold"""
    fill_constants(g, rng, int(f.desc.K), f.weights, f.scales, f.zero_points, f.bias)
