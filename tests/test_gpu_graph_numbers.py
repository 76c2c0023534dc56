"""From a graph to numbers: the reference's own test and builder graphs (tests/golden/fold_cases.json), as plain
nodes with seeded Constant bytes, go through the matchers, through ovfcc_fold_weights_create /
ovfcc_fold_expert_weights_create and through the kernels; the result is compared with a numpy evaluation of the
UNFUSED graph (Convert -> Subtract -> Multiply -> Reshape -> [Transpose] -> MatMul [-> Add], node by node in
float64: tests/graph_eval.py), which knows nothing of the fold.  What the reference's functional tests do with the
TEMPLATE interpreter (src/plugins/intel_cpu/tests/functional/custom/subgraph_tests/src/x64/
matmul_weights_decompression.cpp:37-120 over weights_decompression_builders.cpp:42-205), at the same bounds as the
other parity tests: rel-L2 <= 1e-3 and max-abs <= 2e-2 sqrt(K / 4096) plus half an f16 ulp of the largest output."""
import sys

import numpy as np
import pytest

from fold_graphs import (CASES, GATHER_FORMS, VARIANTS, block_model, builder_graph, convert_fc_graph, fill_fold,
                         gather_graph, grouped_matmul_graph, mlp_model, moe_block, simple_matmul, transposed_graph, variant_graph)
from graph_eval import Evaluator
from openvino_amd import _lib, fc
from openvino_amd._lib import OvfccError
from openvino_amd.graph import Graph
from parity import REL_L2_MAX, max_abs_limit

pytestmark = pytest.mark.gpu
GMM = CASES["grouped_matmul_compressed"]


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def ids(rows, keys):
    return ["-".join(str(r[k]) for k in keys) for r in rows]


@pytest.fixture(scope="module")
def dev():
    d = fc.Device(0)
    yield d
    d.close()


@pytest.fixture()
def req(dev):
    r = fc.InferRequest(dev)
    yield r
    r.close()


def activations(rng, shape):
    """f16-representable values, so that a host-side f32 -> f16 conversion of the activations changes nothing"""
    return rng.normal(0.0, 1.0, shape).astype(np.float16)


def check(y, ref, K, what, scale=1.0):
    y, ref = np.asarray(y, np.float64), np.asarray(ref, np.float64)
    assert y.shape == ref.shape, (what, y.shape, ref.shape)
    assert np.all(np.isfinite(y)), what
    rl2 = float(np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30))
    mab = float(np.max(np.abs(y - ref))) if y.size else 0.0
    limit = scale * max_abs_limit(K) + (float(np.max(np.abs(ref))) if ref.size else 0.0) * 2.0 ** -11
    assert rl2 <= scale * REL_L2_MAX, f"{what}: rel-L2 {rl2:.3e}"
    assert mab <= limit, f"{what}: max-abs {mab:.3e} > {limit:.3e}"


def run_fold(dev, req, g, x, root, rng, rows, what):
    """Match at root, fill the Constants the fold names, create, infer, compare with the unfused graph."""
    f = g.fold_match(root)
    fill_fold(g, f, rng)
    K = int(f.desc.K)
    xs = g.shape(x)
    shape = [rows if d < 0 else d for d in xs[:-1]] + [K]
    X = activations(rng, shape)
    ref = Evaluator(g, {x: X}).value(root)
    w = g.create_weights(dev, f)
    try:
        say(f"{what}: N={f.desc.N} K={K} G={f.desc.group_size} flags={f.desc.flags} rows={X.size // K}")
        y = req.infer(w, X.reshape(-1, K))
        assert y.dtype == (np.float32 if f.desc.out_type == _lib.F32 else np.float16)
        check(y.reshape(ref.shape), ref, K, what)
    finally:
        w.close()
    return f


@pytest.mark.parametrize("p", CASES["builders"], ids=ids(CASES["builders"], ("type", "weights_shape", "group", "transpose_weights", "zp")))
@pytest.mark.parametrize("rows", [1, 37])
def test_builder_subgraphs(dev, req, p, rows):
    g, x, root = builder_graph(p)
    run_fold(dev, req, g, x, root, np.random.default_rng(9000 + rows), rows, f"builder {p}")


@pytest.mark.parametrize("p", CASES["convert_fc_to_compressed"],
                         ids=ids(CASES["convert_fc_to_compressed"], ("type", "with_zp", "grouped", "wei_shape")))
@pytest.mark.parametrize("root_op", ["fully_connected", "matmul"])
def test_convert_fc_to_compressed_rows(dev, req, p, root_op):
    """f32 graphs: scales stored in f32 (rounded to f16 by the library), f32 output."""
    g, x, root = convert_fc_graph(p, root_op)
    f = run_fold(dev, req, g, x, root, np.random.default_rng(9100), 7, f"{root_op} {p}")
    assert f.desc.out_type == _lib.F32 and f.activations_f32 == 1


@pytest.mark.parametrize("p", CASES["transposed_constants"], ids=[p["name"] for p in CASES["transposed_constants"]])
def test_rank1_and_rank0_constants_under_a_transpose(dev, req, p):
    g, x, root = transposed_graph(p)
    f = run_fold(dev, req, g, x, root, np.random.default_rng(9200), 3, p["name"])
    assert f.desc.flags == _lib.W_INPUT_MAJOR


@pytest.mark.parametrize("name,kw,bias", VARIANTS, ids=[v[0] for v in VARIANTS])
def test_fold_variants(dev, req, name, kw, bias):
    g, x, root = variant_graph(kw, bias)
    f = run_fold(dev, req, g, x, root, np.random.default_rng(9300), 9, name)
    assert (f.bias >= 0) == (bias is not None)
    assert f.zp_from_real == int(kw.get("zp_type") in ("f16", "f32"))


def test_constant_checks(dev):
    """What the creation refuses: a real-typed zero-point that is no integer or out of range, missing data, data of
    a Constant whose shape no longer fits the descriptor."""
    g = Graph()
    x = g.parameter("f16", [-1, 256])
    root = simple_matmul(g, x, zp_type="f16")
    f = g.fold_match(root)
    rng = np.random.default_rng(9400)
    fill_fold(g, f, rng)
    good = g.data[f.zero_points].copy()
    for bad in (3.5, -1.0, 256.0, float("nan")):
        z = good.view(np.float16).copy()
        z[5] = bad
        g.set_data(f.zero_points, z)
        with pytest.raises(OvfccError) as err:
            g.create_weights(dev, f)
        assert err.value.code == _lib.EUNSUPPORTED, bad
    g.set_data(f.zero_points, good)
    g.create_weights(dev, f).close()
    del g.data[f.scales]
    with pytest.raises(OvfccError) as err:
        g.create_weights(dev, f)
    assert err.value.code == _lib.EINVAL
    fill_fold(g, f, rng)
    g.nodes[f.weights].dims[0] += 1
    with pytest.raises(OvfccError) as err:
        g.create_weights(dev, f)
    assert err.value.code == _lib.EINVAL


def test_model_with_siblings_and_a_gated_unit(dev, req):
    """One block as fold_model groups it: q / k / v reading the same activations become one node (horizontal fusion),
    gate and up with Swish and Multiply become one node with a gated linear unit, the down projection stays alone.
    Every group is created from the graph's Constants and checked against the unfused graph at its own roots."""
    rng = np.random.default_rng(9500)
    H, I = 512, 1024
    g, n = block_model(H, I)
    x, x2, x3, gate, up = n["x"], n["x2"], n["x3"], n["gate"], n["up"]
    folds, fused = g.fold_model()
    assert sorted(u.kind for u in fused) == [_lib.FUSED_SINGLE, _lib.FUSED_CONCAT, _lib.FUSED_GLU]
    for f in folds:
        fill_fold(g, f, rng)
    M = 11
    feeds = {x: activations(rng, (M, H)), x2: activations(rng, (M, H)), x3: activations(rng, (M, I))}
    ev = Evaluator(g, feeds)
    for u in fused:
        parts = [g.create_weights(dev, folds[u.parts[i]]) for i in range(u.n_parts)]
        f0 = folds[u.parts[0]]
        X = feeds[f0.activations]
        try:
            if u.kind == _lib.FUSED_GLU:
                node = fc.CompressedWeights.glu(parts[0], parts[1], {1: "swish", 2: "gelu", 3: "gelu_tanh"}[u.glu_type])
                say(f"gated unit over folds {list(u.parts[:2])}")
                y = req.infer(node, X)
                # the unit can amplify the error of the two products underneath: |d out| <= d (1.13 |up| + |gate|)
                amp = 2.13 * max(1.0, float(np.max(np.abs(ev.value(gate)))), float(np.max(np.abs(ev.value(up)))))
                check(y, ev.value(u.root), H, "gated unit", scale=amp)
                node.close()
            elif u.kind == _lib.FUSED_CONCAT:
                node = fc.CompressedWeights.concat(parts)
                say(f"siblings {[int(folds[u.parts[i]].root) for i in range(u.n_parts)]}")
                y = req.infer(node, X)
                col = 0
                for i in range(u.n_parts):
                    f = folds[u.parts[i]]
                    check(y[:, col:col + f.desc.N], ev.value(f.root), H, f"sibling {i}")
                    col += int(f.desc.N)
                assert col == y.shape[1]
                node.close()
            else:
                y = req.infer(parts[0], X)
                check(y, ev.value(f0.root), int(f0.desc.K), "single node")
        finally:
            for p in parts:
                p.close()


@pytest.mark.parametrize("w_type,zp", [("i4", False), ("u4", True), ("u8", True)])
@pytest.mark.parametrize("rows", [1, 3, 40])
def test_mlp_block_from_the_graph(dev, req, w_type, zp, rows):
    """gate / up, Swish, Multiply and the down projection with its bias fold into one MLP group; the node made of it
    (gated unit, then ovfcc_weights_mlp) reproduces the unfused graph, and so does its blob after export and import."""
    rng = np.random.default_rng(9550)
    H, I = 512, 1024
    g, x, root = mlp_model(H, I, w_type, zp)
    folds, fused = g.fold_model()
    (u,) = fused
    assert u.kind == _lib.FUSED_MLP and u.root == root
    for f in folds:
        fill_fold(g, f, rng)
    X = activations(rng, (rows, H))
    ev = Evaluator(g, {x: X})
    ref = ev.value(root)
    gate, up, down = (g.create_weights(dev, folds[u.parts[i]]) for i in range(3))
    unit = fc.CompressedWeights.glu(gate, up, "swish")
    node = fc.CompressedWeights.mlp(unit, down)
    twin = fc.CompressedWeights.import_blob(dev, node.export_blob())
    try:
        say(f"mlp from graph {w_type} zp={zp} rows={rows}")
        y = req.infer(node, X)
        mid = ev.value(folds[u.parts[2]].activations)
        amp = 2.13 * max(1.0, float(np.max(np.abs(ev.value(folds[u.parts[0]].root)))),
                         float(np.max(np.abs(ev.value(folds[u.parts[1]].root)))))
        check(y, ref, I, "mlp", scale=amp * max(1.0, float(np.sqrt(np.mean(mid * mid)))))
        y2 = req.infer(twin, X)
        assert y2.shape == y.shape and np.array_equal(y2.view(np.uint8), y.view(np.uint8))
        assert twin.device_bytes == node.device_bytes
    finally:
        for w in (gate, up, down, unit, node, twin):
            w.close()


def gather_case(case, rng, form):
    g, a, idx, root = gather_graph(case, *GATHER_FORMS[form])
    f = g.fold_gather_matmul(root)
    fill_fold(g, f, rng)
    return g, a, idx, root, f


GATHER = CASES["convert_gather_matmul_to_compressed"]


@pytest.mark.parametrize("case", GATHER, ids=lambda c: f"{c['type']}-{'grouped' if c['grouped'] else 'plain'}-{c['wei_shape']}")
@pytest.mark.parametrize("form", list(GATHER_FORMS))
def test_gather_matmul_experts_from_batched_constants(dev, req, case, form):
    """Expert slices of batched Constants.  The routed entry points want output rows of a multiple of 16 bytes, so
    the reference's N = 5 and N = 1 become 40 and 8 here (the slices that start in the middle of a byte, which odd N
    gives, are covered by the host test); 16 of its experts are kept."""
    rng = np.random.default_rng(9600)
    case = dict(case, wei_shape=[16, 8 * case["wei_shape"][1]] + case["wei_shape"][2:],
                scale_zp_shape=[16, 8 * case["scale_zp_shape"][1]] + case["scale_zp_shape"][2:])
    g, a, idx, root, f = gather_case(case, rng, form)
    assert f.bias_per_expert == int(GATHER_FORMS[form][1] == "per_expert")
    M, top_k = case["index_shape"]
    A = activations(rng, [top_k if d < 0 else d for d in case["in_shape"]])
    indices = rng.integers(0, f.n_experts, (M, top_k)).astype(np.int32)
    ref = Evaluator(g, {a: A, idx: indices}).value(root)
    experts = [g.create_expert_weights(dev, f, e) for e in range(f.n_experts)]
    try:
        say(f"gather {form} {case['type']} E={f.n_experts} N={f.desc.N} K={f.desc.K} G={f.desc.group_size}")
        y = req.gather_matmul(experts, A, indices)
        check(y, ref, int(f.desc.K), f"gather {form}")
    finally:
        for w in experts:
            w.close()
    with pytest.raises(OvfccError):
        g.create_expert_weights(dev, f, f.n_experts)


@pytest.mark.parametrize("shape", GMM["shapes"], ids=lambda c: f"A{c['a_shape']}xB{c['b_shape']}")
@pytest.mark.parametrize("wt", GMM["weights_precisions"])
@pytest.mark.parametrize("zp", GMM["zero_points"])
def test_grouped_matmul_groups_from_batched_constants(dev, req, shape, wt, zp):
    """The reference's functional test of GroupedMatMulCompressed at one scale per channel (its groups of 16 inputs
    are refused by the matcher); the corner shape K = 77, N = 123 with 8-bit weights."""
    if shape.get("corner") and wt in ("u4", "i4"):
        pytest.skip("odd K needs 8-bit weights here")
    rng = np.random.default_rng(9700)
    g, a, offsets, root = grouped_matmul_graph(shape, wt, zp, -1)
    f = g.fold_grouped_matmul(root)
    fill_fold(g, f, rng)
    G_, N, K = shape["b_shape"]
    groups = [g.create_expert_weights(dev, f, e) for e in range(G_)]
    try:
        say(f"grouped {wt} zp={zp} A{shape['a_shape']} B{shape['b_shape']}")
        if offsets is not None:
            counts = rng.integers(0, 9, G_)
            counts[rng.integers(0, G_)] = 0
            ends = np.cumsum(counts).astype(np.int32)
            A = activations(rng, (int(ends[-1]), K))
            ref = Evaluator(g, {a: A, offsets: ends}).value(root)
            y = req.grouped_matmul(groups, A, ends)
        else:
            A = activations(rng, (G_, 5, K))
            ref = Evaluator(g, {a: A}).value(root)
            y = req.grouped_matmul(groups, A)
        check(y, ref, K, "grouped")
    finally:
        for w in groups:
            w.close()


@pytest.mark.parametrize("act", CASES["moe_block"]["activations"])
@pytest.mark.parametrize("compressed", [False, True], ids=["subgraphs", "compressed_nodes"])
def test_moe_block_from_the_graph(dev, req, act, compressed):
    """build_3gemm_bgm_model at a small size: the block fold names the three expert layers; gate and up slices become
    one node with a gated linear unit per expert, and the one-call block is compared with the unfused graph (three
    GatherMatmuls, activation, Multiply, routing Multiply, ReduceSum, Reshape)."""
    rng = np.random.default_rng(9800)
    E, H, I, top_k, M = 5, 256, 512, 2, 6
    g = Graph()
    root, hidden, routing, idx, _ = moe_block(g, "gelu" if act == "gelu_erf" else act, compressed, E, H, I, top_k, [2, -1, H])
    m = g.fold_moe(root)
    for f in (m.gate, m.up, m.down):
        fill_fold(g, f, rng)
    X = activations(rng, (2, M // 2, H))
    R = rng.dirichlet(np.ones(top_k), M).astype(np.float16)
    indices = np.stack([rng.permutation(E)[:top_k] for _ in range(M)]).astype(np.int32)
    ev = Evaluator(g, {hidden: X, routing: R, idx: indices})
    ref = ev.value(root)
    kind = {1: "swish", 2: "gelu", 3: "gelu_tanh"}[m.glu_type]
    gate_up, down = [], []
    try:
        for e in range(E):
            ga, up = g.create_expert_weights(dev, m.gate, e), g.create_expert_weights(dev, m.up, e)
            gate_up.append(fc.CompressedWeights.glu(ga, up, kind))
            ga.close()
            up.close()
            down.append(g.create_expert_weights(dev, m.down, e))
        say(f"moe block {act} compressed={compressed}")
        amp = 2.13 * max(1.0, float(np.max(np.abs(ev.value(m.gate.root)))), float(np.max(np.abs(ev.value(m.up.root)))))
        y = req.moe(gate_up, down, X.reshape(M, H), R, indices)
        check(y.reshape(ref.shape), ref, I, f"moe {act}", scale=2 * amp)
    finally:
        for w in gate_up + down:
            w.close()
