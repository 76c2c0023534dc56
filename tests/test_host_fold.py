"""Graph-side host code under AddressSanitizer and UBSan, and its constant handling against numpy: the graphs of
the reference's tests and builders (tests/fold_graphs.py over tests/golden/fold_cases.json), with seeded Constant
bytes, are written to a case file; tests/host/fold_check.cpp -- built here with g++ from fold.cpp and fold_data.cpp --
runs the matchers and the step from Constants to the arrays ovfcc_weights_create takes, on exactly sized heap
blocks.  Checked: no sanitizer report; the folds equal what the shipped library returns through ctypes; every array
equals an independent numpy reading of the same Constant (slices of batched expert Constants, nibble re-packing,
f32 -> f16 rounding, real zero-points -> u8); and the weight matrix the arrays describe, dequantised, equals the value
of the MatMul's weight input in the unfused graph (tests/graph_eval.py).  No GPU."""
import ctypes
import os
import shutil
import struct
import subprocess

import numpy as np
import pytest

from fold_graphs import (CASES, GATHER_FORMS, VARIANTS, block_model, builder_graph, convert_fc_graph, fill_fold,
                         gather_graph, grouped_matmul_graph, mlp_model, moe_block, simple_matmul, transposed_graph, variant_graph)
from graph_eval import Evaluator, decode_constant
from openvino_amd import _lib
from openvino_amd.graph import Graph

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_TYPE = {v: k for k, v in _lib.TYPE.items()}
MATCH, GATHER, GROUPED, MOE, MODEL = range(5)


def same_struct(a, b, path=""):
    for name, ctype in a._fields_:
        x, y = getattr(a, name), getattr(b, name)
        if isinstance(x, ctypes.Structure):
            same_struct(x, y, path + name + ".")
        elif isinstance(x, ctypes.Array):
            assert list(x) == list(y), path + name
        else:
            assert x == y, (path + name, x, y)


# ---- the cases -----------------------------------------------------------------------------------------------

def special_scales_graph():
    """f32 scales whose rounding to f16 meets every branch: ties, subnormal halves, overflow, signed zeros."""
    g = Graph()
    x = g.parameter("f16", [-1, 256])
    root = simple_matmul(g, x, N=64, K=256, scale_type="f32")
    return g, x, root


SPECIAL = np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 70000.0, -65520.0, 1e-8, 2.0 ** -25,
                    np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -24, 1.5 * 2.0 ** -24, 2.5 * 2.0 ** -24,
                    2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, 2.0 ** -14 - 2.0 ** -24, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11,
                    1 + 2.0 ** -11 + 2.0 ** -20, 2 - 2.0 ** -11, 2 - 2.0 ** -12, np.inf, -np.inf, 3.1415927, 1e-5, 6e-5,
                    6.1e-5, 0.33333334, 1023.75, 2047.5], np.float32)


def all_cases():
    """(name, kind, graph, root, the nodes whose unfused value the arrays must reproduce)"""
    out = []
    for p in CASES["convert_fc_to_compressed"]:
        for root_op in ("fully_connected", "matmul"):
            g, x, root = convert_fc_graph(p, root_op)
            out.append((f"convert_fc {root_op} {p}", MATCH, g, root))
    for p in CASES["transposed_constants"]:
        g, x, root = transposed_graph(p)
        out.append((p["name"], MATCH, g, root))
    for p in CASES["builders"]:
        g, x, root = builder_graph(p)
        out.append((f"builder {p}", MATCH, g, root))
    for name, kw, bias in VARIANTS:
        g, x, root = variant_graph(kw, bias)
        out.append((name, MATCH, g, root))
    g, x, root = special_scales_graph()
    out.append(("special_scales", MATCH, g, root))
    for case in CASES["convert_gather_matmul_to_compressed"]:
        small = dict(case, wei_shape=[min(case["wei_shape"][0], 9)] + case["wei_shape"][1:],
                     scale_zp_shape=[min(case["scale_zp_shape"][0], 9)] + case["scale_zp_shape"][1:])
        for form in GATHER_FORMS:
            g, a, idx, root = gather_graph(small, *GATHER_FORMS[form])
            out.append((f"gather {form} {small}", GATHER, g, root))
    gmm = CASES["grouped_matmul_compressed"]
    for shape in gmm["shapes"]:
        for wt in gmm["weights_precisions"]:
            for zp in gmm["zero_points"]:
                if shape.get("corner") and wt in ("u4", "i4"):
                    continue
                g, a, offsets, root = grouped_matmul_graph(shape, wt, zp, -1)
                out.append((f"grouped {shape} {wt} {zp}", GROUPED, g, root))
    for compressed in (False, True):
        g = Graph()
        root = moe_block(g, "swish", compressed, 3, 256, 384, 2, [2, -1, 256])[0]
        out.append((f"moe compressed={compressed}", MOE, g, root))
    g, _ = block_model()
    out.append(("block model", MODEL, g, -1))
    g, _, _ = mlp_model()
    out.append(("mlp model", MODEL, g, -1))
    return out


def library_folds(kind, g, root):
    if kind == MATCH:
        return [g.fold_match(root)]
    if kind == GATHER:
        return [g.fold_gather_matmul(root)]
    if kind == GROUPED:
        return [g.fold_grouped_matmul(root)]
    if kind == MOE:
        m = g.fold_moe(root)
        return [m.gate, m.up, m.down]
    return g.fold_model()[0]


# ---- reading the driver's output --------------------------------------------------------------------------------

class Reader:
    def __init__(self, blob):
        self.b, self.at = blob, 0

    def i32(self):
        v = struct.unpack_from("<i", self.b, self.at)[0]
        self.at += 4
        return v

    def struct(self, cls):
        v = cls.from_buffer_copy(self.b, self.at)
        self.at += ctypes.sizeof(cls)
        return v

    def array(self, dtype):
        n = struct.unpack_from("<q", self.b, self.at)[0]
        self.at += 8
        v = np.frombuffer(self.b, np.uint8, n, self.at).copy().view(dtype)
        self.at += n
        return v

    def record(self):
        rc = self.i32()
        assert rc == _lib.OK, rc
        return dict(desc=self.struct(_lib.FcDesc), w=self.array(np.uint8), s=self.array(np.float16),
                    z=self.array(np.uint8), b=self.array(np.float16))


# ---- the independent reading of the same Constants ---------------------------------------------------------------

def flat(g, i):
    """Every element a Constant's bytes hold (for 4-bit types that may be one more than its shape has)."""
    t = _TYPE[g.nodes[i].type]
    n = g.data[i].size * 2 if t in ("u4", "i4") else g.data[i].size // {"u8": 1, "i8": 1, "f16": 2, "f32": 4}[t]
    return decode_constant(t, [n], g.data[i])


def half_bits(v32):
    with np.errstate(over="ignore"):
        return np.asarray(v32, np.float32).astype(np.float16).view(np.uint16)


def check_record(name, g, f, rec, expert, n_experts):
    d = rec["desc"]
    N, K, G = int(d.N), int(d.K), int(d.group_size)
    ng, four = K // G, _TYPE[d.w_type] in ("u4", "i4")
    per = N * ng
    # weights: the expert's N K elements, in order; an odd 4-bit count ends in a zero nibble
    w_all = flat(g, f.weights)
    got_w = decode_constant(_TYPE[d.w_type], [N * K], rec["w"])
    assert rec["w"].size == ((N * K + 1) // 2 if four else N * K), name
    assert np.array_equal(got_w, w_all[expert * N * K:(expert + 1) * N * K]), name
    if four and (N * K) & 1:
        assert rec["w"][-1] >> 4 == 0, name
    # scales: f16 as stored, f32 rounded to nearest even; one element replicated
    s_all = flat(g, f.scales)
    want = np.full(per, s_all[0]) if f.scale_broadcast else s_all[expert * per:(expert + 1) * per]
    assert rec["s"].size == per, name
    nan = np.isnan(want)
    assert np.array_equal(rec["s"].view(np.uint16)[~nan], half_bits(want)[~nan]), name
    assert np.all(np.isnan(rec["s"][nan])), name
    # zero-points
    if f.zero_points >= 0:
        zt = _TYPE[g.nodes[f.zero_points].type]
        count_z = 1 if d.zp_scalar else per
        first = 0 if d.zp_scalar else expert * per
        if zt in ("f16", "f32"):
            z_all = flat(g, f.zero_points)
            assert d.zp_type == _lib.TYPE["u8"] and f.zp_from_real == 1
            got_z = rec["z"].astype(np.float64)
        else:
            z_all = flat(g, f.zero_points)
            assert d.zp_type == _lib.TYPE[zt]
            got_z = decode_constant(zt, [count_z], rec["z"])
            assert rec["z"].size == ((count_z + 1) // 2 if zt == "u4" else count_z), name
            if zt == "u4" and count_z & 1:
                assert rec["z"][-1] >> 4 == 0, name
        assert np.array_equal(got_z[:count_z], z_all[first:first + count_z]), name
    else:
        assert rec["z"].size == 0 and d.zp_type == _lib.NONE, name
    # bias
    if f.bias >= 0:
        b_all = flat(g, f.bias)
        per_expert = getattr(f, "bias_per_expert", 0)
        want_b = b_all[expert * N:(expert + 1) * N] if per_expert else b_all[:N]
        assert np.array_equal(rec["b"].view(np.uint16), half_bits(want_b)), name
        assert d.bias_type == _lib.F16
    else:
        assert rec["b"].size == 0, name


def dequantised(rec):
    """The [N, K] matrix the arrays describe: (W - zp) * scale, groups along K; input-major arrays are [K, N]."""
    d = rec["desc"]
    N, K, G = int(d.N), int(d.K), int(d.group_size)
    ng = K // G
    im = bool(d.flags & _lib.W_INPUT_MAJOR)
    w = decode_constant(_TYPE[d.w_type], [K, N] if im else [N, K], rec["w"])
    s = rec["s"].astype(np.float64).reshape([ng, N] if im else [N, ng])
    if d.zp_type != _lib.NONE:
        z = decode_constant(_TYPE[d.zp_type], [1] if d.zp_scalar else ([ng, N] if im else [N, ng]), rec["z"])
    else:
        z = np.zeros(1)
    if im:
        w, s = w.T, s.T
        z = z.T if z.size > 1 else z
    wg = w.reshape(N, ng, G)
    zz = z.reshape(N, ng, 1) if z.size > 1 else z.reshape(1, 1, 1)
    return ((wg - zz) * s.reshape(N, ng, 1)).reshape(N, K)


def unfused_weights(g, ev, f):
    """Value of the weight input of the fold's MatMul / FullyConnected in the unfused graph, as [N, K]."""
    n = g.nodes[f.matmul]
    b = ev.value(int(n.inputs[1]))
    if n.op == _lib.OP["matmul"] and not n.transpose_b:
        b = b.T
    return b


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host compiler")
def test_matchers_and_constant_handling_under_sanitizers(tmp_path):
    exe = str(tmp_path / "fold_check")
    csrc = os.path.join(ROOT, "openvino_amd", "csrc")
    src = [os.path.join(ROOT, "tests", "host", "fold_check.cpp")] + [os.path.join(csrc, n) for n in
                                                                    ("fold.cpp", "fold_data.cpp", "plan.cpp", "repack.cpp")]
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-static-libasan", "-static-libubsan", "-pthread", "-I" + os.path.join(ROOT, "include"), "-I" + csrc,
           "-I" + os.path.join(ROOT, "tests", "host"), "-o", exe] + src
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr[-4000:]

    rng = np.random.default_rng(7700)
    cases = all_cases()
    expected = []
    blob = [struct.pack("<i", len(cases))]
    for name, kind, g, root in cases:
        folds = library_folds(kind, g, root)
        for f in folds:
            fill_fold(g, f, rng)
        if name == "special_scales":
            s = np.frombuffer(g.data[folds[0].scales].tobytes(), np.float32).copy()
            s[:SPECIAL.size] = SPECIAL
            s[SPECIAL.size:] = rng.integers(0, 2 ** 32, s.size - SPECIAL.size, dtype=np.uint32).view(np.float32)
            g.set_data(folds[0].scales, s)
        expected.append(folds)
        blob.append(struct.pack("<iii", kind, root, len(g.nodes)))
        blob += [bytes(n) for n in g.nodes]
        for i in range(len(g.nodes)):
            if i in g.data:
                blob += [struct.pack("<q", g.data[i].size), g.data[i].tobytes()]
            else:
                blob.append(struct.pack("<q", -1))
    case_file, out_file = str(tmp_path / "cases.bin"), str(tmp_path / "out.bin")
    with open(case_file, "wb") as fh:
        fh.write(b"".join(blob))
    env = {k: v for k, v in os.environ.items() if not k.startswith("OVFCC_")}
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0"
    run = subprocess.run([exe, case_file, out_file], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, (run.stdout[-4000:], run.stderr[-4000:])
    assert f"{len(cases)} cases" in run.stdout

    with open(out_file, "rb") as fh:
        rd = Reader(fh.read())
    checked = 0
    for (name, kind, g, root), folds in zip(cases, expected):
        assert rd.i32() == _lib.OK, name
        ev = Evaluator(g, {})
        if kind == MATCH:
            same_struct(rd.struct(_lib.Fold), folds[0], name + ": ")
            groups = [(folds[0], 1)]
        elif kind in (GATHER, GROUPED):
            same_struct(rd.struct(_lib.GatherFold), folds[0], name + ": ")
            groups = [(folds[0], int(folds[0].n_experts))]
        elif kind == MOE:
            same_struct(rd.struct(_lib.MoeFold), g.fold_moe(root), name + ": ")
            groups = [(f, int(f.n_experts)) for f in folds]
        else:
            n = rd.i32()
            assert n == len(folds)
            for f in folds:
                same_struct(rd.struct(_lib.Fold), f, name + ": ")
            lib_fused = g.fold_model()[1]
            assert rd.i32() == len(lib_fused)
            for u in lib_fused:
                same_struct(rd.struct(_lib.Fused), u, name + ": ")
            groups = [(f, 1) for f in folds]
        for f, n_experts in groups:
            batched = n_experts > 1 or kind in (GATHER, GROUPED, MOE)
            for e in range(n_experts):
                rec = rd.record()
                check_record(f"{name} expert {e}", g, f, rec, e, n_experts)
                if name == "special_scales":
                    continue
                got = dequantised(rec)
                if batched:
                    node = g.nodes[f.root]
                    want = ev.value(int(node.inputs[1]))
                    if node.op in (_lib.OP["gather_matmul_compressed"], _lib.OP["grouped_matmul_compressed"]):
                        rest = [int(node.inputs[k]) for k in range(node.n_inputs)]
                        scale, zp = (rest[4], rest[5]) if node.op == _lib.OP["gather_matmul_compressed"] else (None, None)
                        want = ev.decompress(want, scale, zp)
                    want = want[e]
                else:
                    want = unfused_weights(g, ev, f)
                # f32 scales are rounded to f16 on the way: half an ulp relative; f16 scales give the same matrix
                f32_scales = _TYPE[g.nodes[f.scales].type] == "f32"
                if f32_scales:
                    assert np.allclose(got, want, rtol=2.0 ** -11, atol=0), name
                else:
                    assert np.array_equal(got, want), name
                checked += 1
    assert rd.at == len(rd.b)
    assert checked > 300
