"""GPU parity of nodes that allow per-token int8 activations (W8A8) against the CPU oracle of that arithmetic: the
integer part is exact, so the only differences are the f32 epilogue and the output rounding."""
import sys

import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc
from parity import check_parity, oracle_y

pytestmark = pytest.mark.gpu

T = {"u8": 3, "i8": 4}


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


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


def dq_reference(oracle, c, x=None):
    zp = None if c.zp is None else c.zp.astype(np.float32)
    return oracle.fc_dynquant_reference(c.x if x is None else x, c.w, T[c.w_type], c.scale, zp, c.bias, N=c.N, K=c.K)


@pytest.mark.parametrize("wt,zt,N,K,bias,out", [("u8", "u8", 256, 512, True, "f32"), ("u8", "none", 512, 384, False, "f16"),
                                                ("i8", "none", 256, 1024, True, "f16"), ("u8", "u8", 768, 128, False, "f32")])
def test_dynquant_prefill_matches_integer_oracle(oracle, dev, req, monkeypatch, wt, zt, N, K, bias, out):
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")   # the policy keeps grids this small on the f16 kernels
    say(f"dynquant {wt}/{zt} N={N} K={K} bias={bias} out={out}")
    c = datagen.make_case(1100, 300, K, N, wt, K, zt, with_bias=bias)
    c.x[5] = 0                                    # an all-zero row: the clamp decides its scale
    c.x[6] *= 40                                  # a row with a large range
    w = fc.CompressedWeights.from_case(dev, c, output_type=out, dynamic_quantization=True)
    try:
        for M in (49, 128, 129, 300):
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_prefill_i8_w8", info
            ref = dq_reference(oracle, c, c.x[:M])
            if out == "f32":                      # exact integers, f32 epilogue: a few ulps of f32
                assert oracle.rel_l2(y, ref) < 1e-6, (M, oracle.rel_l2(y, ref))
                assert np.all(np.abs(y - ref) <= np.abs(ref) * 1e-6 + 1e-6)
            else:
                assert np.array_equal(y.view(np.uint16), ref.astype(np.float16).view(np.uint16)) or \
                    np.mean(y.view(np.uint16) != ref.astype(np.float16).view(np.uint16)) < 1e-3   # f32 ties
                assert oracle.rel_l2(y.astype(np.float32), ref) < 5e-4
            # against the unquantised arithmetic: the quantisation noise and nothing else
            plain = oracle_y(oracle, c, x=c.x[:M])
            assert oracle.rel_l2(y.astype(np.float32), plain) < 3e-2
            assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
        # decode row counts and a forced decode kernel compute in f16: the flag is a permission
        y = req.infer(w, c.x[:32])
        assert req.last_kernel()["kernel"] == _lib.KERNEL_DECODE
        check_parity(oracle, y, oracle_y(oracle, c, x=c.x[:32]), K, "decode rows", output_rounding_slack=True)
    finally:
        w.close()


def test_dynquant_flag_without_a_kernel_is_ignored(oracle, dev, req, monkeypatch):
    """4-bit weights with groups of 64, 8-bit weights with grouped scales or a narrow node: the permission has no
    integer kernel to take effect in; nor does it take effect where the integer kernel's grid would leave most of the
    chip idle."""
    say("dynquant ignored")
    c = datagen.make_case(1111, 200, 512, 256, "u8", 512, "u8")
    w = fc.CompressedWeights.from_case(dev, c, dynamic_quantization=True)
    try:
        y = req.infer(w, c.x)
        assert req.last_kernel()["name"] != "fcc_prefill_i8_w8"
        check_parity(oracle, y, oracle_y(oracle, c), 512, "small grid", output_rounding_slack=True)
    finally:
        w.close()
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    for wt, zt, N, K, G in (("u4", "u4", 256, 512, 64), ("u4", "u8", 256, 512, 128), ("u8", "u8", 256, 512, 128),
                            ("u8", "u8", 128, 512, 512)):
        c = datagen.make_case(1110, 200, K, N, wt, G, zt)
        w = fc.CompressedWeights.from_case(dev, c, dynamic_quantization=True)
        try:
            y = req.infer(w, c.x)
            assert not req.last_kernel()["name"].startswith("fcc_prefill_i8")
            check_parity(oracle, y, oracle_y(oracle, c), K, f"{wt} G={G} N={N}", output_rounding_slack=True)
        finally:
            w.close()


def test_dynquant_llama70b_shape(oracle, dev, req):
    """Config 4's q/o projection (8192 -> 8192, u8 per-channel) at M = 1024 through the integer kernel, sampled rows."""
    say("dynquant 70B q/o")
    c = datagen.config4("qo", 1024)
    w = fc.CompressedWeights.from_case(dev, c, output_type="f32", dynamic_quantization=True)
    try:
        y = req.infer(w, c.x)
        assert req.last_kernel()["name"] == "fcc_prefill_i8_w8"
        pick = np.array([0, 1, 500, 777, 1023])
        ref = dq_reference(oracle, c, c.x[pick])
        assert oracle.rel_l2(y[pick], ref) < 1e-6
        plain = oracle_y(oracle, c, x=c.x[pick])
        r = oracle.rel_l2(y[pick], plain)
        say(f"   rel-L2 against the f16-activation oracle: {r:.2e}")
        assert r < 2e-2
    finally:
        w.close()


def test_dynquant_with_gated_linear_unit(oracle, dev, req, monkeypatch):
    """SwiGLU on top of the integer path: the unit applied to the integer oracle's gate and up halves."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    say("dynquant + glu")
    c = datagen.make_case(1120, 200, 512, 512, "u8", 512, "u8", with_bias=True)
    for kind, second in (("swish", False), ("gelu_tanh", True)):
        w = fc.CompressedWeights.from_case(dev, c, output_type="f32", glu=kind, glu_gate_second=second,
                                           dynamic_quantization=True)
        try:
            y = req.infer(w, c.x)
            assert req.last_kernel()["name"] == "fcc_prefill_i8_w8" and y.shape == (200, 256)
            ref = oracle.glu(dq_reference(oracle, c), {"swish": 1, "gelu_tanh": 3}[kind], second)
            assert oracle.rel_l2(y, ref) < 2e-6, oracle.rel_l2(y, ref)
        finally:
            w.close()


# ---- 4-bit weights with groups of 128 inputs (W4A8) ----

TN = {"none": 0, "u4": 1, "i4": 2, "u8": 3, "i8": 4}


def dq4_reference(oracle, c, x, act_group):
    return oracle.fc_dynquant_grouped_reference(x, c.w, TN[c.w_type], c.scale, c.zp, TN[c.zp_type], c.bias, N=c.N, K=c.K,
                                                group_size=c.group_size, act_group=act_group, zp_scalar=c.zp_scalar)


@pytest.mark.parametrize("mode", ["per_token", "per_group"])
@pytest.mark.parametrize("wt,zt,N,K,bias,out", [("u4", "u4", 256, 512, True, "f32"), ("u4", "none", 512, 384, False, "f16"),
                                                ("i4", "none", 256, 1024, True, "f32"), ("u4", "u4", 768, 128, False, "f32")])
def test_w4a8_prefill_matches_integer_oracle(oracle, dev, req, monkeypatch, mode, wt, zt, N, K, bias, out):
    """4-bit weights, scales and zero-points per 128 inputs, activations int8 per token or per row and group: the
    integer sums are exact, so against the oracle of the same arithmetic only the f32 sum over the groups (in k-block
    order on the GPU, in double in the oracle) and the output rounding differ."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")   # the policy keeps grids this small on the f16 kernels
    say(f"w4a8 {mode} {wt}/{zt} N={N} K={K} bias={bias} out={out}")
    c = datagen.make_case(1200, 300, K, N, wt, 128, zt, with_bias=bias)
    c.x[5] = 0
    c.x[6] *= 40
    c.x[7, 130:] *= 25                            # groups of very different range in one row
    w = fc.CompressedWeights.from_case(dev, c, output_type=out, dynamic_quantization=mode)
    name = "fcc_prefill_i8_w4_grouped" if mode == "per_group" else "fcc_prefill_i8_w4"
    try:
        for M in (49, 128, 129, 300):
            y = req.infer(w, c.x[:M])
            assert req.last_kernel()["name"] == name, req.last_kernel()
            ref = dq4_reference(oracle, c, c.x[:M], 128 if mode == "per_group" else K)
            tol = 2e-6 if out == "f32" else 5e-4
            assert oracle.rel_l2(y.astype(np.float32), ref) < tol, (M, oracle.rel_l2(y.astype(np.float32), ref))
            if out == "f32":
                assert np.all(np.abs(y - ref) <= 4e-6 * np.max(np.abs(ref)))
            plain = oracle_y(oracle, c, x=c.x[:M])
            assert oracle.rel_l2(y.astype(np.float32), plain) < 3e-2
            assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
        y = req.infer(w, c.x[:32])                # decode row counts compute in f16: the flag is a permission
        assert req.last_kernel()["kernel"] == _lib.KERNEL_DECODE
        check_parity(oracle, y, oracle_y(oracle, c, x=c.x[:32]), K, "decode rows", output_rounding_slack=True)
    finally:
        w.close()


def test_w4a8_scalar_zero_point_and_gated_linear_unit(oracle, dev, req, monkeypatch):
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    say("w4a8 scalar zp + glu")
    c = datagen.make_case(1210, 200, 512, 512, "u4", 128, "u4", with_bias=True)
    c.zp, c.zp_scalar = np.array([7], np.uint8), True
    for kind, second, mode in (("swish", False, "per_group"), ("gelu_tanh", True, "per_token")):
        w = fc.CompressedWeights.from_case(dev, c, output_type="f32", glu=kind, glu_gate_second=second,
                                           dynamic_quantization=mode)
        try:
            y = req.infer(w, c.x)
            assert req.last_kernel()["name"].startswith("fcc_prefill_i8_w4") and y.shape == (200, 256)
            full = dq4_reference(oracle, c, c.x, 128 if mode == "per_group" else c.K)
            ref = oracle.glu(full, {"swish": 1, "gelu_tanh": 3}[kind], second)
            assert oracle.rel_l2(y, ref) < 4e-6, oracle.rel_l2(y, ref)
        finally:
            w.close()


@pytest.mark.parametrize("mode", ["per_token", "per_group"])
def test_w4a8_llama8b_prefill_shape(oracle, dev, req, mode):
    """Config 3's q/o projection (4096 -> 4096, i4 g128, outlier channels) at M = 2048 through the integer kernel,
    sampled rows."""
    say(f"w4a8 8B q/o {mode}")
    c = datagen.config3("qo", 2048)
    w = fc.CompressedWeights.from_case(dev, c, output_type="f32", dynamic_quantization=mode)
    try:
        y = req.infer(w, c.x)
        assert req.last_kernel()["name"].startswith("fcc_prefill_i8_w4")
        pick = np.array([0, 1, 500, 777, 2047])
        ref = dq4_reference(oracle, c, c.x[pick], 128 if mode == "per_group" else c.K)
        assert oracle.rel_l2(y[pick], ref) < 2e-6
        plain = oracle_y(oracle, c, x=c.x[pick])
        r = oracle.rel_l2(y[pick], plain)
        say(f"   rel-L2 against the f16-activation oracle: {r:.2e}")
        # the configuration's outlier channels (x 20) set a token's scale: per-token noise is several times the
        # per-group noise, where an outlier only costs its own group of 128 inputs
        assert r < (2e-2 if mode == "per_group" else 1e-1)
    finally:
        w.close()


# ---- asymmetric form: unsigned 8-bit activations with a zero-point per token ----

def dq_asym_reference(oracle, c, x=None):
    zp = None if c.zp is None else c.zp.astype(np.float32)
    return oracle.fc_dynquant_asym_reference(c.x if x is None else x, c.w, T[c.w_type], c.scale, zp, c.bias, N=c.N, K=c.K)


@pytest.mark.parametrize("wt,zt,N,K,bias,out", [("u8", "u8", 256, 512, True, "f32"), ("u8", "none", 512, 384, False, "f16"),
                                                ("i8", "none", 256, 1024, True, "f32"), ("u8", "u8", 768, 128, False, "f32"),
                                                ("u8", "u8", 256, 4096, True, "f32")])
def test_dynquant_asymmetric_matches_integer_oracle(oracle, dev, req, monkeypatch, wt, zt, N, K, bias, out):
    """OVFCC_DYNQUANT_ASYM: the quantisation kernel's half arithmetic, the column sums of the node and the
    zero-point terms of the epilogue against the oracle's sum_k (q - za)(w - zp) -- rows that straddle zero, rows
    with an offset, a constant row, rows on one side of zero (clamped zero-point), the largest half."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    say(f"dynquant asym {wt}/{zt} N={N} K={K} bias={bias} out={out}")
    c = datagen.make_case(1150, 300, K, N, wt, K, zt, with_bias=bias)
    x = c.x.astype(np.float32)
    x += np.linspace(-3, 3, 300, dtype=np.float32)[:, None]     # every row its own offset
    x[5] = 0                                      # constant rows: d = 0.003
    x[6] *= 40
    x[7] = 0.125
    x[8] = np.abs(x[8]) + 1                       # all positive: zero-point below 0, clamped
    x[9] = -np.abs(x[9]) - 1                      # all negative: zero-point above 255, clamped
    x[10, 3] = 65504
    xh = x.astype(np.float16)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out, dynamic_quantization="asymmetric")
    try:
        for M in (49, 128, 129, 300):
            y = req.infer(w, xh[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_prefill_i8_w8_asym", info
            ref = dq_asym_reference(oracle, c, xh[:M])
            # the row with 65504 overflows its half scale, and an f16 result its range: the same on both sides
            with np.errstate(over="ignore"):
                fin = np.isfinite(ref if out == "f32" else ref.astype(np.float16)).all(axis=1)
            assert np.array_equal(np.isfinite(y).all(axis=1), fin)
            if out == "f32":
                assert oracle.rel_l2(y[fin], ref[fin]) < 1e-6, (M, oracle.rel_l2(y[fin], ref[fin]))
                assert np.all(np.abs(y[fin] - ref[fin]) <= np.abs(ref[fin]) * 1e-6 + 1e-6)
            else:
                assert np.mean(y[fin].view(np.uint16) != ref[fin].astype(np.float16).view(np.uint16)) < 1e-3   # f32 ties
                assert oracle.rel_l2(y[fin].astype(np.float32), ref[fin]) < 5e-4
            # against the unquantised arithmetic on rows that straddle zero: the quantisation noise and nothing else
            # (the zero-point enters q unrounded and is stored rounded, as in the reference: up to half a step of
            # offset per row, which weights without a zero-point of their own add up coherently)
            ok = fin.copy()
            ok[[8, 9][:max(0, min(2, M - 8))]] = False
            plain = oracle_y(oracle, c, x=xh[:M])
            assert oracle.rel_l2(y[ok].astype(np.float32), plain[ok]) < 6e-2
            assert np.array_equal(req.infer(w, xh[:M]).view(np.uint8), y.view(np.uint8))
        y = req.infer(w, xh[:32])                 # decode row counts compute in f16: the flag is a permission
        assert req.last_kernel()["kernel"] == _lib.KERNEL_DECODE
    finally:
        w.close()


def test_dynquant_asymmetric_with_gated_linear_unit_and_copies(oracle, dev, req, monkeypatch):
    """The zero-point terms in the gated epilogue (gate and up tiles interleaved: the column sums follow the tiled
    channel order), a clone of the node and a node imported from its blob (their column sums are made anew)."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    c = datagen.make_case(1160, 150, 512, 512, "u8", 512, "u8", with_bias=True)
    xh = (c.x.astype(np.float32) + 1.5).astype(np.float16)
    w = fc.CompressedWeights.from_case(dev, c, output_type="f32", glu="swish", dynamic_quantization="asymmetric")
    w2 = w.clone()
    w3 = fc.CompressedWeights.import_blob(dev, w.export_blob())   # ... and so does a node that comes back from its blob
    try:
        full = dq_asym_reference(oracle, c, xh)
        ref = oracle.glu(full, oracle.GLU_SWISH, False)
        first = None
        for node in (w, w2, w3):
            y = req.infer(node, xh)
            assert req.last_kernel()["name"] == "fcc_prefill_i8_w8_asym"
            assert y.shape == (150, 256) and oracle.rel_l2(y, ref) < 2e-6
            first = y if first is None else first
            assert np.array_equal(y.view(np.uint8), first.view(np.uint8))
    finally:
        w3.close()
        w2.close()
        w.close()
