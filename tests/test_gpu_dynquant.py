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
    """4-bit weights, grouped scales or a narrow node: the permission has no integer kernel to take effect in; nor
    does it take effect where the integer kernel's grid would leave most of the chip idle."""
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
    for wt, zt, N, K, G in (("u4", "u4", 256, 512, 128), ("u8", "u8", 256, 512, 128), ("u8", "u8", 128, 512, 512)):
        c = datagen.make_case(1110, 200, K, N, wt, G, zt)
        w = fc.CompressedWeights.from_case(dev, c, dynamic_quantization=True)
        try:
            y = req.infer(w, c.x)
            assert req.last_kernel()["name"] != "fcc_prefill_i8_w8"
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
