"""The 4-bit prefill kernel with 256 x 256 tiles (four waves of 512 registers), forced onto shapes small enough for
the oracle to cover every output: weight types, zero-point forms, scale grouping, bias, both output types, the
gated linear unit, ragged last row tiles, odd k-block counts."""
import numpy as np
import pytest

from openvino_amd import datagen, fc
from parity import check_parity, glu_reference, oracle_y

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


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


@pytest.mark.parametrize("wt,zt,N,K,G,out,bias", [
    ("i4", "none", 512, 512, 128, "f16", False),     # the benchmark's format
    ("u4", "u4", 256, 384, 128, "f16", True),        # zero-point table, odd number of k-blocks
    ("u4", "u8", 512, 1024, 256, "f32", True),       # a group spans two k-blocks
    ("u4", "none", 256, 640, 640, "f32", True),      # one group per channel: scale in the epilogue
    ("u4", "u4", 256, 128, 128, "f16", False),       # a single k-block
])
def test_big_tiles_small_shapes(oracle, dev, req, monkeypatch, wt, zt, N, K, G, out, bias):
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    monkeypatch.setenv("OVFCC_PREFILL_ROWS", "128")
    monkeypatch.setenv("OVFCC_PREFILL_BIG", "1")
    c = datagen.make_case(1300, 700, K, N, wt, G, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out)
    ref = oracle_y(oracle, c)
    try:
        for M in (129, 256, 300, 700):
            say(f"big tiles {wt}/{zt} N={N} K={K} G={G} out={out} bias={bias} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_prefill_big_w4" and info["tile_m"] == 256 and info["block"] == 256, info
            assert info["grid"][0] == (N // 256) * ((M + 255) // 256), info
            check_parity(oracle, y, ref[:M], K, f"{info}", output_rounding_slack=True)
            assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
    finally:
        w.close()


@pytest.mark.parametrize("kind", ["swish", "gelu_tanh"])
@pytest.mark.parametrize("wt,zt,N,K,G", [("u4", "u4", 1024, 512, 128), ("i4", "none", 512, 512, 512)])
def test_big_tiles_gated_linear_unit(oracle, dev, req, monkeypatch, wt, zt, N, K, G, kind):
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    monkeypatch.setenv("OVFCC_PREFILL_ROWS", "128")
    monkeypatch.setenv("OVFCC_PREFILL_BIG", "1")
    M = 2 * 256 + 5
    c = datagen.make_case(1301, M, K, N, wt, G, zt, with_bias=True)
    ref, amp = glu_reference(oracle, c, kind)
    for out in ("f16", "f32"):
        w = fc.CompressedWeights.from_case(dev, c, output_type=out, glu=kind)
        try:
            say(f"big tiles glu {kind} {wt}/{zt} N={N} K={K} G={G} out={out}")
            y = req.infer(w, c.x)
            info = req.last_kernel()
            assert info["name"] == "fcc_prefill_big_w4", info
            check_parity(oracle, y, ref, K, f"{info}", output_rounding_slack=True, limit_scale=amp)
        finally:
            w.close()
