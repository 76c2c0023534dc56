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


def test_big_tiles_real_shape_every_row_of_a_channel_slab(oracle, dev, req):
    """Llama-3-8B gate/up (4096 -> 14336, i4 g128 with outlier channels) at M = 8192, the shape the policy gives to
    the 256 x 256 kernel by itself: every one of the 8192 rows of two 256-channel slabs (one inside, the last one)
    against the oracle run on those channels' weights."""
    M = 8192
    c = datagen.config3("gate_up", M)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        say("big tiles, gate/up at M = 8192, full slabs")
        y = req.infer(w, c.x)
        info = req.last_kernel()
        assert info["name"] == "fcc_prefill_big_w4" and info["tile_m"] == 256, info
        ng = c.K // c.group_size
        for n0 in (7 * 256, c.N - 256):
            rows = slice(n0, n0 + 256)
            sub = datagen.FcCase(M, c.K, 256, c.group_size, c.w_type, c.zp_type,
                                 c.w.reshape(c.N, c.K // 2)[rows].copy().ravel(),
                                 c.scale.reshape(c.N, ng)[rows].copy(), None, c.x, None)
            ref = oracle_y(oracle, sub)
            check_parity(oracle, y[:, rows], ref, c.K, f"slab {n0}", output_rounding_slack=True)
    finally:
        w.close()


@pytest.mark.parametrize("wt,zt,N,K,G,out,bias,glu", [("i4", "none", 1024, 1024, 128, "f16", False, None),
                                                      ("u4", "u4", 512, 640, 128, "f32", True, None),
                                                      ("u4", "u4", 1024, 512, 128, "f16", True, "swish"),
                                                      ("u4", "none", 512, 768, 768, "f32", False, None)])
def test_big_tiles_against_the_128_row_kernel(oracle, dev, req, monkeypatch, wt, zt, N, K, G, out, bias, glu):
    """The two kernels on the same inputs.  They are not the same bits: the 256-row kernel's waves each walk the whole
    of K while the 128-row kernel's two k-groups sum halves of every k-block and add them at the end, so the f32
    sums differ in their last bits.  What holds: f32 outputs agree to a few ulps of f32 (of the largest output), f16
    outputs are equal or one half-precision step apart, and few are apart (a rounding tie moved, not an error)."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    monkeypatch.setenv("OVFCC_PREFILL_ROWS", "128")
    c = datagen.make_case(1310, 1000, K, N, wt, G, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out, glu=glu)
    try:
        for M in (512, 1000):
            say(f"big vs 128-row tiles {wt}/{zt} N={N} K={K} G={G} out={out} glu={glu} M={M}")
            monkeypatch.setenv("OVFCC_PREFILL_BIG", "1")
            yb = req.infer(w, c.x[:M])
            assert req.last_kernel()["name"] == "fcc_prefill_big_w4"
            monkeypatch.setenv("OVFCC_PREFILL_BIG", "0")
            ya = req.infer(w, c.x[:M])
            assert req.last_kernel()["name"] == "fcc_prefill_async_w4" and req.last_kernel()["split_k"] == 1
            if out == "f32":
                scale = float(np.max(np.abs(ya)))
                assert np.max(np.abs(ya - yb)) <= 8e-6 * scale, np.max(np.abs(ya - yb)) / scale
            else:
                a32, b32 = ya.astype(np.float32), yb.astype(np.float32)
                scale = float(np.max(np.abs(a32)))
                # one half-precision step at the value's magnitude, or the f32 disagreement where the value is tiny
                step = np.maximum(np.spacing(np.maximum(np.abs(ya), np.abs(yb))).astype(np.float32), 8e-6 * scale)
                assert np.all(np.abs(a32 - b32) <= step), float(np.max(np.abs(a32 - b32) / step))
                assert np.count_nonzero(ya != yb) < 0.01 * ya.size, np.count_nonzero(ya != yb) / ya.size
    finally:
        w.close()
