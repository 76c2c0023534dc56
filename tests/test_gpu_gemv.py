"""GPU parity of the matrix-vector decode kernel (one to four rows, 4-bit weights, groups of 128 inputs) against the
CPU oracle: every division of K over the waves of a workgroup (2, 4 or 8 k-blocks per wave, 1 to 16 waves), both
ways of electing the wave that adds the partial sums, every row count, zero-point table / constant / none, bias, both
output types, the gated linear unit, and the same bits on every repetition."""
import sys

import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc
from parity import check_parity, glu_reference, oracle_y

pytestmark = pytest.mark.gpu


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


# (w_type, zp_type, N, K, k-blocks per wave forced at creation, bias)
SHAPES = [
    ("u4", "u4", 272, 1024, 2, True),      # 4 waves per tile, ragged tile count, ticket
    ("u4", "u4", 64, 1024, 4, False),      # 2 waves
    ("i4", "none", 48, 1024, 8, True),     # 1 wave: a reduction over one partial sum
    ("i4", "none", 256, 4096, 8, False),   # 4 waves, the shape class of the benchmark's q / o node
    ("u4", "u8", 128, 4096, 2, True),      # 16 waves: closing barrier
    ("u4", "none", 64, 14336, 8, True),    # 14 waves (down projection): closing barrier, no zero-point at all
    ("i4", "none", 32, 2048, 4, False),    # 4 waves
    ("u4", "u4", 80, 3072, 4, True),       # 6 waves
]


@pytest.mark.parametrize("wt,zt,N,K,C,bias", SHAPES)
@pytest.mark.parametrize("out", ["f16", "f32"])
def test_gemv_rows_one_to_four(oracle, dev, req, monkeypatch, wt, zt, N, K, C, bias, out):
    monkeypatch.setenv("OVFCC_GEMV_C", str(C))
    c = datagen.make_case(7000 + N + K, 4, K, N, wt, 128, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out)
    ref = oracle_y(oracle, c)
    try:
        for M in (1, 2, 3, 4):
            say(f"gemv {wt}/{zt} N={N} K={K} C={C} out={out} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_gemv_w4" and info["block"] == 64 * (K // 128 // C), info
            assert y.dtype == (np.float32 if out == "f32" else np.float16)
            check_parity(oracle, y, ref[:M], K, f"M={M} {info}", output_rounding_slack=True)
            for _ in range(3):    # partial sums are added in wave order whichever wave arrives last
                assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
    finally:
        w.close()


def test_gemv_scalar_zero_point(oracle, dev, req):
    """One zero-point for the whole node (Shape{}): it travels as a constant, not as a table."""
    c = datagen.make_case(7101, 4, 2048, 96, "u4", 128, "u8", with_bias=True)
    zp = np.array([11], dtype=np.uint8)
    c = datagen.FcCase(c.M, c.K, c.N, c.group_size, c.w_type, "u8", c.w, c.scale, zp, c.x, c.bias, zp_scalar=1)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        y = req.infer(w, c.x[:3])
        assert req.last_kernel()["name"] == "fcc_gemv_w4"
        check_parity(oracle, y, oracle_y(oracle, c)[:3], c.K, "scalar zp", output_rounding_slack=True)
    finally:
        w.close()


@pytest.mark.parametrize("wt,zt,N,K,C,kind,second", [("u4", "u4", 512, 1024, 2, "swish", False),
                                                    ("i4", "none", 256, 2048, 4, "gelu", True),
                                                    ("i4", "none", 128, 4096, 8, "gelu_tanh", False),
                                                    ("u4", "u8", 64, 4096, 4, "swish", True)])
def test_gemv_gated_linear_unit(oracle, dev, req, monkeypatch, wt, zt, N, K, C, kind, second):
    """Gate and up tile of 16 channels share a workgroup of 2 K / (128 C) waves."""
    monkeypatch.setenv("OVFCC_GEMV_C", str(C))
    c = datagen.make_case(7200 + N, 4, K, N, wt, 128, zt, with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c, glu=kind, glu_gate_second=second)
    try:
        for M in (1, 2, 4):
            say(f"gemv glu {kind} {wt}/{zt} N={N} K={K} C={C} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_gemv_w4" and info["block"] == 128 * (K // 128 // C), info
            ref, amp = glu_reference(oracle, c, kind, second, x=c.x[:M])
            check_parity(oracle, y, ref, K, f"M={M} {info}", output_rounding_slack=True, limit_scale=amp)
    finally:
        w.close()


def test_gemv_tiny_and_huge_activations(oracle, dev, req):
    """Half of the activations are staged multiplied by 2^-4: values below 2^-10 lose bits there (at most 2^-21
    absolute each), subnormal activations and activations near the top of the half range must come out right."""
    c = datagen.make_case(7300, 4, 1024, 64, "u4", 128, "u4")
    x = c.x.astype(np.float32)
    x[0] *= 2.0 ** -12                        # around 2^-12: below the exact range of the staging multiply
    x[1] = np.where(np.arange(c.K) % 3 == 0, 6.0e-8, 0.0)   # the smallest subnormal half
    x[2] = np.where(np.arange(c.K) % 128 == 5, 60000.0, x[2])  # near the largest half
    xh = x.astype(np.float16)
    w = fc.CompressedWeights.from_case(dev, c, output_type="f32")
    try:
        y = req.infer(w, xh)
        assert req.last_kernel()["name"] == "fcc_gemv_w4"
        ref = oracle_y(oracle, c, x=xh)
        for m in range(4):
            scale = float(np.max(np.abs(ref[m]))) or 1.0
            err = float(np.max(np.abs(y[m] - ref[m])))
            say(f"   row {m}: max |y| {scale:.3e}, max-abs error {err:.3e}")
            # 1e-3 of the row's own magnitude, plus what 2^-21 per input can add: K/2 inputs * 15 * max scale 0.02
            assert err <= 1e-3 * scale + 2.0 ** -21 * (c.K / 2) * 15 * 0.02, (m, err, scale)
    finally:
        w.close()


def test_gemv_falls_back_where_it_does_not_fit(dev, req):
    """Groups of 256 inputs, 8-bit weights, five rows, K / 128 not divisible: the streaming kernel runs instead."""
    for wt, zt, N, K, G, M in (("u4", "u4", 64, 1024, 256, 1), ("u8", "u8", 64, 1024, 128, 1),
                              ("u4", "u4", 64, 1024, 128, 5), ("u4", "none", 64, 128 * 9, 128, 1)):
        c = datagen.make_case(7400, M, K, N, wt, G, zt)
        w = fc.CompressedWeights.from_case(dev, c)
        try:
            req.infer(w, c.x[:M])
            assert req.last_kernel()["name"] != "fcc_gemv_w4", (wt, zt, N, K, G, M)
        finally:
            w.close()
