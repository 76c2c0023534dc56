"""GPU parity of the 16-row decode kernel with stationary activations (five to 48 rows, 4-bit weights, groups of 128
inputs) against the CPU oracle: every division of K over the waves of a workgroup (2, 4 or 8 k-blocks per wave),
every row count class (part of a row tile, a whole one, part of the second, two, part of the third, three), workgroups that visit one, two
and many channel tiles, zero-point table / constant / none, bias, both output types, the same bits on every
repetition, the gated linear unit, and the node shapes of the benchmark; and of its sibling for five to 16 rows that
streams the activations instead (K too long to keep them: the down projection)."""
import sys

import numpy as np
import pytest

from openvino_amd import datagen, fc
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


# (w_type, zp_type, N, K, k-blocks per wave forced at creation, workgroups per row tile forced (0: policy), bias)
SHAPES = [
    ("u4", "u4", 272, 1024, 2, 0, True),     # 4 waves, 17 channel tiles, one visit each
    ("u4", "u4", 272, 1024, 2, 5, False),    # ... 5 workgroups: four visits for two of them, three for the rest
    ("u4", "u4", 64, 1024, 4, 2, True),      # 2 waves, two visits each
    ("i4", "none", 48, 1024, 8, 1, True),    # 2 waves walk all three tiles; symmetric weights (zero-point 8)
    ("i4", "none", 256, 4096, 4, 0, False),  # 8 waves, 128 KiB of activations through LDS
    ("u4", "u8", 128, 4096, 2, 0, True),     # 16 waves, 8-bit zero-point table
    ("u4", "u8", 128, 4096, 2, 3, True),     # ... three workgroups: two buffers of partial sums would be needed
    ("u4", "none", 64, 2048, 4, 0, True),    # no zero-point at all: the second MFMA chain is skipped
    ("u4", "u4", 80, 3072, 4, 2, True),      # 6 waves
    ("u4", "u4", 96, 4096, 8, 4, False),     # tables for 4 waves of 8 k-blocks: 8 waves of 4
    ("u4", "none", 32, 256, 2, 0, True),     # 1 wave adds all four row groups itself
]


@pytest.mark.parametrize("wt,zt,N,K,C,grid,bias", SHAPES)
@pytest.mark.parametrize("out", ["f16", "f32"])
def test_gemv16_rows_five_to_forty_eight(oracle, dev, req, monkeypatch, wt, zt, N, K, C, grid, bias, out):
    monkeypatch.setenv("OVFCC_GEMV_C", str(C))
    if grid:
        monkeypatch.setenv("OVFCC_GEMV16_GRID", str(grid))
    c = datagen.make_case(7500 + N + K, 48, K, N, wt, 128, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out)
    ref = oracle_y(oracle, c)
    try:
        for M in (5, 8, 15, 16, 17, 31, 32, 33, 48):
            say(f"gemv16 {wt}/{zt} N={N} K={K} C={C} grid={grid} out={out} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            if K == 4096 and C == 2 and grid:
                # 16 waves x 8 KiB of activations leave no room for a second buffer of partial sums
                assert info["name"] != "fcc_gemv16_w4", info
                continue
            # tables laid out for eight k-blocks per wave are read by two waves per row, four k-blocks each
            assert info["name"] == "fcc_gemv16_w4" and info["block"] == 64 * (K // 128 // min(C, 4)), info
            assert info["grid"][0] == (grid or N // 16) and info["grid"][1] == (M + 15) // 16, info
            assert y.dtype == (np.float32 if out == "f32" else np.float16)
            check_parity(oracle, y, ref[:M], K, f"M={M} {info}", output_rounding_slack=True)
            for _ in range(3):    # partial sums are added in wave order
                assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
    finally:
        w.close()


def test_gemv16_scalar_zero_point(oracle, dev, req):
    """One zero-point for the whole node (Shape{}): it travels as a constant, not as a table."""
    c = datagen.make_case(7601, 12, 2048, 96, "u4", 128, "u8", with_bias=True)
    zp = np.array([11], dtype=np.uint8)
    c = datagen.FcCase(c.M, c.K, c.N, c.group_size, c.w_type, "u8", c.w, c.scale, zp, c.x, c.bias, zp_scalar=1)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        y = req.infer(w, c.x)
        assert req.last_kernel()["name"] == "fcc_gemv16_w4"
        check_parity(oracle, y, oracle_y(oracle, c), c.K, "scalar zp", output_rounding_slack=True)
    finally:
        w.close()


def test_gemv16_tiny_and_huge_activations(oracle, dev, req):
    """Half of the activations are multiplied by 2^-4 in their registers: values below 2^-10 lose bits there (at most
    2^-21 absolute each); subnormal activations, activations near the top of the half range and a row of zeros
    between rows of ordinary values must come out right."""
    c = datagen.make_case(7700, 8, 1024, 64, "u4", 128, "u4")
    x = c.x.astype(np.float32)
    x[0] *= 2.0 ** -12
    x[1] = np.where(np.arange(c.K) % 3 == 0, 6.0e-8, 0.0)   # the smallest subnormal half
    x[2] = np.where(np.arange(c.K) % 128 == 5, 60000.0, x[2])  # near the largest half
    x[3] = 0.0
    xh = x.astype(np.float16)
    w = fc.CompressedWeights.from_case(dev, c, output_type="f32")
    try:
        y = req.infer(w, xh)
        assert req.last_kernel()["name"] == "fcc_gemv16_w4"
        ref = oracle_y(oracle, c, x=xh)
        assert np.all(y[3] == 0.0)
        for m in range(8):
            scale = float(np.max(np.abs(ref[m]))) or 1.0
            err = float(np.max(np.abs(y[m] - ref[m])))
            say(f"   row {m}: max |y| {scale:.3e}, max-abs error {err:.3e}")
            # 1e-3 of the row's own magnitude, plus what 2^-21 per input can add: K/2 inputs * 15 * max scale 0.02
            assert err <= 1e-3 * scale + 2.0 ** -21 * (c.K / 2) * 15 * 0.02, (m, err, scale)
    finally:
        w.close()


@pytest.mark.parametrize("name,N,K", [("q/o", 4096, 4096), ("k/v", 1024, 4096), ("gate/up", 14336, 4096)])
def test_gemv16_benchmark_nodes(oracle, dev, req, name, N, K):
    """The Llama-3-8B projections whose activations fit in LDS, at the benchmark's row counts, against the oracle on
    a sample of channels."""
    c = datagen.make_case(7800 + N, 48, K, N, "i4", 128, "none")
    w = fc.CompressedWeights.from_case(dev, c)
    rng = np.random.default_rng(5)
    cols = np.sort(rng.choice(N, size=256, replace=False))
    ref = oracle_y(oracle, c, n_index=cols)
    try:
        for M in (8, 16, 32, 48):
            say(f"gemv16 {name} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            # one round of workgroups (two for up to 8 rows) and one row tile: the activations are streamed
            streamed = (name in ("q/o", "k/v") and M <= 16) or (name == "gate/up" and M <= 8)
            assert info["name"] == ("fcc_gemv16s_w4" if streamed else "fcc_gemv16_w4"), info
            check_parity(oracle, y[:, cols], ref[:M], K, f"{name} M={M} {info}")
    finally:
        w.close()


@pytest.mark.parametrize("wt,zt,N,K,C,grid,kind,second", [("u4", "u4", 512, 1024, 2, 0, "swish", False),
                                                         ("i4", "none", 256, 2048, 4, 3, "gelu", True),
                                                         ("i4", "none", 128, 4096, 8, 0, "gelu_tanh", False),
                                                         ("u4", "u4", 64, 4096, 4, 1, "swish", True)])
def test_gemv16_gated_linear_unit(oracle, dev, req, monkeypatch, wt, zt, N, K, C, grid, kind, second):
    """Gate and up tile of 16 channels are two visits of one workgroup; the gate values wait in registers."""
    monkeypatch.setenv("OVFCC_GEMV_C", str(C))
    if grid:
        monkeypatch.setenv("OVFCC_GEMV16_GRID", str(grid))
    c = datagen.make_case(7950 + N, 48, K, N, wt, 128, zt, with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c, glu=kind, glu_gate_second=second)
    try:
        for M in (5, 16, 17, 32, 40):
            say(f"gemv16 glu {kind} {wt}/{zt} N={N} K={K} C={C} grid={grid} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_gemv16_w4" and info["block"] == 64 * (K // 128 // min(C, 4)), info
            assert info["grid"][0] == (grid or N // 32) and info["grid"][1] == (M + 15) // 16, info
            assert y.shape == (M, N // 2)
            ref, amp = glu_reference(oracle, c, kind, second, x=c.x[:M])
            check_parity(oracle, y, ref, K, f"M={M} {info}", output_rounding_slack=True, limit_scale=amp)
            assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
    finally:
        w.close()


# (w_type, zp_type, N, K, k-blocks per wave of the tables, parts, workgroups per row tile forced, bias, output)
SPLIT_SHAPES = [
    ("u4", "u4", 64, 1024, 8, 4, 0, True, "f16"),     # tables for 1 wave of 8: four parts of one wave with 2 k-blocks
    ("u4", "u4", 272, 1024, 8, 2, 5, True, "f32"),    # two parts of one wave with 4; several visits
    ("i4", "none", 48, 2048, 4, 2, 0, False, "f16"),  # tables for 4 waves of 4: two parts of 4 waves with 2
    ("u4", "u8", 96, 4096, 8, 4, 2, True, "f16"),     # 4 waves, zero-point table, three visits
    ("i4", "none", 64, 14336, 8, 4, 0, True, "f16"),  # the down projection's K: 14 waves per part
    ("u4", "u4", 80, 14336, 8, 4, 3, False, "f32"),   # ... with a zero-point table and two visits
]


@pytest.mark.parametrize("wt,zt,N,K,C,parts,grid,bias,out", SPLIT_SHAPES)
def test_gemv16_k_in_parts(oracle, dev, req, monkeypatch, wt, zt, N, K, C, parts, grid, bias, out):
    """K cut in parts across workgroups, partial sums added by a second launch: every row count class, the same bits
    on every repetition (the parts are added in a fixed order)."""
    monkeypatch.setenv("OVFCC_GEMV_C", str(C))
    monkeypatch.setenv("OVFCC_GEMV16_SPLIT", str(parts))
    if grid:
        monkeypatch.setenv("OVFCC_GEMV16_GRID", str(grid))
    c = datagen.make_case(7650 + N + K, 48, K, N, wt, 128, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out)
    ref = oracle_y(oracle, c)
    try:
        for M in (5, 16, 17, 33, 48):
            say(f"gemv16 parts {wt}/{zt} N={N} K={K} C={C} parts={parts} grid={grid} out={out} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_gemv16_w4" and info["split_k"] == parts, info
            assert info["grid"] == (grid or N // 16, (M + 15) // 16, parts), info
            assert info["block"] == 64 * (K // 128 // (C // parts) // parts), info
            check_parity(oracle, y, ref[:M], K, f"M={M} {info}", output_rounding_slack=True)
            assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
    finally:
        w.close()


def test_gemv16_two_parts_by_policy(oracle, dev, req):
    """K = 8192 (the q / o class of Llama-3-70B): 16 rows of activations are 256 KiB, so the planner cuts K in two
    parts, at any row count from five on."""
    c = datagen.make_case(7870, 48, 8192, 256, "u4", 128, "u4", with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    ref = oracle_y(oracle, c)
    try:
        for M in (5, 16, 32):
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            say(f"gemv16 K=8192 M={M} {info}")
            assert info["name"] == "fcc_gemv16_w4" and info["split_k"] == 2, info
            check_parity(oracle, y, ref[:M], c.K, f"K=8192 M={M} {info}", output_rounding_slack=True)
    finally:
        w.close()


def test_gemv16_down_projection(oracle, dev, req):
    """The benchmark's down projection (14336 -> 4096): up to 16 rows the kernel that streams its activations (one
    workgroup of 14 waves per channel tile, K whole), from 17 rows on stationary activations with K in four parts."""
    K, N = 14336, 4096
    c = datagen.make_case(7860, 48, K, N, "i4", 128, "none")
    w = fc.CompressedWeights.from_case(dev, c)
    cols = np.sort(np.random.default_rng(6).choice(N, size=256, replace=False))
    ref = oracle_y(oracle, c, n_index=cols)
    try:
        for M in (5, 8, 13, 16, 17, 32, 48):
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            say(f"gemv16 down M={M} {info}")
            if M <= 16:
                assert info["name"] == "fcc_gemv16s_w4" and info["split_k"] == 1 and info["block"] == 64 * 14, info
                assert info["grid"] == (N // 16, 1, 1), info
            else:
                assert info["name"] == "fcc_gemv16_w4" and info["split_k"] == 4 and info["block"] == 64 * 14, info
            check_parity(oracle, y[:, cols], ref[:M], K, f"down M={M} {info}")
            assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
    finally:
        w.close()


# (w_type, zp_type, N, K, k-blocks per wave, bias, output)
STREAM_SHAPES = [
    ("u4", "u4", 64, 1024, 2, True, "f16"),      # 4 waves of 2 k-blocks: both activation buffers filled once, no refill
    ("u4", "u4", 272, 1024, 8, False, "f32"),    # 1 wave walks all of K: six refills, adds its own four row groups
    ("i4", "none", 48, 2048, 4, True, "f16"),    # 4 waves of 4; symmetric weights (zero-point 8 as a constant)
    ("u4", "u8", 96, 4096, 8, True, "f16"),      # 8-bit zero-point table, two words per channel and wave
    ("u4", "none", 32, 256, 2, True, "f32"),     # 1 wave, 2 k-blocks, no zero-point
    ("u4", "u4", 80, 14336, 8, False, "f32"),    # the down projection's K: 14 waves, 112 KiB of LDS
    ("i4", "none", 64, 14336, 8, True, "f16"),
    ("u4", "u4", 64, 4096, 2, True, "f16"),      # 16 waves: the largest workgroup, 128 KiB of LDS
]


@pytest.mark.parametrize("tiles", [1, 2, 4])
@pytest.mark.parametrize("wt,zt,N,K,C,bias,out", STREAM_SHAPES)
def test_gemv16_streamed_activations(oracle, dev, req, monkeypatch, wt, zt, N, K, C, bias, out, tiles):
    """The 16-row kernel that streams its activations through a double buffer per wave, taken wherever it can run
    (OVFCC_GEMV16_STREAM = 1): every division of K over the waves, rows short of a tile (loaded out of range, so
    that the count of loads in flight does not depend on M) and a whole tile, the same bits on every repetition."""
    monkeypatch.setenv("OVFCC_GEMV_C", str(C))
    monkeypatch.setenv("OVFCC_GEMV16_STREAM", "1")
    monkeypatch.setenv("OVFCC_GEMV16_STREAM_TILES", str(tiles))   # channel tiles per workgroup, where N divides
    if (N // 16) % tiles:
        tiles = 1
    c = datagen.make_case(7450 + N + K, 16, K, N, wt, 128, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out)
    ref = oracle_y(oracle, c)
    try:
        for M in (5, 8, 15, 16):
            say(f"gemv16s {wt}/{zt} N={N} K={K} C={C} out={out} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["name"] == "fcc_gemv16s_w4" and info["block"] == 64 * (K // 128 // C), info
            assert info["grid"] == (N // 16 // tiles, 1, 1) and info["split_k"] == 1, info
            assert y.dtype == (np.float32 if out == "f32" else np.float16)
            check_parity(oracle, y, ref[:M], K, f"M={M} {info}", output_rounding_slack=True)
            for _ in range(3):    # partial sums are added in wave order
                assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
        # 17 rows and the switch: other kernels
        monkeypatch.setenv("OVFCC_GEMV16_STREAM", "0")
        req.infer(w, c.x[:8])
        assert req.last_kernel()["name"] != "fcc_gemv16s_w4"
    finally:
        w.close()


@pytest.mark.parametrize("seed", range(10))
def test_gemv16_streamed_random_nodes(oracle, dev, req, monkeypatch, seed):
    """Seeded sweep of the streaming kernel: formats, K and its division over the waves, channel counts, row counts,
    bias and output type that the table above does not pair up."""
    rng = np.random.default_rng(7460 + seed)
    monkeypatch.setenv("OVFCC_GEMV16_STREAM", "1")
    for _ in range(4):
        C = int(rng.choice([2, 4, 8]))
        waves = int(rng.integers(1, 17))
        K = 128 * C * waves
        wt = str(rng.choice(["u4", "i4"]))
        zt = str(rng.choice(["none", "u4", "u8"])) if wt == "u4" else "none"
        N = 16 * int(rng.integers(1, 40))
        M = int(rng.integers(5, 17))
        bias, out = bool(rng.integers(0, 2)), str(rng.choice(["f16", "f32"]))
        tiles = int(rng.choice([1, 2, 4]))
        monkeypatch.setenv("OVFCC_GEMV_C", str(C))
        monkeypatch.setenv("OVFCC_GEMV16_STREAM_TILES", str(tiles))
        if (N // 16) % tiles:
            tiles = 1
        what = f"seed {seed}: {wt}/{zt} N={N} K={K} C={C} waves={waves} tiles={tiles} M={M} bias={bias} out={out}"
        say(what)
        c = datagen.make_case(int(rng.integers(1, 1 << 30)), M, K, N, wt, 128, zt, with_bias=bias)
        w = fc.CompressedWeights.from_case(dev, c, output_type=out)
        try:
            y = req.infer(w, c.x)
            info = req.last_kernel()
            assert info["name"] == "fcc_gemv16s_w4" and info["block"] == 64 * waves, (what, info)
            assert info["grid"] == (N // 16 // tiles, 1, 1), (what, info)
            check_parity(oracle, y, oracle_y(oracle, c), K, f"{what} {info}", output_rounding_slack=True)
        finally:
            w.close()


def test_gemv16_streamed_two_tiles_by_policy(oracle, dev, req):
    """More channel tiles than compute units: two tiles per workgroup share a k-block of activations.  One round of
    workgroups (4096 -> 8192: 512 tiles, 256 workgroups) is taken up to 16 rows, more than one (4096 -> 14336: 448
    workgroups) up to 8."""
    for N, rows in ((8192, (5, 8, 16)), (14336, (8,))):
        K = 4096
        c = datagen.make_case(7880 + N, 16, K, N, "u4", 128, "u4", with_bias=True)
        w = fc.CompressedWeights.from_case(dev, c)
        cols = np.sort(np.random.default_rng(8).choice(N, size=256, replace=False))
        ref = oracle_y(oracle, c, n_index=cols)
        try:
            for M in rows:
                y = req.infer(w, c.x[:M])
                info = req.last_kernel()
                say(f"gemv16s two tiles N={N} M={M} {info}")
                assert info["name"] == "fcc_gemv16s_w4" and info["grid"] == (N // 32, 1, 1), info
                check_parity(oracle, y[:, cols], ref[:M], K, f"N={N} M={M} {info}")
            y = req.infer(w, c.x[:16])
            if N == 14336:
                assert req.last_kernel()["name"] == "fcc_gemv16_w4", req.last_kernel()
        finally:
            w.close()


def test_gemv16_streamed_tiny_and_huge_activations(oracle, dev, req, monkeypatch):
    """Subnormal activations, activations near the top of the half range and a row of zeros through the streaming
    kernel (same arithmetic as the stationary one: half of the activations are multiplied by 2^-4 in registers)."""
    monkeypatch.setenv("OVFCC_GEMV16_STREAM", "1")
    c = datagen.make_case(7701, 8, 2048, 64, "u4", 128, "u4")
    x = c.x.astype(np.float32)
    x[0] *= 2.0 ** -12
    x[1] = np.where(np.arange(c.K) % 3 == 0, 6.0e-8, 0.0)
    x[2] = np.where(np.arange(c.K) % 128 == 5, 60000.0, x[2])
    x[3] = 0.0
    xh = x.astype(np.float16)
    w = fc.CompressedWeights.from_case(dev, c, output_type="f32")
    try:
        y = req.infer(w, xh)
        assert req.last_kernel()["name"] == "fcc_gemv16s_w4"
        ref = oracle_y(oracle, c, x=xh)
        assert np.all(y[3] == 0.0)
        for m in range(8):
            scale = float(np.max(np.abs(ref[m]))) or 1.0
            err = float(np.max(np.abs(y[m] - ref[m])))
            assert err <= 1e-3 * scale + 2.0 ** -21 * (c.K / 2) * 15 * 0.02, (m, err, scale)
    finally:
        w.close()


def test_gemv16_leaves_what_does_not_fit(dev, req):
    """Groups of 64 inputs, 8-bit weights, K whose k-blocks the waves cannot share out (K = 128 x 9): other kernels."""
    for wt, zt, N, K, G in (("u4", "none", 64, 128 * 9, 128), ("u4", "u4", 64, 1024, 64), ("u8", "u8", 64, 1024, 128)):
        c = datagen.make_case(7900, 8, K, N, wt, G, zt)
        w = fc.CompressedWeights.from_case(dev, c)
        try:
            req.infer(w, c.x)
            assert req.last_kernel()["name"] != "fcc_gemv16_w4", (wt, zt, N, K, G)
        finally:
            w.close()
