"""GPU parity: the HIP path through the C ABI against the CPU oracle.

Tolerances (float path): relative L2 error <= 1e-3 and max-abs error <= 2e-2*sqrt(K/4096) against the
fp32 dequantise-then-matmul oracle.  Golden vectors of the reference's own tests must come out exactly.
"""
import sys

import numpy as np
import pytest

from golden_cases import fc_cases
from openvino_amd import _lib, datagen, fc
from parity import check_parity, oracle_y, run_case

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


GOLD = fc_cases()


@pytest.mark.parametrize("g", GOLD, ids=[g["id"] for g in GOLD])
def test_golden_vectors_exact(dev, req, g):
    """Every value of these cases is exact in float16, so the f16 device path must reproduce it bit for bit."""
    say(f"golden {g['id']} N={g['N']} K={g['K']}")
    c = datagen.FcCase(g["M"], g["K"], g["N"], g["group_size"], g["w_type"], "none" if g["zp"] is None else "u8",
                       g["w"], g["scale"].astype(np.float16), g["zp"], g["x"].astype(np.float16),
                       None if g["bias"] is None else g["bias"].astype(np.float16), zp_scalar=g["zp_scalar"])
    x = c.x.reshape(g["x_shape"])
    y, info = run_case(dev, req, c, x=x)
    assert y.shape == tuple(g["x_shape"][:-1]) + (g["N"],)
    assert np.array_equal(y.reshape(g["M"], g["N"]).astype(np.float32), g["expected"]), (g["source"], info)


@pytest.mark.parametrize("n_pad", [16, 128])
@pytest.mark.parametrize("M", [1, 40])
def test_golden_accumulation_on_tiled_kernels(dev, req, n_pad, M):
    """The int4 accumulation vector (all weights 1, all activations 1, K = 4096) widened to a tiled shape:
    every output is exactly 4096 on the decode and the prefill kernel."""
    say(f"accumulation N={n_pad} M={M}")
    c = datagen.FcCase(M, 4096, n_pad, 128, "u4", "none", np.full(n_pad * 2048, 0x11, np.uint8),
                       np.ones((n_pad, 32), np.float16), None, np.ones((M, 4096), np.float16))
    y, info = run_case(dev, req, c)
    assert info["kernel"] != _lib.KERNEL_PLAIN
    assert np.all(y.astype(np.float32) == 4096.0), info


SMALL = [
    # w_type, zp_type, N, K, G, with_bias
    ("u4", "u4", 128, 512, 128, False), ("u4", "none", 256, 256, 128, True), ("i4", "none", 128, 1024, 128, False),
    ("i4", "u4", 128, 512, 256, True), ("u4", "u8", 384, 384, 128, False), ("u8", "u8", 128, 512, 512, False),
    ("u8", "none", 128, 256, 128, True), ("u8", "u8", 256, 384, 128, False), ("i8", "none", 128, 256, 256, False),
    ("u4", "u4", 48, 256, 128, False),      # tiled, N not a multiple of 128: decode kernel in 32-row chunks
    ("u4", "u4", 40, 200, 50, True),        # untiled: plain kernel
    ("i4", "none", 24, 96, 32, False),      # untiled
    ("u8", "u8", 8, 6, 6, False),
]
MS = [1, 2, 3, 15, 16, 17, 31, 32, 33, 63, 65, 130, 257]


@pytest.mark.parametrize("wt,zt,N,K,G,bias", SMALL)
def test_small_shapes_all_row_counts(oracle, dev, req, wt, zt, N, K, G, bias):
    c = datagen.make_case(11, max(MS), K, N, wt, G, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c)
    ref = oracle_y(oracle, c)
    seen = set()
    try:
        for M in MS:
            say(f"small {wt}/{zt} N={N} K={K} G={G} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            seen.add(info["name"])
            check_parity(oracle, y, ref[:M], K, f"{wt}/{zt} N={N} K={K} M={M} {info}", output_rounding_slack=True)
    finally:
        w.close()
    if w.desc.N % 16 == 0 and K % 128 == 0 and G % 128 == 0:
        assert "fcc_plain" not in seen


def test_scalar_zero_point_and_3d_activations(oracle, dev, req):
    say("scalar zp, 3-D x")
    c = datagen.make_case(5, 6, 256, 128, "u8", 256, "u8", zp_range=(100, 157))
    c.zp = c.zp[:1].copy()
    c.zp_scalar = True
    x3 = c.x.reshape(2, 3, 256)
    y, info = run_case(dev, req, c, x=x3)
    assert y.shape == (2, 3, 128)
    check_parity(oracle, y.reshape(6, 128), oracle_y(oracle, c), 256, str(info), output_rounding_slack=True)
    c4 = datagen.make_case(6, 5, 256, 64, "u4", 128, "u4")
    c4.zp = np.array([0x07], np.uint8)
    c4.zp_scalar = True
    y, info = run_case(dev, req, c4)
    check_parity(oracle, y, oracle_y(oracle, c4), 256, str(info), output_rounding_slack=True)


@pytest.mark.parametrize("M", [1, 24, 70])
@pytest.mark.parametrize("wt,N,K,G", [("u4", 128, 512, 128), ("u8", 128, 256, 256), ("i4", 24, 96, 32)])
def test_f32_output_type(oracle, dev, req, wt, N, K, G, M):
    """output_type f32: same arithmetic, no output cast; the f16 result is its exact rounding."""
    say(f"f32 out {wt} N={N} K={K} M={M}")
    c = datagen.make_case(17, M, K, N, wt, G, "none" if wt == "i4" else wt, with_bias=True)
    w32 = fc.CompressedWeights.from_case(dev, c, output_type="f32")
    w16 = fc.CompressedWeights.from_case(dev, c)
    try:
        y32 = req.infer(w32, c.x)
        y16 = req.infer(w16, c.x)
    finally:
        w32.close()
        w16.close()
    assert y32.dtype == np.float32 and y32.shape == (M, N)
    ref = oracle_y(oracle, c)
    check_parity(oracle, y32, ref, K, "f32 out")
    assert oracle.rel_l2(y32, ref) < 3e-4
    assert np.array_equal(y32.astype(np.float16).view(np.uint16), y16.view(np.uint16))


def test_zero_rows(dev, req):
    say("M = 0")
    c = datagen.make_case(5, 0, 256, 128, "u4", 128, "u4")
    y, _ = run_case(dev, req, c)
    assert y.shape == (0, 128)


@pytest.mark.parametrize("split", [1, 2, 3, 8, 32])
@pytest.mark.parametrize("M", [1, 20])
def test_decode_split_k_is_deterministic(oracle, dev, req, split, M):
    """Any split gives the oracle's answer, and repeated launches give identical bits (the reduction order is
    fixed and the arrival counters return to zero)."""
    say(f"split {split} M={M}")
    c = datagen.make_case(21, M, 4096, 256, "i4", 128, "none")
    w = fc.CompressedWeights.from_case(dev, c)
    ref = oracle_y(oracle, c)
    try:
        req.force_kernel(_lib.KERNEL_DECODE, split)
        first = req.infer(w, c.x)
        info = req.last_kernel()
        # the small-batch kernel raises a forced split until its slice of X fits in LDS
        assert info["split_k"] <= max(1, split) or info["name"].startswith("fcc_batch")
        check_parity(oracle, first, ref, 4096, f"split {split}")
        for _ in range(5):
            assert np.array_equal(req.infer(w, c.x).view(np.uint16), first.view(np.uint16))
    finally:
        req.force_kernel()
        w.close()


def test_kernel_policy(dev, req, monkeypatch):
    say("policy")
    c = datagen.make_case(3, 130, 256, 128, "u4", 128, "u4")
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        assert w.tiled
        req.infer(w, c.x[:1])
        assert req.last_kernel()["name"] == "fcc_gemv_w4"    # one to four rows, 4-bit weights, groups of 128
        req.infer(w, c.x[:5])
        assert req.last_kernel()["name"] == "fcc_gemv16_w4"  # five to 32 rows of such a node, activations fit in LDS
        req.infer(w, c.x[:32])
        assert req.last_kernel()["name"] == "fcc_gemv16_w4"
        monkeypatch.setenv("OVFCC_GEMV16", "0")
        req.infer(w, c.x[:5])
        assert req.last_kernel()["name"] == "fcc_decode_w4"
        req.infer(w, c.x[:32])
        assert req.last_kernel()["name"] == "fcc_batch_w4"
        monkeypatch.delenv("OVFCC_GEMV16")
        req.infer(w, c.x[:48])
        assert req.last_kernel()["name"] == "fcc_gemv16_w4" and req.last_kernel()["grid"][1] == 3
        req.infer(w, c.x[:128])          # three launches of 43, 43 and 42 rows
        assert req.last_kernel()["name"] == "fcc_gemv16_w4" and req.last_kernel()["grid"][1] == 3
        monkeypatch.setenv("OVFCC_GEMV16", "0")
        req.infer(w, c.x[:128])          # ... of the small-batch kernel
        assert req.last_kernel()["kernel"] == _lib.KERNEL_DECODE and req.last_kernel()["tile_m"] == 48
        monkeypatch.delenv("OVFCC_GEMV16")
        req.infer(w, c.x[:129])
        assert req.last_kernel()["kernel"] == _lib.KERNEL_PREFILL
        req.force_kernel(_lib.KERNEL_PLAIN)
        with pytest.raises(fc.OvfccError):
            req.infer(w, c.x[:1])
        req.force_kernel(_lib.KERNEL_DECODE)
        with pytest.raises(fc.OvfccError):
            req.infer(w, c.x[:49])
        req.force_kernel()
        with pytest.raises(fc.OvfccError):
            req.infer(w, c.x[:, :100])
    finally:
        w.close()


def test_mid_row_counts_on_a_wide_node(oracle, dev, req):
    """49..128 rows: where the async prefill kernel's grid (64-row tiles, K split) fills the chip -- here from two
    row tiles on -- one prefill launch, otherwise two or three decode launches; all within the oracle bounds."""
    say("mid row counts")
    c = datagen.make_case(840, 128, 2048, 8192, "u4", 128, "u4", with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    ref = oracle_y(oracle, c)
    try:
        for M, family in ((48, _lib.KERNEL_DECODE), (49, _lib.KERNEL_DECODE), (64, _lib.KERNEL_DECODE),
                          (65, _lib.KERNEL_PREFILL), (96, _lib.KERNEL_PREFILL), (128, _lib.KERNEL_PREFILL)):
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["kernel"] == family, (M, info)
            if family == _lib.KERNEL_PREFILL:
                assert info["name"] == "fcc_prefill_async_w4" and info["tile_m"] == 64 and info["split_k"] > 1, info
            check_parity(oracle, y, ref[:M], c.K, f"M={M} {info}", output_rounding_slack=True)
    finally:
        w.close()


@pytest.mark.parametrize("batch", ["0", "1"])
@pytest.mark.parametrize("wt,zt,N,K,G", [("u4", "u4", 272, 1024, 128), ("i4", "none", 128, 2048, 256),
                                         ("u8", "u8", 144, 512, 512), ("u8", "none", 256, 1024, 128)])
def test_both_decode_kernels_every_row_count(oracle, dev, req, monkeypatch, wt, zt, N, K, G, batch):
    """The streaming kernel (M <= 32) and the small-batch kernel (M <= 48) each forced over their whole range of
    row counts, with channel-tile counts that leave the last workgroup ragged, with and without a forced split."""
    monkeypatch.setenv("OVFCC_DECODE_BATCH", batch)
    monkeypatch.setenv("OVFCC_GEMV", "0")     # one to four rows would otherwise take the matrix-vector kernel
    top = 48 if batch == "1" else 32
    c = datagen.make_case(41, top, K, N, wt, G, zt, with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    ref = oracle_y(oracle, c)
    try:
        for split in (0, 1, 3):
            req.force_kernel(_lib.KERNEL_DECODE, split)
            for M in (1, 4, 5, 15, 16, 17, 31, 32, 33, 47, 48):
                if M > top:
                    continue
                say(f"decode batch={batch} {wt}/{zt} N={N} K={K} split={split} M={M}")
                y = req.infer(w, c.x[:M])
                info = req.last_kernel()
                assert info["name"].startswith("fcc_batch" if batch == "1" else "fcc_decode"), info
                check_parity(oracle, y, ref[:M], K, f"{info}", output_rounding_slack=True)
    finally:
        req.force_kernel()
        w.close()


@pytest.mark.parametrize("variant", ["async", "async64", "ring", "lds"])
@pytest.mark.parametrize("wt,zt,N,K,G,out", [
    ("u4", "u4", 256, 512, 128, "f16"), ("i4", "none", 512, 1024, 256, "f16"), ("u4", "u8", 256, 768, 128, "f32"),
    ("u4", "none", 256, 512, 512, "f16"),            # one group per channel: exact integers, scale in the epilogue
    ("u8", "u8", 256, 512, 512, "f32"), ("u8", "u8", 256, 512, 128, "f16"), ("i8", "none", 512, 256, 128, "f16"),
    ("u8", "none", 256, 1024, 256, "f16"),
])
def test_256_wide_prefill_kernels_small_shapes(oracle, dev, req, monkeypatch, wt, zt, N, K, G, out, variant):
    """The prefill kernels with 256-channel tiles -- register-fed weights with every operand loaded straight into
    LDS (4-bit only), register-fed weights through a register ring, and weights dequantised into LDS -- forced
    onto shapes small enough for the oracle to cover every output: every weight type, zero-point form, scale
    grouping, bias, both output types, row counts that leave the last row tile ragged, odd k-block counts."""
    four_bit = wt in ("u4", "i4")
    if variant.startswith("async") and not four_bit:
        pytest.skip("the all-asynchronous kernel takes 4-bit weights; 8-bit nodes run the register-ring kernel")
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    monkeypatch.setenv("OVFCC_PREFILL_DIRECT", "0" if variant == "lds" else "1")
    monkeypatch.setenv("OVFCC_PREFILL_ASYNC", "1" if variant.startswith("async") else "0")
    monkeypatch.setenv("OVFCC_PREFILL_ROWS", "64" if variant == "async64" else "128")   # tile height of the async kernel
    c = datagen.make_case(51, 300, K, N, wt, G, zt, with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c, output_type=out)
    ref = oracle_y(oracle, c)
    want = {"async": "fcc_prefill_async", "async64": "fcc_prefill_async", "ring": "fcc_prefill_direct",
            "lds": "fcc_prefill_wide"}[variant]
    try:
        for M in (129, 256, 300) + ((49, 64, 65) if variant == "async64" else ()):
            say(f"256-wide prefill {variant} {wt}/{zt} N={N} K={K} G={G} out={out} M={M}")
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            if M <= 128:
                req.force_kernel(_lib.KERNEL_PREFILL)      # the policy would cut these rows into decode launches
                y = req.infer(w, c.x[:M])
                info = req.last_kernel()
                req.force_kernel()
            if variant != "lds" or K % 256 == 0:
                assert info["name"].startswith(want), info
            if variant.startswith("async"):
                assert info["tile_m"] == (64 if variant == "async64" else 128), info
            # grouped scales: these kernels round (q - zp) * s once to f16, an error of the same size as the
            # rounding of an f16 output, so the slack applies to the f32 output as well
            check_parity(oracle, y, ref[:M], K, f"{info}", output_rounding_slack=True)
    finally:
        w.close()


@pytest.mark.parametrize("wt,zt,N,K,G", [("i4", "none", 256, 2048, 128), ("u4", "u4", 512, 1280, 256),
                                         ("u4", "none", 256, 1024, 1024), ("u8", "u8", 256, 1536, 128),
                                         ("i8", "none", 512, 1024, 1024)])
@pytest.mark.parametrize("split", [2, 3, 8])
@pytest.mark.parametrize("rows", ["128", "64"])
def test_prefill_split_k_is_deterministic(oracle, dev, req, monkeypatch, wt, zt, N, K, G, split, rows):
    """The register-fed prefill kernels with K split over workgroups: any split gives the oracle's answer
    (ragged last split, ragged last row tile, bias, per-channel scale in the fix-up), repeated launches give
    identical bits, and the arrival counters return to zero."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    monkeypatch.setenv("OVFCC_PREFILL_ROWS", rows)
    c = datagen.make_case(61, 200, K, N, wt, G, zt, with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    ref = oracle_y(oracle, c)
    try:
        req.force_kernel(_lib.KERNEL_PREFILL, split)
        say(f"prefill split {split} {wt}/{zt} N={N} K={K} G={G}")
        first = req.infer(w, c.x)
        info = req.last_kernel()
        want = "fcc_prefill_async_w4" if wt in ("u4", "i4") else "fcc_prefill_direct_w8"
        assert info["name"] == want and info["split_k"] > 1, info
        check_parity(oracle, first, ref, K, f"{info}", output_rounding_slack=True)
        for _ in range(4):
            assert np.array_equal(req.infer(w, c.x).view(np.uint16), first.view(np.uint16))
        req.force_kernel(_lib.KERNEL_PREFILL, 1)
        one = req.infer(w, c.x)
        assert req.last_kernel()["split_k"] == 1
        check_parity(oracle, one, ref, K, "unsplit", output_rounding_slack=True)
    finally:
        req.force_kernel()
        w.close()


def test_decode_and_prefill_agree(oracle, dev, req):
    """Same inputs through both tiled kernels at M = 32 (full output, every tile)."""
    say("decode vs prefill")
    c = datagen.make_case(31, 32, 4096, 1024, "u4", 128, "u4")
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        req.force_kernel(_lib.KERNEL_DECODE)
        yd = req.infer(w, c.x)
        req.force_kernel(_lib.KERNEL_PREFILL)
        yp = req.infer(w, c.x)
        assert req.last_kernel()["kernel"] == _lib.KERNEL_PREFILL
    finally:
        req.force_kernel()
        w.close()
    ref = oracle_y(oracle, c)
    check_parity(oracle, yd, ref, 4096, "decode")
    check_parity(oracle, yp, ref, 4096, "prefill")
    assert oracle.rel_l2(yd.astype(np.float32), yp.astype(np.float32)) < 1e-3


def test_two_requests_interleaved(oracle, dev):
    """Two requests (streams) over the same weights give the same bits as one."""
    say("two requests")
    c = datagen.make_case(41, 8, 2048, 512, "i4", 128, "none")
    w = fc.CompressedWeights.from_case(dev, c)
    a, b = fc.InferRequest(dev), fc.InferRequest(dev)
    try:
        ya = a.infer(w, c.x)
        yb = b.infer(w, c.x[::-1].copy())
        assert np.array_equal(ya.view(np.uint16), yb[::-1].view(np.uint16))
    finally:
        a.close()
        b.close()
        w.close()


def test_horizontal_fusion_matches_separate_nodes(oracle, dev, req):
    """Q/K/V-style fusion: the fused node's columns equal the separate nodes' outputs (up to the last f16 bit:
    the launch decomposition, and with it the summation order, depends on N) and meet the oracle bounds."""
    say("concat")
    K = 1024
    cases = [datagen.make_case(50 + i, 64, K, n, "u4", 128, "u4", with_bias=True) for i, n in enumerate((256, 128, 128))]
    x = cases[0].x
    parts = [fc.CompressedWeights.from_case(dev, c) for c in cases]
    fused = fc.CompressedWeights.concat(parts)
    try:
        assert fused.N == 512 and fused.tiled
        for M in (1, 4, 64):
            y = req.infer(fused, x[:M]).astype(np.float32)
            sep = np.concatenate([req.infer(p, x[:M]) for p in parts], axis=1).astype(np.float32)
            assert np.all(np.abs(y - sep) <= np.abs(sep) * 2.0 ** -10 + 1e-6)
            ref = np.concatenate([oracle_y(oracle, c, x=x[:M]) for c in cases], axis=1)
            check_parity(oracle, y, ref, K, f"fused M={M}", output_rounding_slack=True)
        other = fc.CompressedWeights.from_case(dev, datagen.make_case(60, 1, 2 * K, 64, "u4", 128, "u4", with_bias=True))
        with pytest.raises(fc.OvfccError):
            fc.CompressedWeights.concat([parts[0], other])
        other.close()
    finally:
        fused.close()
        for p in parts:
            p.close()


GROUPED = [
    # w_type, zp_type, N, K, G, bias, rows per item
    ("u4", "u4", 256, 1024, 128, True, [5, 0, 48, 17, 1]),            # few rows everywhere: small-batch kernel
    ("u8", "u8", 128, 512, 512, False, [3, 33, 16]),                  # 8-bit, per-channel
    ("u4", "u4", 512, 1280, 128, False, [70, 3, 0, 129, 48, 300]),    # more rows: prefill kernel, slices of <= 128 rows
    ("i4", "none", 256, 2048, 2048, True, [64, 65]),                  # per-channel scale in the epilogue
    ("u4", "none", 256, 512, 128, False, [1] * 70 + [100]),           # more slices than one launch holds
    ("u4", "u4", 4096, 256, 128, False, [128] * 32),                  # as one node it would take 256-row tiles
]


@pytest.mark.parametrize("wt,zt,N,K,G,bias,rows", GROUPED)
def test_grouped_run_matches_oracle_and_separate_runs(oracle, dev, req, monkeypatch, wt, zt, N, K, G, bias, rows):
    """A grouped run over nodes of one shape (mixture-of-experts layers: one node per expert, its own weights and
    gathered rows): every item meets the oracle bounds, and repeated runs give identical bits.  (The planner
    would give grids this small to the square prefill kernel, which has no grouped form: the 256-wide one is
    forced.)"""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    say(f"grouped {wt}/{zt} N={N} K={K} G={G} rows={rows[:8]}")
    n_weights = min(len(rows), 6)
    cases = [datagen.make_case(700 + i, max(rows), K, N, wt, G, zt, with_bias=bias) for i in range(n_weights)]
    ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
    try:
        items = [(ws[i % n_weights], cases[i % n_weights].x[:m]) for i, m in enumerate(rows)]
        ys = req.infer_grouped(items)
        info = req.last_kernel()
        assert "grouped" in info["name"], info
        assert ("prefill" in info["name"]) == (max(rows) > 48), info
        for i, (m, y) in enumerate(zip(rows, ys)):
            assert y.shape == (m, N)
            if m:
                c = cases[i % n_weights]
                check_parity(oracle, y, oracle_y(oracle, c, x=c.x[:m]), K, f"item {i} M={m} {info}",
                             output_rounding_slack=True)
        again = req.infer_grouped(items)
        for y, z in zip(ys, again):
            assert np.array_equal(y.view(np.uint16), z.view(np.uint16))
    finally:
        for w in ws:
            w.close()


@pytest.mark.parametrize("wt,zt,G,bias", [("u4", "u4", 128, True), ("i4", "none", 1024, False), ("u4", "u8", 128, False)])
def test_grouped_run_slice_heights(oracle, dev, req, monkeypatch, wt, zt, G, bias):
    """The grouped prefill kernel's four tile heights (64, 80, 96, 128 rows; OVFCC_PREFILL_ROWS) over items whose row
    counts straddle them, K cut in parts or not: every item within the oracle bounds at every height, the same bits
    at every height that does not change the cut along K, and the height the policy picks for these counts."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    rows = [79, 80, 81, 96, 97, 54, 71, 65, 1, 128]
    N, K = 512, 1024
    say(f"grouped slice heights {wt}/{zt} G={G}")
    cases = [datagen.make_case(760 + i, max(rows), K, N, wt, G, zt, with_bias=bias) for i in range(4)]
    ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
    try:
        items = [(ws[i % 4], cases[i % 4].x[:m]) for i, m in enumerate(rows)]
        seen = {}
        for height in (128, 96, 80, 64):
            monkeypatch.setenv("OVFCC_PREFILL_ROWS", str(height))
            ys = req.infer_grouped(items)
            info = req.last_kernel()
            assert info["name"] == "fcc_prefill_async_grouped_w4" and info["tile_m"] == height, info
            for i, (m, y) in enumerate(zip(rows, ys)):
                c = cases[i % 4]
                check_parity(oracle, y, oracle_y(oracle, c, x=c.x[:m]), K, f"height {height} item {i} M={m} {info}",
                             output_rounding_slack=True)
            seen[height] = (info["split_k"], ys)
        for height in (96, 80, 64):
            if seen[height][0] == seen[128][0]:
                for y, z in zip(seen[height][1], seen[128][1]):
                    assert np.array_equal(y.view(np.uint16), z.view(np.uint16)), height
        monkeypatch.delenv("OVFCC_PREFILL_ROWS")
        req.infer_grouped([(ws[0], cases[0].x[:70]), (ws[1], cases[1].x[:66]), (ws[2], cases[2].x[:75])])
        assert req.last_kernel()["tile_m"] == 80, req.last_kernel()
        req.infer_grouped([(ws[0], cases[0].x[:90]), (ws[1], cases[1].x[:66])])
        assert req.last_kernel()["tile_m"] == 96, req.last_kernel()
    finally:
        for w in ws:
            w.close()


def test_grouped_run_falls_back_item_by_item(oracle, dev, req):
    """Items of different shapes, an untiled node, or a forced kernel cannot share a launch: the run still gives
    every item's result (through the ordinary per-node path)."""
    say("grouped fallback")
    a = datagen.make_case(720, 20, 512, 128, "u4", 128, "u4")
    b = datagen.make_case(721, 7, 256, 256, "u8", 128, "u8")
    c = datagen.make_case(722, 9, 200, 40, "u4", 50, "u4")  # untiled
    ws = [fc.CompressedWeights.from_case(dev, k) for k in (a, b, c)]
    try:
        ys = req.infer_grouped([(w, k.x) for w, k in zip(ws, (a, b, c))])
        assert "grouped" not in req.last_kernel()["name"]
        for y, k in zip(ys, (a, b, c)):
            check_parity(oracle, y, oracle_y(oracle, k), k.K, "mixed", output_rounding_slack=True)
        req.force_kernel(_lib.KERNEL_PREFILL)
        y = req.infer_grouped([(ws[0], a.x), (ws[0], a.x[:3])])
        assert req.last_kernel()["kernel"] == _lib.KERNEL_PREFILL and "grouped" not in req.last_kernel()["name"]
        check_parity(oracle, y[0], oracle_y(oracle, a), a.K, "forced", output_rounding_slack=True)
        assert req.infer_grouped([]) == []
        with pytest.raises(fc.OvfccError):
            req.infer_grouped_device([(ws[0], 0, 0, 4)])
    finally:
        req.force_kernel()
        for w in ws:
            w.close()


def test_grouped_run_mixtral_experts(oracle, dev, req):
    """Benchmark configuration 5 at its real shape: the gate matrices of all eight experts over their routed
    tokens in one launch, sampled rows against the oracle."""
    say("grouped mixtral gate")
    routes = datagen.moe_routing()
    cases = [datagen.config5_expert(e, "gate", len(t)) for e, t in enumerate(routes)]
    ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
    try:
        ys = req.infer_grouped([(w, c.x) for w, c in zip(ws, cases)])
        info = req.last_kernel()
        assert info["name"] == "fcc_prefill_async_grouped_w4", info
        for e, (c, y) in enumerate(zip(cases, ys)):
            pick = np.array([0, c.M // 2, c.M - 1])
            check_parity(oracle, y[pick], oracle_y(oracle, c, x=c.x[pick]), c.K, f"expert {e}")
    finally:
        for w in ws:
            w.close()


def test_prefill_splits_only_the_last_partial_round(oracle, dev, req, monkeypatch):
    """More tiles than compute units with a small remainder, OVFCC_PREFILL_TAIL = 1: the whole rounds run unsplit,
    the remaining tiles are cut along K so that the last round fills the chip.  Every row against the numpy oracle
    (itself pinned against the C oracle in the CPU tests), identical bits on repeats, and the unsplit launch."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    monkeypatch.setenv("OVFCC_PREFILL_TAIL", "1")
    M, K, N = 3400, 2048, 2560          # 10 x 27 = 270 tiles of 128 x 256
    say(f"tail split M={M} K={K} N={N}")
    c = datagen.make_case(810, M, K, N, "u4", 128, "u4", with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        y = req.infer(w, c.x)
        info = req.last_kernel()
        n_cus = info["grid"][0] - 270   # (270 - full) * (split - 1) extra workgroups
        assert info["name"] == "fcc_prefill_async_w4" and info["split_k"] > 1 and n_cus > 0, info
        ref = oracle.fc_reference_numpy(c.x, c.w, oracle.U4, c.scale, c.zp, oracle.U4, c.bias, N=N, K=K, group_size=128)
        check_parity(oracle, y, ref, K, f"{info}", output_rounding_slack=True)
        for _ in range(3):
            assert np.array_equal(req.infer(w, c.x).view(np.uint16), y.view(np.uint16))
        monkeypatch.setenv("OVFCC_PREFILL_TAIL", "0")
        whole = req.infer(w, c.x)
        assert req.last_kernel()["split_k"] == 1 and req.last_kernel()["grid"][0] == 270
        check_parity(oracle, whole, ref, K, "unsplit", output_rounding_slack=True)
    finally:
        w.close()


def test_weight_blob_export_import(oracle, dev, req):
    """A node exported as a host blob and imported again gives identical bits (tiled, untiled, fused and
    gated nodes); damaged blobs are refused."""
    say("weight blob")
    tiled = datagen.make_case(830, 40, 512, 256, "u4", 128, "u4", with_bias=True)
    plain = datagen.make_case(831, 9, 200, 40, "u8", 50, "u8")
    scalar = datagen.make_case(832, 5, 256, 64, "u8", 128, "u8")
    scalar.zp, scalar.zp_scalar = np.array([131], np.uint8), True
    ws = [fc.CompressedWeights.from_case(dev, tiled), fc.CompressedWeights.from_case(dev, plain),
          fc.CompressedWeights.from_case(dev, scalar), fc.CompressedWeights.from_case(dev, tiled, glu="swish")]
    ws.append(fc.CompressedWeights.concat([ws[0], ws[0]]))
    xs = [tiled.x, plain.x, scalar.x, tiled.x, tiled.x]
    try:
        for w, x in zip(ws, xs):
            blob = w.export_blob()
            back = fc.CompressedWeights.import_blob(dev, blob)
            try:
                assert (back.N, back.K, back.N_out, back.tiled) == (w.N, w.K, w.N_out, w.tiled)
                assert back.device_bytes == w.device_bytes
                for M in (1, x.shape[0]):
                    assert np.array_equal(req.infer(back, x[:M]).view(np.uint16), req.infer(w, x[:M]).view(np.uint16))
                assert np.array_equal(back.export_blob(), blob)
            finally:
                back.close()
        blob = ws[0].export_blob()
        for damage in ("magic", "version", "short", "shape", "size"):
            bad = blob.copy()
            if damage == "magic":
                bad[0] ^= 1
            elif damage == "version":
                bad[8] += 1
            elif damage == "short":
                bad = bad[:-16]
            elif damage == "shape":
                bad[16:24] = np.frombuffer(np.int64(512).tobytes(), np.uint8)       # N: 256 -> 512
            else:
                bad[16 + 56 + 8:16 + 56 + 16] = np.frombuffer(np.uint64(1 << 40).tobytes(), np.uint8)  # w_bytes
            with pytest.raises(fc.OvfccError):
                fc.CompressedWeights.import_blob(dev, bad)
    finally:
        for w in ws:
            w.close()


def gather_matmul_reference(oracle, cases, A, indices):
    """Y[i, m] = expert indices[m, i] applied to A[i or 0, m]: the op's definition
    (src/common/transformations/src/ov_ops/gather_matmul.cpp:38-130), expert by expert with the FC oracle."""
    M, top_k = indices.shape
    N = cases[0].N
    ref = np.zeros((top_k, M, N), np.float32)
    for e, c in enumerate(cases):
        for i in range(top_k):
            rows = np.nonzero(indices[:, i] == e)[0]
            if rows.size:
                ref[i, rows] = oracle_y(oracle, c, x=A[i if A.shape[0] > 1 else 0, rows])
    return ref


@pytest.mark.parametrize("M,a_batches", [(1, 1), (5, 1), (64, 2), (200, 1), (200, 2)])
def test_gather_matmul(oracle, dev, req, monkeypatch, M, a_batches):
    """GatherMatmulCompressed: eight experts, top-2 routing from seeded logits (uneven loads, some experts idle at
    small M); every output row against the oracle of the expert that the indices name."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    say(f"gather matmul M={M} a_batches={a_batches}")
    E, top_k, K, N = 8, 2, 512, 256
    cases = [datagen.make_case(860 + e, 1, K, N, "u4", 128, "u4", with_bias=True) for e in range(E)]
    ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
    rng = np.random.default_rng(870 + M)
    logits = rng.standard_normal((M, E))
    indices = np.argsort(-logits, axis=1, kind="stable")[:, :top_k].astype(np.int32)
    A = rng.standard_normal((a_batches, M, K)).astype(np.float16)
    try:
        y = req.gather_matmul(ws, A, indices)
        assert y.shape == (top_k, M, N)
        ref = gather_matmul_reference(oracle, cases, A, indices)
        check_parity(oracle, y.reshape(-1, N), ref.reshape(-1, N), K, f"M={M} {req.last_kernel()}",
                     output_rounding_slack=True)
        assert np.array_equal(req.gather_matmul(ws, A, indices).view(np.uint16), y.view(np.uint16))
        bad = indices.copy()
        bad[0, 0] = E
        with pytest.raises(fc.OvfccError):
            req.gather_matmul(ws, A, bad)
        with pytest.raises(fc.OvfccError):
            req.gather_matmul_device(ws, 0, 3, indices, 0)        # a_batches neither 1 nor top_k
    finally:
        for w in ws:
            w.close()


@pytest.mark.parametrize("M,a_batches", [(1, 1), (9, 2), (130, 1), (700, 2)])
def test_gather_matmul_routed_on_the_device(oracle, dev, req, monkeypatch, M, a_batches):
    """GatherMatmulCompressed with the indices in device memory: bucketed by the routing kernel.  Every output row
    against the oracle and, where the host-bucketed call runs the same grouped kernel, bit for bit against it; a
    pair whose index names no expert gets a row of zeros in Y."""
    say(f"gather matmul routed M={M} a_batches={a_batches}")
    E, top_k, K, N = 8, 2, 512, 256
    cases = [datagen.make_case(860 + e, 1, K, N, "u4", 128, "u4", with_bias=True) for e in range(E)]
    ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
    rng = np.random.default_rng(870 + M)
    logits = rng.standard_normal((M, E))
    indices = np.argsort(-logits, axis=1, kind="stable")[:, :top_k].astype(np.int32)
    A = rng.standard_normal((a_batches, M, K)).astype(np.float16)
    try:
        y = req.gather_matmul(ws, A, indices, device_indices=True)
        assert req.last_kernel()["name"] == "fcc_prefill_async_grouped_w4"
        ref = gather_matmul_reference(oracle, cases, A, indices)
        check_parity(oracle, y.reshape(-1, N), ref.reshape(-1, N), K, f"M={M} routed", output_rounding_slack=True)
        bad = indices.copy()
        bad[0, 0], bad[M - 1, 1] = E, -3
        got = req.gather_matmul(ws, A, bad, device_indices=True, y_fill=7.0)
        # the two unrouted pairs' rows read as zeros (not as whatever Y held), every other row is unchanged
        assert np.all(got[0, 0].view(np.uint16) == 0) and np.all(got[1, M - 1].view(np.uint16) == 0)
        got[0, 0], got[1, M - 1] = y[0, 0], y[1, M - 1]
        assert np.array_equal(got.view(np.uint16), y.view(np.uint16))
        monkeypatch.setenv("OVFCC_MOE_HOST_ROUTING", "1")
        monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
        y_host = req.gather_matmul(ws, A, indices)
        if req.last_kernel()["name"] == "fcc_prefill_async_grouped_w4":
            assert np.array_equal(y_host.view(np.uint16), y.view(np.uint16))
        else:                       # few rows per expert: node by node through the decode kernels
            assert M < 700
            check_parity(oracle, y_host.reshape(-1, N), ref.reshape(-1, N), K, f"M={M} host-routed",
                         output_rounding_slack=True)
    finally:
        for w in ws:
            w.close()


def test_requests_on_concurrent_threads(oracle, dev):
    """Different requests may run concurrently from different threads (the reference runs infer requests on a
    task executor): four threads, one request each, shared weights, mixed row counts; every result bit-equal to
    the single-threaded one, errors stay on the thread that caused them."""
    import threading
    say("concurrent threads")
    c = datagen.make_case(880, 300, 1024, 512, "u4", 128, "u4", with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    rows = [1, 7, 40, 100, 300]
    one = fc.InferRequest(dev)
    want = {m: one.infer(w, c.x[:m]) for m in rows}
    one.close()
    failures = []

    def work(tid):
        req = fc.InferRequest(dev)
        try:
            for it in range(20):
                m = rows[(it + tid) % len(rows)]
                y = req.infer(w, c.x[:m])
                if not np.array_equal(y.view(np.uint16), want[m].view(np.uint16)):
                    failures.append((tid, it, m))
                if it % 7 == 3:
                    try:
                        req.infer(w, c.x[:m, :100])
                        failures.append((tid, it, "no error"))
                    except fc.OvfccError as e:
                        if "K" not in str(e):
                            failures.append((tid, it, str(e)))
        except Exception as e:  # noqa: BLE001 - reported below
            failures.append((tid, repr(e)))
        finally:
            req.close()

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    try:
        assert not any(t.is_alive() for t in threads)
        assert not failures, failures[:5]
    finally:
        w.close()


def test_more_rows_than_32_bit_offsets_reach(oracle, dev, req):
    """M K 2 >= 2^31 bytes of activations: the fast kernels address them with 32-bit offsets, so the node runs as
    consecutive row blocks; rows on both sides of the block boundary, the first and the last against the oracle."""
    K, N = 8192, 256
    block = (((1 << 31) - 1) // (2 * K)) & ~127          # 130 944 rows
    M = block + 128 + 300
    say(f"long node M={M} K={K} (block {block})")
    c = datagen.make_case(880, 4096, K, N, "i4", 128, "none", with_bias=True)
    reps = (M + 4095) // 4096
    x = np.tile(c.x, (reps, 1))[:M]
    x[block - 1] *= np.float16(0.5)                      # distinct rows around the boundary
    x[block] *= np.float16(-1.0)
    x[M - 1] *= np.float16(0.25)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        y = req.infer(w, x)
        assert req.last_kernel()["kernel"] == _lib.KERNEL_PREFILL
        pick = np.array([0, 1, 4095, 4096, block - 2, block - 1, block, block + 1, block + 127, block + 128, M - 2, M - 1])
        check_parity(oracle, y[pick], oracle_y(oracle, c, x=x[pick]), K, "long node")
        assert np.array_equal(y[:4096].view(np.uint16), y[4096:8192].view(np.uint16))     # equal rows, equal results
    finally:
        w.close()


def test_plain_kernel_beyond_its_row_axis(oracle, dev, req):
    """More than 65 535 rows on a node that keeps OpenVINO's layout: row blocks again."""
    say("plain kernel, 70 000 rows")
    c = datagen.make_case(881, 1000, 200, 40, "u4", 50, "u4")
    x = np.tile(c.x, (70, 1))
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        y = req.infer(w, x)
        assert req.last_kernel()["name"] == "fcc_plain" and y.shape == (70000, 40)
        pick = np.array([0, 999, 65534, 65535, 65536, 69999])
        check_parity(oracle, y[pick], oracle_y(oracle, c, x=x[pick]), 200, "plain long", output_rounding_slack=True)
    finally:
        w.close()


@pytest.mark.parametrize("wt,zt,N,K,G,scalar_zp", [
    ("u4", "u4", 256, 512, 128, False),      # tiled, zero-point table
    ("i4", "none", 512, 256, 64, False),     # tiled, two groups per k-block
    ("u8", "u8", 64, 256, 256, False),       # tiled, one group per channel
    ("u8", "u8", 128, 256, 128, True),       # scalar zero-point: untouched by the transposition
    ("u4", "u4", 25, 100, 50, False),        # OpenVINO layout (plain kernel), odd N: rows share bytes
    ("i8", "none", 7, 96, 32, False),
])
def test_input_major_constants(oracle, dev, req, wt, zt, N, K, G, scalar_zp):
    """W [K, N] with scales / zero-points [K / G, N] (OVFCC_W_INPUT_MAJOR, a MatMul with transpose_b = false): the
    node is the [N, K] node -- same outputs bit for bit, same exported image -- and meets the oracle bounds."""
    say(f"input-major {wt}/{zt} N={N} K={K} G={G} scalar_zp={scalar_zp}")
    c = datagen.make_case(870, 70, K, N, wt, G, zt, with_bias=True)
    if scalar_zp:
        c.zp, c.zp_scalar = np.array([119], np.uint8), True
    w_kn, s_kn, z_kn = datagen.to_input_major(c)
    a = fc.CompressedWeights.from_case(dev, c)
    b = fc.CompressedWeights(dev, w_kn, s_kn, z_kn, c.bias, N=N, K=K, group_size=G, w_type=wt, zp_type=zt,
                             zp_scalar=c.zp_scalar, input_major=True)
    ref = oracle_y(oracle, c)
    try:
        assert np.array_equal(a.export_blob(), b.export_blob())
        for M in (1, 5, 33, 70):
            ya, yb = req.infer(a, c.x[:M]), req.infer(b, c.x[:M])
            assert np.array_equal(ya.view(np.uint16), yb.view(np.uint16)), M
            check_parity(oracle, yb, ref[:M], K, f"M={M} {req.last_kernel()}", output_rounding_slack=True)
    finally:
        a.close()
        b.close()


def test_device_memory_helpers(dev):
    """malloc / upload / device-to-device copy / download round trip, odd sizes included."""
    say("device memory helpers")
    for n in (1, 17, 4096, (1 << 20) + 3):
        a = np.random.default_rng(n).integers(0, 256, size=n, dtype=np.uint8)
        p, q = dev.malloc(n), dev.malloc(n)
        try:
            dev.upload(p, a)
            dev.copy(q, p, n)
            assert np.array_equal(dev.download(q, (n,), np.uint8), a)
        finally:
            dev.free(p)
            dev.free(q)


@pytest.mark.parametrize("wt,zt,zp_top", [("i8", "u8", 255), ("i4", "u8", 255), ("i4", "u4", 15)])
def test_signed_weights_with_zero_points(oracle, dev, req, wt, zt, zp_top):
    """Signed weights with per-group zero-points, zero-points at the top of their range included: the stored form is
    unsigned with the zero-point raised by 8 / 128, which fits the tiled table's byte only for 4-bit zero-points;
    the other two keep OpenVINO's layout and run the plain kernel."""
    say(f"signed weights with zero-points {wt}/{zt}")
    c = datagen.make_case(3100, 20, 512, 64, wt, 128, zt, with_bias=True)
    zp = c.zp.copy()
    if zt == "u8":
        zp.reshape(-1)[::3] = zp_top            # 255: beyond what one byte holds once the offset is added
        zp.reshape(-1)[1::3] = 200
    else:
        zp[:] = 0xFF                            # every 4-bit zero-point 15
    c = datagen.FcCase(c.M, c.K, c.N, c.group_size, c.w_type, c.zp_type, c.w, c.scale, zp, c.x, c.bias)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        assert w.tiled == (zt == "u4")
        ref = oracle_y(oracle, c)
        for M in (1, 5, 20):
            y = req.infer(w, c.x[:M])
            check_parity(oracle, y, ref[:M], c.K, f"M={M} {req.last_kernel()}", output_rounding_slack=True)
    finally:
        w.close()


def test_grouped_run_with_different_scalar_zero_points(oracle, dev, req):
    """Experts whose scalar zero-points differ agree in every descriptor field (the scalar lives beside it): they
    must not share a grouped launch, which carries one constant for all; each still gets its own result."""
    say("grouped, scalar zero-points differ")
    cases, ws = [], []
    for i, zpv in enumerate((3, 11, 7)):
        c = datagen.make_case(3200 + i, 24, 512, 256, "u4", 128, "u8", with_bias=False)
        c = datagen.FcCase(c.M, c.K, c.N, c.group_size, c.w_type, "u8", c.w, c.scale, np.array([zpv], np.uint8), c.x,
                           None, zp_scalar=True)
        cases.append(c)
        ws.append(fc.CompressedWeights.from_case(dev, c))
    try:
        ys = req.infer_grouped([(w, c.x) for w, c in zip(ws, cases)])
        assert "grouped" not in req.last_kernel()["name"]
        for y, c in zip(ys, cases):
            check_parity(oracle, y, oracle_y(oracle, c), c.K, "scalar zp per expert", output_rounding_slack=True)
        same = req.infer_grouped([(ws[1], cases[1].x), (ws[1], cases[1].x[:9])])   # equal constants: one launch
        assert "grouped" in req.last_kernel()["name"]
        check_parity(oracle, same[1], oracle_y(oracle, cases[1], x=cases[1].x[:9]), 512, "equal scalar zp",
                     output_rounding_slack=True)
    finally:
        for w in ws:
            w.close()


def test_grouped_run_more_than_64_slices(oracle, dev, req):
    """More slices than one grouped launch carries (64): the list runs in batches, and a short last batch for which
    the planner picks no grouped kernel runs slice by slice -- every item still gets its result."""
    say("grouped, 70 items")
    c = datagen.make_case(3300, 12, 512, 128, "u4", 128, "u4", with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        rows = [1 + (i * 5) % 12 for i in range(70)]
        ys = req.infer_grouped([(w, c.x[:m]) for m in rows])
        ref = oracle_y(oracle, c)
        for m, y in zip(rows, ys):
            check_parity(oracle, y, ref[:m], c.K, f"M={m}", output_rounding_slack=True)
    finally:
        w.close()
    # prefill row counts: 64 slices fill the chip with 256-wide tiles and share a launch, the remaining six do not
    c = datagen.make_case(3301, 64, 1024, 512, "u4", 128, "u4", with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        rows = [50 + i % 15 for i in range(70)]
        ys = req.infer_grouped([(w, c.x[:m]) for m in rows])
        say(f"   last launch: {req.last_kernel()['name']}")
        assert "grouped" not in req.last_kernel()["name"]       # the tail ran slice by slice
        ref = oracle_y(oracle, c)
        for m, y in zip(rows, ys):
            check_parity(oracle, y, ref[:m], c.K, f"M={m}", output_rounding_slack=True)
    finally:
        w.close()
