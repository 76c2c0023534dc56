"""GPU parity of 4-bit nodes with groups of 64 and 32 inputs -- two and four groups per 128-input k-block, the group
sizes of the reference's own decompression tests besides 128
(src/plugins/intel_cpu/tests/functional/custom/subgraph_tests/src/x64/matmul_weights_decompression.cpp:37-120) --
against the CPU oracle, through every kernel family that carries them: streaming decode, small-batch decode,
all-asynchronous prefill (both tile heights, split-K, grouped), square prefill, with every zero-point form and the
gated-linear-unit epilogue.  Bounds as everywhere: rel-L2 <= 1e-3, max-abs <= 2e-2 sqrt(K / 4096)."""
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


MS = [1, 2, 3, 4, 5, 15, 16, 17, 31, 32, 33, 48, 49, 63, 65, 128, 130, 257]
SHAPES = [
    # w_type, zp_type, N, K, bias
    ("u4", "u4", 128, 512, False), ("i4", "none", 256, 256, True), ("u4", "u8", 384, 384, False),
    ("u4", "none", 48, 256, True),        # N % 128 != 0: decode kernels in chunks
    ("i4", "u4", 512, 1024, True),
]


def run_rows(oracle, req, w, c, ref, rows, what):
    seen = set()
    for M in rows:
        y = req.infer(w, c.x[:M])
        info = req.last_kernel()
        seen.add(info["name"])
        check_parity(oracle, y, ref[:M], c.K, f"{what} M={M} {info}", output_rounding_slack=True)
    return seen


@pytest.mark.parametrize("G", [32, 64])
@pytest.mark.parametrize("wt,zt,N,K,bias", SHAPES)
def test_every_row_count(oracle, dev, req, wt, zt, N, K, bias, G):
    say(f"small groups {wt}/{zt} N={N} K={K} G={G}")
    c = datagen.make_case(1200 + G, max(MS), K, N, wt, G, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        assert w.tiled
        seen = run_rows(oracle, req, w, c, oracle_y(oracle, c), MS, f"{wt}/{zt} N={N} K={K} G={G}")
        say(f"   kernels: {sorted(seen)}")
        assert "fcc_plain" not in seen
    finally:
        w.close()


def test_groups_that_stay_untiled(oracle, dev, req):
    """Groups of 16 inputs, and groups below 128 inputs under 8-bit weights, keep OpenVINO's layout and the plain kernel."""
    for wt, zt, G in (("u4", "u4", 16), ("u8", "u8", 64), ("i8", "none", 32)):
        say(f"untiled {wt} G={G}")
        c = datagen.make_case(1210, 20, 256, 64, wt, G, zt)
        w = fc.CompressedWeights.from_case(dev, c)
        try:
            assert not w.tiled
            seen = run_rows(oracle, req, w, c, oracle_y(oracle, c), [1, 20], f"{wt} G={G}")
            assert seen == {"fcc_plain"}
        finally:
            w.close()


VARIANTS = {
    # name: (environment, rows, expected kernel)
    "streaming": ({"OVFCC_DECODE_BATCH": "0"}, [1, 2, 4, 5, 9, 16, 17, 32], "fcc_decode_w4"),
    "streaming_rt2": ({"OVFCC_DECODE_BATCH": "0", "OVFCC_DECODE_RT": "2"}, [1, 3, 4], "fcc_decode_w4"),
    "streaming_rt4": ({"OVFCC_DECODE_BATCH": "0", "OVFCC_DECODE_RT": "4"}, [1, 4], "fcc_decode_w4"),
    "streaming_l2": ({"OVFCC_DECODE_BATCH": "0", "OVFCC_DECODE_XLDS": "0"}, [1, 4], "fcc_decode_w4"),
    "batch": ({"OVFCC_DECODE_BATCH": "1"}, [1, 5, 16, 17, 32, 33, 48], "fcc_batch_w4"),
    "batch_rt2": ({"OVFCC_DECODE_BATCH": "1", "OVFCC_DECODE_RT": "2"}, [3, 16, 40], "fcc_batch_w4"),
    "batch_4waves": ({"OVFCC_DECODE_BATCH": "1", "OVFCC_DECODE_WAVES": "4"}, [7, 48], "fcc_batch_w4"),
    "async64": ({"OVFCC_PREFILL_WIDE": "1", "OVFCC_PREFILL_ROWS": "64"}, [49, 64, 129, 300], "fcc_prefill_async_w4"),
    "async128": ({"OVFCC_PREFILL_WIDE": "1", "OVFCC_PREFILL_ROWS": "128"}, [49, 128, 129, 300], "fcc_prefill_async_w4"),
    "square": ({"OVFCC_PREFILL_WIDE": "0"}, [49, 128, 129, 300], "fcc_prefill_w4"),
    "no_async": ({"OVFCC_PREFILL_WIDE": "1", "OVFCC_PREFILL_ASYNC": "0"}, [129, 300], "fcc_prefill_w4"),
}


@pytest.mark.parametrize("variant", sorted(VARIANTS))
@pytest.mark.parametrize("G,zt,scalar", [(32, "u4", False), (64, "u4", False), (32, "none", False), (64, "u8", False),
                                        (32, "u4", True), (64, "u8", True)])
def test_each_kernel_variant(oracle, dev, req, monkeypatch, G, zt, scalar, variant):
    env, rows, want = VARIANTS[variant]
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    N, K = 512, 1024
    say(f"small groups {variant} G={G} zp={zt} scalar={scalar}")
    c = datagen.make_case(1220 + G, max(rows), K, N, "u4" if zt != "none" else "i4", G, zt, with_bias=True)
    if scalar:
        c.zp = np.array([0x09], np.uint8) if zt == "u4" else np.array([11], np.uint8)
        c.zp_scalar = True
    ref = oracle_y(oracle, c)
    for out in ("f16", "f32"):
        w = fc.CompressedWeights.from_case(dev, c, output_type=out)
        try:
            force = _lib.KERNEL_PREFILL if want.startswith("fcc_prefill") else _lib.KERNEL_DECODE
            req.force_kernel(force)
            seen = run_rows(oracle, req, w, c, ref, rows, f"{variant} G={G} {zt} {out}")
            assert seen == {want}, seen
            if variant in ("streaming", "batch", "async64", "async128"):
                # split-K: any split gives the oracle's answer, the same bits on every launch
                for split in (2, 3):
                    req.force_kernel(force, split)
                    M = rows[-1]
                    y = req.infer(w, c.x[:M])
                    info = req.last_kernel()
                    assert info["split_k"] > 1, info
                    check_parity(oracle, y, ref[:M], K, f"{variant} split {split} {info}", output_rounding_slack=True)
                    assert np.array_equal(req.infer(w, c.x[:M]).view(np.uint8), y.view(np.uint8))
        finally:
            req.force_kernel()
            w.close()


@pytest.mark.parametrize("G", [32, 64])
@pytest.mark.parametrize("kind,second", [("swish", False), ("gelu_tanh", True)])
def test_gated_linear_unit(oracle, dev, req, monkeypatch, G, kind, second):
    """SwiGLU / GeGLU epilogue over small groups, all row counts; then the 256-wide prefill kernel forced."""
    N, K = 512, 512
    say(f"small groups glu {kind} second={second} G={G}")
    c = datagen.make_case(1240 + G, 300, K, N, "u4", G, "u4", with_bias=True)
    w = fc.CompressedWeights.from_case(dev, c, glu=kind, glu_gate_second=second)
    ref, amp = glu_reference(oracle, c, kind, second)
    try:
        seen = set()
        for wide in (None, "1"):
            if wide:
                monkeypatch.setenv("OVFCC_PREFILL_WIDE", wide)
            for M in (1, 3, 4, 5, 16, 17, 48, 49, 130, 300):
                y = req.infer(w, c.x[:M])
                info = req.last_kernel()
                seen.add(info["name"])
                assert y.shape == (M, N // 2)
                check_parity(oracle, y, ref[:M], K, f"glu G={G} M={M} {info}", output_rounding_slack=True,
                             limit_scale=amp)
        say(f"   kernels: {sorted(seen)}")
        assert {"fcc_decode_w4", "fcc_batch_w4", "fcc_prefill_w4", "fcc_prefill_async_w4"} <= seen, seen
    finally:
        w.close()


@pytest.mark.parametrize("G", [32, 64])
@pytest.mark.parametrize("rows", [[3, 40, 0, 17, 48], [100, 64, 128, 1], [30, 64, 2, 50]])
def test_grouped_run_and_gather_matmul(oracle, dev, req, monkeypatch, G, rows):
    """The grouped forms of the small-batch and the all-asynchronous kernel (mixture-of-experts layers)."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    N, K = 512, 1024
    say(f"small groups grouped G={G} rows={rows}")
    cases = [datagen.make_case(1260 + i, max(rows), K, N, "u4", G, "u4", with_bias=True) for i in range(len(rows))]
    ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
    try:
        ys = req.infer_grouped([(w, c.x[:m]) for w, c, m in zip(ws, cases, rows)])
        info = req.last_kernel()
        assert "grouped" in info["name"], info
        for i, (m, y, c) in enumerate(zip(rows, ys, cases)):
            if m:
                check_parity(oracle, y, oracle_y(oracle, c, x=c.x[:m]), K, f"item {i} M={m} {info}",
                             output_rounding_slack=True)
        # GatherMatmulCompressed over the same experts, top-2 routing
        M, E = 40, len(ws)
        rng = np.random.default_rng(1270 + G)
        indices = np.argsort(-rng.standard_normal((M, E)), axis=1, kind="stable")[:, :2].astype(np.int32)
        A = rng.standard_normal((1, M, K)).astype(np.float16)
        y = req.gather_matmul(ws, A, indices)
        for s in range(2):
            for m in range(M):
                c = cases[indices[m, s]]
                check_parity(oracle, y[s, m:m + 1], oracle_y(oracle, c, x=A[0, m:m + 1]), K, f"gather slot {s} row {m}",
                             output_rounding_slack=True)
    finally:
        for w in ws:
            w.close()


@pytest.mark.parametrize("G", [32, 64])
def test_concat_blob_and_clone(oracle, dev, req, G):
    """Horizontal fusion, export / import and clone keep the small-group parameter layout intact."""
    say(f"small groups concat / blob G={G}")
    K = 512
    parts = [datagen.make_case(1280 + i, 20, K, n, "u4", G, "u4", with_bias=True) for i, n in enumerate((128, 32, 96))]
    for p in parts[1:]:
        p.x = parts[0].x
    ws = [fc.CompressedWeights.from_case(dev, c) for c in parts]
    fused = fc.CompressedWeights.concat(ws)
    blob = fused.export_blob()
    back = fc.CompressedWeights.import_blob(dev, blob)
    twin = back.clone()
    try:
        ref = np.concatenate([oracle_y(oracle, c) for c in parts], axis=1)
        y = req.infer(fused, parts[0].x)
        check_parity(oracle, y, ref, K, f"concat {req.last_kernel()}", output_rounding_slack=True)
        for other in (back, twin):
            assert np.array_equal(req.infer(other, parts[0].x).view(np.uint16), y.view(np.uint16))
    finally:
        for w in ws + [fused, back, twin]:
            w.close()


@pytest.mark.parametrize("G", [32, 64])
def test_llama_kv_projection(oracle, dev, req, G):
    """A real shape (K = 4096, N = 1024, symmetric int4) at the benchmark distributions: M = 1, 32 and 2048 within
    the unrelaxed bounds."""
    say(f"small groups llama k/v G={G}")
    c = datagen.make_case(1290 + G, 2048, 4096, 1024, "i4", G, "none")
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        for M in (1, 32, 2048):
            pick = np.arange(M) if M <= 32 else np.array([0, 1, 63, 64, 127, 128, 1000, 2047])
            y = req.infer(w, c.x[:M])
            check_parity(oracle, y[pick], oracle_y(oracle, c, x=c.x[:M][pick]), 4096, f"M={M} {req.last_kernel()}")
    finally:
        w.close()
