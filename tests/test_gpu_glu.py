"""GPU parity of nodes with a fused gated-linear-unit epilogue (SwiGLU and its Gelu variants) against the CPU oracle,
through every kernel family."""
import sys

import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc
from parity import check_parity, glu_reference

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


MS = [1, 3, 4, 5, 16, 17, 33, 48, 49, 100, 130, 300]
CASES = [
    # w_type, zp_type, N (= 2 L), K, G, bias, glu, gate_second
    ("u4", "u4", 512, 1024, 128, True, "swish", False),
    ("i4", "none", 256, 2048, 128, False, "swish", True),
    ("u4", "none", 512, 512, 512, True, "gelu", False),        # one group per channel: scale in the epilogue
    ("u8", "u8", 256, 512, 128, True, "gelu_tanh", False),
    ("u8", "none", 512, 768, 768, False, "swish", True),
    ("u4", "u4", 96, 256, 128, True, "swish", False),          # tiled, N % 128 != 0: decode kernels in chunks
    ("u4", "u4", 40, 200, 50, True, "gelu", True),             # untiled: plain kernel
]


def run_rows(oracle, req, w, c, kind, second, what, rows=MS):
    seen = set()
    for M in rows:
        y = req.infer(w, c.x[:M])
        info = req.last_kernel()
        seen.add(info["name"])
        assert y.shape == (M, c.N // 2)
        ref, amp = glu_reference(oracle, c, kind, second, x=c.x[:M])
        check_parity(oracle, y, ref, c.K, f"{what} M={M} {info}", output_rounding_slack=True, limit_scale=amp)
    return seen


@pytest.mark.parametrize("wt,zt,N,K,G,bias,kind,second", CASES)
def test_glu_every_row_count(oracle, dev, req, wt, zt, N, K, G, bias, kind, second):
    say(f"glu {kind} second={second} {wt}/{zt} N={N} K={K} G={G}")
    c = datagen.make_case(900, max(MS), K, N, wt, G, zt, with_bias=bias)
    w = fc.CompressedWeights.from_case(dev, c, glu=kind, glu_gate_second=second)
    try:
        assert w.N_out == N // 2
        seen = run_rows(oracle, req, w, c, kind, second, "auto")
        say(f"   kernels: {sorted(seen)}")
    finally:
        w.close()


@pytest.mark.parametrize("variant", ["async", "async128", "ring", "lds"])
@pytest.mark.parametrize("wt,zt,N,K,G,kind", [("u4", "u4", 512, 1024, 128, "swish"), ("i4", "none", 512, 512, 512, "gelu"),
                                             ("u8", "u8", 512, 512, 128, "swish"), ("u8", "none", 256, 512, 512, "gelu_tanh")])
def test_glu_256_wide_prefill_kernels(oracle, dev, req, monkeypatch, wt, zt, N, K, G, kind, variant):
    """The three prefill kernels with 128 x 256 tiles, forced on small shapes (the planner would pick the square one)."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    if variant == "async128":     # the planner gives grids this small 64-row tiles; cover the 128-row form too
        if wt[1] == "8":
            pytest.skip("8-bit nodes run the register-ring kernel")
        monkeypatch.setenv("OVFCC_PREFILL_ROWS", "128")
        variant = "async"
    if variant == "ring":
        monkeypatch.setenv("OVFCC_PREFILL_ASYNC", "0")
    if variant == "lds":
        monkeypatch.setenv("OVFCC_PREFILL_DIRECT", "0")
    say(f"glu wide {variant} {kind} {wt}/{zt} N={N} K={K} G={G}")
    c = datagen.make_case(910, 300, K, N, wt, G, zt, with_bias=True)
    for out in ("f16", "f32"):
        w = fc.CompressedWeights.from_case(dev, c, output_type=out, glu=kind)
        try:
            seen = run_rows(oracle, req, w, c, kind, False, f"{variant} {out}", rows=[129, 300])
            want = {"async": "fcc_prefill_async_w4", "ring": f"fcc_prefill_direct_w{wt[1]}", "lds": f"fcc_prefill_wide_w{wt[1]}"}
            if wt[1] == "8" and variant == "async":
                want["async"] = "fcc_prefill_direct_w8"
            assert seen == {want[variant]}, seen
            if variant == "async" and wt[1] == "4":
                req.force_kernel(_lib.KERNEL_PREFILL, 3)     # split-K: the epilogue runs in the fix-up
                y = req.infer(w, c.x)
                assert req.last_kernel()["split_k"] > 1
                ref, amp = glu_reference(oracle, c, kind)
                check_parity(oracle, y, ref, K, "split-K", output_rounding_slack=True, limit_scale=amp)
                assert np.array_equal(req.infer(w, c.x).view(np.uint8), y.view(np.uint8))
        finally:
            req.force_kernel()
            w.close()


def test_glu_from_two_nodes_equals_concatenated_constants(oracle, dev, req):
    """ovfcc_weights_glu(gate, up) gives the bits of the node created from the concatenated constants."""
    say("glu from parts")
    K, L = 1024, 256
    g = datagen.make_case(920, 64, K, L, "u4", 128, "u4", with_bias=True)
    u = datagen.make_case(921, 64, K, L, "u4", 128, "u4", with_bias=True)
    both = datagen.FcCase(64, K, 2 * L, 128, "u4", "u4", np.concatenate([g.w, u.w]), np.concatenate([g.scale, u.scale]),
                          np.concatenate([g.zp, u.zp]), g.x, np.concatenate([g.bias, u.bias]))
    wg, wu = fc.CompressedWeights.from_case(dev, g), fc.CompressedWeights.from_case(dev, u)
    fused = fc.CompressedWeights.glu(wg, wu, "swish")
    whole = fc.CompressedWeights.from_case(dev, both, glu="swish")
    try:
        assert fused.N_out == L and fused.tiled
        for M in (1, 4, 20, 64):
            a, b = req.infer(fused, g.x[:M]), req.infer(whole, g.x[:M])
            assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
            ref, amp = glu_reference(oracle, both, "swish", x=g.x[:M])
            check_parity(oracle, a, ref, K, f"parts M={M}", output_rounding_slack=True, limit_scale=amp)
            # and the unfused graph: two nodes, then the unit on their f16 outputs
            yg, yu = req.infer(wg, g.x[:M]).astype(np.float32), req.infer(wu, g.x[:M]).astype(np.float32)
            sep = oracle.glu(np.concatenate([yg, yu], axis=1), 1)
            assert oracle.rel_l2(a.astype(np.float32), sep) < 1e-3
        with pytest.raises(fc.OvfccError):
            fc.CompressedWeights.glu(fused, wu)
        with pytest.raises(fc.OvfccError):
            fc.CompressedWeights.concat([fused, fused])
    finally:
        for w in (wg, wu, fused, whole):
            w.close()


def test_glu_llama_gate_up(oracle, dev, req):
    """Llama-3-8B gate/up (4096 -> 2 x 14336, int4 g128) with SwiGLU at decode and prefill row counts, sampled rows."""
    say("glu llama gate/up")
    c = datagen.config3("gate_up", 512)
    u = datagen.make_case(931, 1, c.K, c.N, "i4", 128, "none")
    wg = fc.CompressedWeights.from_case(dev, c)
    wu = fc.CompressedWeights.from_case(dev, u)
    fused = fc.CompressedWeights.glu(wg, wu, "swish")
    both = datagen.FcCase(512, c.K, 2 * c.N, 128, "i4", "none", np.concatenate([c.w, u.w]),
                          np.concatenate([c.scale, u.scale]), None, c.x, None)
    try:
        for M in (1, 4, 32, 512):
            y = req.infer(fused, c.x[:M])
            info = req.last_kernel()
            pick = np.unique(np.array([0, M // 2, M - 1]))
            ref, amp = glu_reference(oracle, both, "swish", x=c.x[:M][pick])
            r = check_parity(oracle, y[pick], ref, c.K, f"M={M} {info}", output_rounding_slack=True, limit_scale=amp)
            say(f"   M={M}: {info['name']} rel-L2={r[0]:.2e} max-abs={r[1]:.2e}")
    finally:
        for w in (wg, wu, fused):
            w.close()


def test_glu_grouped_run(oracle, dev, req, monkeypatch):
    """Experts with fused SwiGLU in one grouped launch (prefill kernel), and with few rows (item-by-item fallback:
    the grouped small-batch kernel has no gated form)."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    say("glu grouped")
    K, N = 1024, 512
    cases = [datagen.make_case(940 + i, 100, K, N, "u4", 128, "u4", with_bias=True) for i in range(3)]
    ws = [fc.CompressedWeights.from_case(dev, c, glu="swish") for c in cases]
    try:
        for rows, grouped in (([100, 7, 64], True), ([5, 20, 1], False)):
            ys = req.infer_grouped([(w, c.x[:m]) for w, c, m in zip(ws, cases, rows)])
            info = req.last_kernel()
            assert ("grouped" in info["name"]) == grouped, info
            for c, m, y in zip(cases, rows, ys):
                assert y.shape == (m, N // 2)
                ref, amp = glu_reference(oracle, c, "swish", x=c.x[:m])
                check_parity(oracle, y, ref, K, f"rows {rows} {info}", output_rounding_slack=True, limit_scale=amp)
    finally:
        for w in ws:
            w.close()


def test_glu_gather_matmul(oracle, dev, req, monkeypatch):
    """A mixture-of-experts gate/up stage with fused SwiGLU through the GatherMatmulCompressed entry point."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    say("glu gather matmul")
    E, top_k, K, N, M = 4, 2, 512, 512, 150
    cases = [datagen.make_case(950 + e, 1, K, N, "i4", 128, "none") for e in range(E)]
    ws = [fc.CompressedWeights.from_case(dev, c, glu="swish") for c in cases]
    rng = np.random.default_rng(951)
    indices = np.argsort(-rng.standard_normal((M, E)), axis=1, kind="stable")[:, :top_k].astype(np.int32)
    A = rng.standard_normal((1, M, K)).astype(np.float16)
    try:
        y = req.gather_matmul(ws, A, indices)
        assert y.shape == (top_k, M, N // 2)
        for e, c in enumerate(cases):
            for i in range(top_k):
                rows = np.nonzero(indices[:, i] == e)[0]
                if rows.size:
                    ref, amp = glu_reference(oracle, c, "swish", x=A[0, rows])
                    check_parity(oracle, y[i, rows], ref, K, f"expert {e} slot {i}", output_rounding_slack=True,
                                 limit_scale=amp)
    finally:
        for w in ws:
            w.close()
