"""GPU parity of the mixture-of-experts block (MOECompressed with three projections per expert) through the C ABI
against the oracle's composition of FullyConnected, gated linear unit and routing-weighted sum."""
import numpy as np
import pytest

from openvino_amd import datagen, fc
from parity import REL_L2_MAX, max_abs_limit
from test_oracle_moe import expert_args, make_layer, routed

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


def check(oracle, y, ref, K, what):
    """The FullyConnected bounds, widened for two projections in a row and the f16 rounding of the result: the
    down projection's bound counts twice (its own arithmetic, and the error its input carries from the gate/up
    projection, which |down| <= 1 per unit of input here keeps below the same bound)."""
    y = np.asarray(y, np.float32)
    assert y.shape == ref.shape and np.all(np.isfinite(y)), what
    rl2, mab = oracle.rel_l2(y, ref), oracle.max_abs(y, ref)
    limit = 2 * max_abs_limit(K) + float(np.max(np.abs(ref))) * 2.0 ** -11 if ref.size else 0.0
    assert rl2 <= 2 * REL_L2_MAX, f"{what}: rel-L2 {rl2:.3e}"
    assert mab <= limit, f"{what}: max-abs {mab:.3e} > {limit:.3e}"


@pytest.mark.parametrize("M", [1, 7, 48, 300])
@pytest.mark.parametrize("wt,zt,G,kind,out", [("u4", "u4", 128, "swish", "f16"), ("i4", "none", 128, "gelu_tanh", "f32"),
                                              ("u8", "u8", 256, "swish", "f16")])
def test_moe_block(oracle, dev, req, monkeypatch, M, wt, zt, G, kind, out):
    """Eight experts, top-2 routing from seeded logits (uneven loads; idle experts at small M), softmax weights:
    every output row against the oracle; a second call gives the same bits; one-hot routing gives the named
    expert's own FullyConnected chain bit for bit."""
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    E, top_k, H, I = 8, 2, 256, 512
    say(f"moe {wt}/{zt} G={G} {kind} out={out} M={M}")
    gu, dn = make_layer(930, E, H, I, wt=wt, zt=zt, G=G)
    wg = [fc.CompressedWeights.from_case(dev, c, glu=kind) for c in gu]
    wd = [fc.CompressedWeights.from_case(dev, c, output_type=out) for c in dn]
    idx, routing = routed(931 + M, M, E, top_k)
    x = np.random.default_rng(932).standard_normal((M, H)).astype(np.float16)
    glu_type = {"swish": 1, "gelu": 2, "gelu_tanh": 3}[kind]
    try:
        y = req.moe(wg, wd, x, routing, idx)
        assert y.shape == (M, H) and y.dtype == (np.float32 if out == "f32" else np.float16)
        ref = oracle.moe_reference(x, routing, idx, [expert_args(c) for c in gu], [expert_args(c) for c in dn], glu_type)
        check(oracle, y, ref, max(H, I), f"M={M} {req.last_kernel()}")
        assert np.array_equal(req.moe(wg, wd, x, routing, idx).view(np.uint8), y.view(np.uint8))
        # one-hot routing: selection 1 alone; equals that expert's two nodes run one after the other
        one = np.zeros_like(routing)
        one[:, 1] = 1
        y1 = req.moe(wg, wd, x, one, idx)
        for m in range(min(M, 5)):
            e = int(idx[m, 1])
            chain = req.infer(wd[e], req.infer(wg[e], x[m:m + 1]))
            assert oracle.rel_l2(y1[m:m + 1].astype(np.float32), chain.astype(np.float32)) < 2e-3, (m, e)
    finally:
        for w in wg + wd:
            w.close()


def test_moe_rejects_what_it_cannot_run(oracle, dev, req):
    E, H, I = 4, 128, 256
    gu, dn = make_layer(940, E, H, I)
    wg = [fc.CompressedWeights.from_case(dev, c, glu="swish") for c in gu]
    wd = [fc.CompressedWeights.from_case(dev, c) for c in dn]
    plain_gate = [fc.CompressedWeights.from_case(dev, c) for c in gu]          # no gated linear unit
    idx, routing = routed(941, 6, E, 2)
    x = np.zeros((6, H), np.float16)
    try:
        with pytest.raises(fc.OvfccError):
            req.moe(plain_gate, wd, x, routing, idx)
        with pytest.raises(fc.OvfccError):
            req.moe(wg, wg, x, routing, idx)                                   # down nodes of the wrong shape
        bad = idx.copy()
        bad[2, 1] = E
        with pytest.raises(fc.OvfccError):
            req.moe(wg, wd, x, routing, bad)
        assert req.moe(wg, wd, x[:0], routing[:0], idx[:0]).shape == (0, H)
        y = req.moe(wg, wd, x, routing, idx)                                   # zero input: biases only, finite
        assert np.all(np.isfinite(y.astype(np.float32)))
    finally:
        for w in wg + wd + plain_gate:
            w.close()


@pytest.mark.parametrize("M", [1, 7, 48, 300, 1100])
@pytest.mark.parametrize("wt,zt,G,kind,out", [("u4", "u4", 128, "swish", "f16"), ("i4", "none", 128, "gelu_tanh", "f32")])
def test_moe_block_routed_on_the_device(oracle, dev, req, monkeypatch, M, wt, zt, G, kind, out):
    """The same block with the indices in device memory: the buckets are cut by the routing kernel.  Against the
    oracle, and against the call that buckets on the host: bit for bit where that call also runs the grouped
    prefill kernel (a row's result does not depend on the slice it sits in), otherwise -- few rows per expert run
    node by node through the decode kernels -- within the rounding of the f16 results."""
    E, top_k, H, I = 8, 2, 256, 512
    say(f"moe routed {wt}/{zt} G={G} {kind} out={out} M={M}")
    gu, dn = make_layer(930, E, H, I, wt=wt, zt=zt, G=G)
    wg = [fc.CompressedWeights.from_case(dev, c, glu=kind) for c in gu]
    wd = [fc.CompressedWeights.from_case(dev, c, output_type=out) for c in dn]
    idx, routing = routed(931 + M, M, E, top_k)
    x = np.random.default_rng(932).standard_normal((M, H)).astype(np.float16)
    glu_type = {"swish": 1, "gelu": 2, "gelu_tanh": 3}[kind]
    try:
        y = req.moe(wg, wd, x, routing, idx, device_indices=True)
        assert req.last_kernel()["name"] == "fcc_prefill_async_grouped_w4"
        ref = oracle.moe_reference(x, routing, idx, [expert_args(c) for c in gu], [expert_args(c) for c in dn], glu_type)
        check(oracle, y, ref, max(H, I), f"M={M} routed")
        assert np.array_equal(req.moe(wg, wd, x, routing, idx, device_indices=True).view(np.uint8), y.view(np.uint8))
        assert np.array_equal(req.moe(wg, wd, x, routing, idx).view(np.uint8), y.view(np.uint8))  # uploads, then routes
        monkeypatch.setenv("OVFCC_MOE_HOST_ROUTING", "1")
        monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
        y_host = req.moe(wg, wd, x, routing, idx)
        if req.last_kernel()["name"] == "fcc_prefill_async_grouped_w4":
            assert np.array_equal(y_host.view(np.uint8), y.view(np.uint8)), "host- and device-routed results differ"
        else:
            check(oracle, y_host, ref, max(H, I), f"M={M} host-routed")
            assert M < 300
    finally:
        for w in wg + wd:
            w.close()


def test_moe_routed_index_outside_the_experts(oracle, dev, req):
    """Device indices cannot be checked without waiting for them: a pair whose index names no expert adds nothing
    to its row; every other row is what it is without that pair."""
    E, top_k, H, I, M = 8, 2, 256, 512, 40
    say("moe routed, bad index")
    gu, dn = make_layer(950, E, H, I)
    wg = [fc.CompressedWeights.from_case(dev, c, glu="swish") for c in gu]
    wd = [fc.CompressedWeights.from_case(dev, c) for c in dn]
    idx, routing = routed(951, M, E, top_k)
    x = np.random.default_rng(952).standard_normal((M, H)).astype(np.float16)
    try:
        good = req.moe(wg, wd, x, routing, idx, device_indices=True)
        bad = idx.copy()
        bad[3, 1], bad[17, 0], bad[39, 1] = E, -1, 1 << 20
        got = req.moe(wg, wd, x, routing, bad, device_indices=True)
        zeroed = routing.copy()
        zeroed[3, 1], zeroed[17, 0], zeroed[39, 1] = 0, 0, 0
        want = req.moe(wg, wd, x, zeroed, idx, device_indices=True)
        rows = [3, 17, 39]
        keep = np.setdiff1d(np.arange(M), rows)
        assert np.array_equal(got[keep].view(np.uint16), good[keep].view(np.uint16))
        assert np.array_equal(got[rows].view(np.uint16), want[rows].view(np.uint16))
    finally:
        for w in wg + wd:
            w.close()


def test_moe_routed_refuses_what_only_the_host_route_runs(oracle, dev, req):
    """8-bit experts have no grouped launch with a table in device memory: OVFCC_EUNSUPPORTED, while the
    host-index call runs them."""
    E, H, I = 4, 256, 512
    gu, dn = make_layer(960, E, H, I, wt="u8", zt="u8", G=256)
    wg = [fc.CompressedWeights.from_case(dev, c, glu="swish") for c in gu]
    wd = [fc.CompressedWeights.from_case(dev, c) for c in dn]
    idx, routing = routed(961, 6, E, 2)
    x = np.random.default_rng(962).standard_normal((6, H)).astype(np.float16)
    try:
        with pytest.raises(fc.OvfccError) as err:
            req.moe(wg, wd, x, routing, idx, device_indices=True)
        assert err.value.code == -2            # OVFCC_EUNSUPPORTED
        assert req.moe(wg, wd, x, routing, idx).shape == (6, H)
    finally:
        for w in wg + wd:
            w.close()
