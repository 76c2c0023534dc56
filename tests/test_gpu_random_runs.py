"""Seeded random shapes through the C ABI against the numpy restatement of the oracle's formula (itself pinned against
the C oracle in the CPU tests): single nodes of every weight type and row count the planner distinguishes, grouped
runs at every slice height, and the device-routed expert block with skewed routings, idle experts and indices that
name no expert.  Complements the fixed cases of the other GPU tests with shapes nobody chose."""
import numpy as np
import pytest

from openvino_amd import datagen, fc
from parity import REL_L2_MAX

pytestmark = pytest.mark.gpu

TAG = {"u4": "U4", "i4": "I4", "u8": "U8", "i8": "I8", "none": "NONE"}


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


def reference(oracle, c, x):
    return oracle.fc_reference_numpy(x, c.w, getattr(oracle, TAG[c.w_type]), c.scale, c.zp, getattr(oracle, TAG[c.zp_type]),
                                     c.bias, N=c.N, K=c.K, group_size=c.group_size)


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_single_nodes(oracle, dev, req, seed):
    rng = np.random.default_rng(seed)
    seen = set()
    for n in range(60):
        wt = str(rng.choice(["u4", "i4", "u8", "i8"]))
        zt = "none" if wt in ("i4", "i8") else str(rng.choice(["none", "u4", "u8"] if wt == "u4" else ["none", "u8"]))
        K = int(rng.choice([128, 256, 384, 512, 1024, 2048, 4096]))
        N = int(rng.choice([16, 48, 64, 128, 256, 512, 1024, 2048]))
        G = int(rng.choice([g for g in (32, 64, 128, 256, K) if K % g == 0 and (g >= 128 or wt in ("u4", "i4"))]))
        M = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 48, 49, 64, 65, 80, 100, 128, 129, 200, 300, 513]))
        out = str(rng.choice(["f16", "f32"]))
        c = datagen.make_case(int(rng.integers(1 << 30)), M, K, N, wt, G, zt, with_bias=bool(rng.integers(2)))
        say(f"random node {seed}/{n}: {wt}/{zt} G={G} K={K} N={N} M={M} out={out}")
        w = fc.CompressedWeights.from_case(dev, c, output_type=out)
        try:
            y = req.infer(w, c.x).astype(np.float64)
            info = req.last_kernel()
            seen.add(info["name"])
            rl2 = oracle.rel_l2(y, reference(oracle, c, c.x))
            assert np.all(np.isfinite(y)) and rl2 <= REL_L2_MAX, f"{info}: rel-L2 {rl2:.3e}"
        finally:
            w.close()
    assert len(seen) >= 5, seen   # the draw reaches several kernel families


@pytest.mark.parametrize("seed", [201, 202])
def test_random_grouped_runs(oracle, dev, req, monkeypatch, seed):
    monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
    rng = np.random.default_rng(seed)
    for n in range(25):
        wt, zt, G = [("u4", "u4", 128), ("u4", "u8", 128), ("i4", "none", 128), ("u4", "none", 0), ("u4", "u4", 256)][rng.integers(5)]
        K = int(rng.choice([256, 512, 1024, 2048]))
        N = int(rng.choice([256, 512, 1024]))
        G = G or K
        rows = [int(rng.integers(49, 200)) if rng.random() < 0.8 else int(rng.integers(0, 49)) for _ in range(int(rng.integers(1, 9)))]
        rows[0] = max(rows[0], 49)
        height = int(rng.choice([0, 64, 80, 96, 128]))
        if height:
            monkeypatch.setenv("OVFCC_PREFILL_ROWS", str(height))
        else:
            monkeypatch.delenv("OVFCC_PREFILL_ROWS", raising=False)
        cases = [datagen.make_case(int(rng.integers(1 << 30)), max(rows), K, N, wt, G, zt, with_bias=bool(rng.integers(2)))
                 for _ in range(min(len(rows), 3))]
        say(f"random grouped {seed}/{n}: {wt}/{zt} G={G} K={K} N={N} rows={rows} height={height}")
        ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
        try:
            ys = req.infer_grouped([(ws[i % len(ws)], cases[i % len(ws)].x[:m]) for i, m in enumerate(rows)])
            info = req.last_kernel()   # (a grouped kernel, or the last item's own where the run went item by item)
            for i, (m, y) in enumerate(zip(rows, ys)):
                assert y.shape == (m, N)
                if m:
                    c = cases[i % len(ws)]
                    rl2 = oracle.rel_l2(y.astype(np.float64), reference(oracle, c, c.x[:m]))
                    assert rl2 <= REL_L2_MAX, f"item {i} M={m} {info}: rel-L2 {rl2:.3e}"
        finally:
            for w in ws:
                w.close()


def test_random_routed_expert_blocks(oracle, dev, req):
    rng = np.random.default_rng(301)
    H, I, E = 512, 1024, 8
    gu = [datagen.make_case(9000 + e, 1, H, 2 * I, "u4", 128, "u4") for e in range(E)]
    dn = [datagen.make_case(9100 + e, 1, I, H, "u4", 128, "u4") for e in range(E)]
    wg = [fc.CompressedWeights.from_case(dev, c, glu="swish") for c in gu]
    wd = [fc.CompressedWeights.from_case(dev, c) for c in dn]

    def eargs(c):
        return dict(w=c.w, w_type=oracle.U4, scale=c.scale, zp=c.zp, zp_type=oracle.U4, bias=None, N=c.N, K=c.K,
                    group_size=c.group_size)
    try:
        for n in range(20):
            M = int(rng.choice([40, 100, 256, 300, 512, 700, 1000]))
            top_k = int(rng.choice([1, 2, 4]))
            p = rng.dirichlet(np.full(E, float(rng.choice([0.3, 1.0, 5.0]))))
            idx = np.stack([rng.choice(E, size=top_k, replace=False, p=p) for _ in range(M)]).astype(np.int32)
            if n % 3 == 0:
                idx[rng.integers(M), 0] = -1 if n % 2 else E + 3   # names no expert: selects nothing
            x = (rng.standard_normal((M, H)) * 0.5).astype(np.float16)
            r = rng.uniform(0.1, 0.9, size=(M, top_k)).astype(np.float16)
            valid = (idx >= 0) & (idx < E)
            say(f"random expert block {n}: M={M} top_k={top_k} rows per expert {np.bincount(idx[valid], minlength=E).tolist()}")
            y = req.moe(wg, wd, x, r, idx, device_indices=True).astype(np.float32)
            pick = rng.choice(M, size=min(M, 16), replace=False)
            ref = oracle.moe_reference(x[pick], np.where(valid, r, 0).astype(np.float16)[pick], np.where(valid, idx, 0)[pick],
                                       [eargs(c) for c in gu], [eargs(c) for c in dn], 1)
            rl2 = oracle.rel_l2(y[pick], ref)
            assert np.all(np.isfinite(y)) and rl2 <= 2 * REL_L2_MAX, f"{req.last_kernel()}: rel-L2 {rl2:.3e}"
            if valid.all():
                assert np.array_equal(req.moe(wg, wd, x, r, idx, device_indices=False).astype(np.float32), y)
    finally:
        for w in wg + wd:
            w.close()
