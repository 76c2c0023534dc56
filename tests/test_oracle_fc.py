"""Pins oracle.ovo_fc_reference.

1. exact golden vectors of the reference's GPU unit tests (tests/golden/fc_golden.json);
2. an independent numpy float64 restatement on random cases of every supported type;
3. algebraic invariants chosen so that a dropped term, a wrong group index, a swapped
   nibble or a transposed operand fails at least one of them.
"""
import numpy as np
import pytest

from golden_cases import fc_cases
from openvino_amd import datagen

GOLD = fc_cases()
T = {"u4": 1, "i4": 2, "u8": 3, "i8": 4}
ZT = {"none": 0, "u4": 1, "u8": 3}


def run_oracle(o, c: datagen.FcCase, x=None, **kw):
    return o.fc_reference(c.x if x is None else x, c.w, T[c.w_type], c.scale, c.zp, ZT[c.zp_type], c.bias,
                          N=c.N, K=c.K, group_size=c.group_size, zp_scalar=c.zp_scalar, **kw)


def run_numpy(o, c: datagen.FcCase, x=None):
    return o.fc_reference_numpy(c.x if x is None else x, c.w, T[c.w_type], c.scale, c.zp, ZT[c.zp_type], c.bias,
                                N=c.N, K=c.K, group_size=c.group_size, zp_scalar=c.zp_scalar)


@pytest.mark.parametrize("g", GOLD, ids=[g["id"] for g in GOLD])
@pytest.mark.parametrize("half_inputs", [False, True], ids=["f32in", "f16in"])
def test_golden_vectors_exact(oracle, g, half_inputs):
    """Every golden value is exactly representable, so float and double accumulation, float32 and
    float16 inputs must all reproduce it bit for bit."""
    x = g["x"].astype(np.float16) if half_inputs else g["x"]
    scale = g["scale"].astype(np.float16) if half_inputs else g["scale"]
    bias = None if g["bias"] is None else (g["bias"].astype(np.float16) if half_inputs else g["bias"])
    zp_type = oracle.NONE if g["zp"] is None else oracle.U8
    for acc64 in (False, True):
        y = oracle.fc_reference(x, g["w"], T[g["w_type"]], scale, g["zp"], zp_type, bias, N=g["N"], K=g["K"],
                                group_size=g["group_size"], zp_scalar=g["zp_scalar"], acc_f64=acc64)
        assert y.shape == g["expected"].shape
        assert np.array_equal(y, g["expected"]), g["source"]
    yn = oracle.fc_reference_numpy(x, g["w"], T[g["w_type"]], scale, g["zp"], zp_type, bias, N=g["N"], K=g["K"],
                                   group_size=g["group_size"], zp_scalar=g["zp_scalar"])
    assert np.array_equal(yn, g["expected"].astype(np.float64))
    # float zero-points (the reference tests G1/G2 hold them as f32) give the same answer
    if g["zp"] is not None:
        y = oracle.fc_reference(x, g["w"], T[g["w_type"]], scale, g["zp"].astype(np.float32), oracle.F32, bias,
                                N=g["N"], K=g["K"], group_size=g["group_size"], zp_scalar=g["zp_scalar"])
        assert np.array_equal(y, g["expected"])


CASES = [
    ("u4", "u4", 128, 256, 48, 5), ("u4", "none", 64, 256, 33, 3), ("i4", "none", 128, 384, 40, 4),
    ("i4", "u4", 32, 96, 17, 2), ("u8", "u8", 256, 256, 24, 7), ("u8", "none", 16, 64, 9, 1),
    ("u4", "u8", 128, 128, 16, 1),
]


@pytest.mark.parametrize("wt,zt,G,K,N,M", CASES)
def test_matches_numpy_restatement(oracle, wt, zt, G, K, N, M):
    c = datagen.make_case(42, M, K, N, wt, G, zt, with_bias=True)
    ref64 = run_numpy(oracle, c)
    y64 = run_oracle(oracle, c, acc_f64=True)
    y32 = run_oracle(oracle, c, acc_f64=False)
    assert oracle.rel_l2(y64, ref64) < 2e-7
    assert oracle.rel_l2(y32, ref64) < 2e-6
    assert np.max(np.abs(y64 - ref64)) < 1e-5


def test_n_index_subset(oracle):
    c = datagen.make_case(9, 3, 256, 64, "u4", 128, "u4")
    full = run_oracle(oracle, c)
    idx = np.array([63, 0, 17, 17, 5])
    sub = run_oracle(oracle, c, n_index=idx)
    assert np.array_equal(sub, full[:, idx])


def test_invariants(oracle):
    c = datagen.make_case(77, 4, 512, 32, "u4", 128, "u4")
    base = run_oracle(oracle, c, acc_f64=True)

    # (a) zero-point equal to every weight of its group -> exactly zero
    q = np.repeat(np.arange(32 * 4, dtype=np.uint8) % 16, 128)           # [N*ng] values spread over groups
    z = datagen.pack_nibbles(np.arange(32 * 4) % 16)
    cz = datagen.FcCase(4, 512, 32, 128, "u4", "u4", datagen.pack_nibbles(q), c.scale, z, c.x)
    assert np.all(run_oracle(oracle, cz) == 0)

    # (b) doubling every scale doubles the result exactly (power of two)
    c2 = datagen.FcCase(4, 512, 32, 128, "u4", "u4", c.w, (c.scale * np.float16(2)), c.zp, c.x)
    assert np.array_equal(run_oracle(oracle, c2, acc_f64=True), 2 * base)

    # (c) unit-vector probe returns the dequantised column: catches transposed or mis-grouped indexing
    deq = oracle.np_dequantise(c.w, 1, c.scale, c.zp, 1, N=32, K=512, group_size=128)
    for k in (0, 1, 127, 128, 300, 511):
        e = np.zeros((1, 512), np.float16)
        e[0, k] = 1
        assert np.array_equal(run_oracle(oracle, c, x=e)[0].astype(np.float64), deq[:, k].astype(np.float32))

    # (d) i4 weights equal u4 weights xor 8 with zero-point 8
    ci = datagen.make_case(5, 3, 256, 16, "i4", 128, "none")
    cu = datagen.FcCase(3, 256, 16, 128, "u4", "u8", ci.w ^ 0x88, ci.scale, np.full(16 * 2, 8, np.uint8), ci.x)
    assert np.array_equal(run_oracle(oracle, ci), run_oracle(oracle, cu))

    # (e) one group spanning K equals per-channel parameters replicated per group
    cp = datagen.make_case(6, 2, 256, 8, "u8", 256, "u8")
    cg = datagen.FcCase(2, 256, 8, 128, "u8", "u8", cp.w, np.repeat(cp.scale, 2, axis=1), np.repeat(cp.zp, 2), cp.x)
    assert np.array_equal(run_oracle(oracle, cp), run_oracle(oracle, cg))

    # (f) permuting output channels permutes the result
    perm = np.random.default_rng(1).permutation(32)
    wq = oracle.unpack_u4(c.w, 32 * 512).reshape(32, 512)[perm]
    zq = oracle.unpack_u4(c.zp, 32 * 4).reshape(32, 4)[perm]
    cperm = datagen.FcCase(4, 512, 32, 128, "u4", "u4", datagen.pack_nibbles(wq), c.scale[perm],
                           datagen.pack_nibbles(zq), c.x)
    assert np.array_equal(run_oracle(oracle, cperm, acc_f64=True), base[:, perm])

    # (g) bias is added once, after the sum
    b = np.arange(32, dtype=np.float16)
    cb = datagen.FcCase(4, 512, 32, 128, "u4", "u4", c.w, c.scale, c.zp, c.x, bias=b)
    assert np.allclose(run_oracle(oracle, cb, acc_f64=True), base + b.astype(np.float32), rtol=0, atol=1e-5)


def test_rejects_bad_arguments(oracle):
    c = datagen.make_case(1, 1, 256, 8, "u4", 128, "u4")
    with pytest.raises(ValueError):
        oracle.fc_reference(c.x, c.w, 1, c.scale, c.zp, 1, N=8, K=256, group_size=100)
    with pytest.raises(ValueError):
        oracle.fc_reference(c.x, c.w, 9, c.scale, c.zp, 1, N=8, K=256, group_size=128)


def test_datagen_packing_matches_oracle(oracle):
    rng = np.random.default_rng(0)
    u = rng.integers(0, 16, 1001, dtype=np.uint8)
    assert np.array_equal(datagen.pack_nibbles(u), oracle.pack_u4(u))
    i = rng.integers(-8, 8, 1000).astype(np.int8)
    assert np.array_equal(datagen.pack_nibbles(i), oracle.pack_i4(i))


def test_datagen_is_seeded_and_in_range(oracle):
    a = datagen.config1()
    b = datagen.config1()
    assert np.array_equal(a.w, b.w) and np.array_equal(a.scale, b.scale) and np.array_equal(a.x, b.x)
    assert a.algorithmic_bytes() == 8_732_672
    s = a.scale.astype(np.float32)
    assert s.min() >= 0.002 - 1e-5 and s.max() <= 0.02 + 1e-5
    c4 = datagen.make_case(3, 1, 512, 64, "u8", 512, "u8", scale_range=(1e-3, 1e-2), zp_range=(100, 157))
    assert c4.zp.min() >= 100 and c4.zp.max() <= 156
    routes = datagen.moe_routing()
    assert sum(len(r) for r in routes) == 512 and len(routes) == 8
    assert len({len(r) for r in routes}) > 1          # uneven per-expert token counts
