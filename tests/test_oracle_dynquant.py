"""Pins the oracle's per-token int8 activation quantisation and the integer FullyConnected on top of it without
retyping the C code: exact cases, error bounds, an independent numpy restatement and the float oracle applied to the
dequantised activations."""
import numpy as np
import pytest

from openvino_amd import datagen


def np_dynquant(x):
    """Independent restatement in numpy's float16 arithmetic."""
    x = np.asarray(x, dtype=np.float16)
    mx = np.maximum(np.abs(x).max(axis=1), np.float16(0.003)).astype(np.float16)
    scale = (np.float16(127) / mx).astype(np.float16)                      # half division
    q = np.rint((x * scale[:, None]).astype(np.float16).astype(np.float32)).clip(-128, 127).astype(np.int8)
    inv = (np.float32(1) / scale.astype(np.float32)).astype(np.float16).astype(np.float32)
    return q, inv, q.astype(np.int32).sum(axis=1).astype(np.int32)


def test_dynquant_matches_numpy_half_arithmetic(oracle):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((64, 384)) * rng.uniform(0.01, 30, (64, 1))).astype(np.float16)
    x[3] = 0                                  # all-zero row: the clamp at 0.003 decides the scale
    x[4, :] = 1e-4                            # below the clamp
    x[5, 7] = 65504                           # largest half
    q, inv, qs = oracle.dynquant_rows(x)
    q2, inv2, qs2 = np_dynquant(x)
    assert np.array_equal(q, q2) and np.array_equal(inv, inv2) and np.array_equal(qs, qs2)
    assert not q[3].any() and qs[3] == 0


def test_dynquant_exact_rows_and_bounds(oracle):
    """A row whose values are j * 2^e with |j| <= 127 and the maximum 127 * 2^e present quantises to exactly j and
    reconstructs exactly; in general |x - q inv| <= inv / 2 plus the half roundings of scale and product."""
    j = np.array([127, -127, 0, 1, -1, 64, -100, 13] * 16, np.float32)
    for e in (-8, -3, 0, 4):
        x = (j * 2.0 ** e).astype(np.float16)[None, :]
        q, inv, qs = oracle.dynquant_rows(x)
        assert np.array_equal(q[0], j.astype(np.int8)) and inv[0] == 2.0 ** e and qs[0] == int(j.sum())
        assert np.array_equal((q[0] * inv[0]).astype(np.float16), x[0])
    rng = np.random.default_rng(2)
    x = rng.standard_normal((32, 512)).astype(np.float16)
    q, inv, qs = oracle.dynquant_rows(x)
    assert q.max() <= 127 and q.min() >= -127 and np.all(np.abs(q).max(axis=1) >= 126)
    err = np.abs(x.astype(np.float32) - q.astype(np.float32) * inv[:, None])
    assert np.all(err <= inv[:, None] * 0.5 + np.abs(x.astype(np.float32)) * 2.0 ** -9)
    assert np.array_equal(qs, q.astype(np.int64).sum(axis=1))


@pytest.mark.parametrize("wt,zt", [("u8", "u8"), ("u8", "none"), ("i8", "none")])
def test_fc_dynquant_equals_float_oracle_on_dequantised_activations(oracle, wt, zt):
    """(sum q (w - zp)) s inv == FC(q inv): the integer path and the float oracle agree on the same quantised
    activations (up to f32 summation), and differ from the unquantised result by the quantisation noise only."""
    c = datagen.make_case(31, 24, 512, 96, wt, 512, zt, with_bias=True)
    T = {"u8": oracle.U8, "i8": oracle.I8}
    zp = None if c.zp is None else c.zp.astype(np.float32)
    y = oracle.fc_dynquant_reference(c.x, c.w, T[wt], c.scale, zp, c.bias, N=c.N, K=c.K)
    q, inv, _ = oracle.dynquant_rows(c.x)
    xd = q.astype(np.float32) * inv[:, None]
    ref = oracle.fc_reference(xd, c.w, T[wt], c.scale, c.zp, oracle.U8 if zt == "u8" else oracle.NONE, c.bias,
                              N=c.N, K=c.K, group_size=c.K, acc_f64=True)
    assert oracle.rel_l2(y, ref) < 2e-6
    plain = oracle.fc_reference(c.x, c.w, T[wt], c.scale, c.zp, oracle.U8 if zt == "u8" else oracle.NONE, c.bias,
                                N=c.N, K=c.K, group_size=c.K)
    assert 1e-4 < oracle.rel_l2(y, plain) < 3e-2
