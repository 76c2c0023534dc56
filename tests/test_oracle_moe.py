"""Pins oracle.moe_reference (test infrastructure) without the reference's code: the reference holds no numeric
vector for the MOE op (its tests compare the fused op against the unfused graph on random data), so the checks are
an independent float64 evaluation of the unfused graph (numpy dequantisation, torch's silu / gelu), and the
properties the definition fixes: which selection gets which routing weight, which expert serves which row, and
linearity in the routing weights."""
import numpy as np
import pytest
import torch

from openvino_amd import datagen
from parity import T, ZT


def expert_args(c):
    return dict(w=c.w, w_type=T[c.w_type], scale=c.scale, zp=c.zp, zp_type=ZT[c.zp_type], bias=c.bias, N=c.N, K=c.K,
                group_size=c.group_size)


def make_layer(seed, E, H, I, wt="u4", zt="u4", G=32, bias=True):
    # 8-bit weights: scales and zero-points that keep the activations of both projections of order one
    kw = dict(scale_range=(2e-4, 2e-3), zp_range=(100, 156)) if wt == "u8" else {}
    gu = [datagen.make_case(seed + e, 1, H, 2 * I, wt, G, zt, with_bias=bias, **kw) for e in range(E)]
    dn = [datagen.make_case(seed + 100 + e, 1, I, H, wt, G, zt, with_bias=bias, **kw) for e in range(E)]
    return gu, dn


def routed(seed, M, E, top_k):
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((M, E))
    idx = np.argsort(-logits, axis=1, kind="stable")[:, :top_k].astype(np.int32)
    p = np.exp(np.take_along_axis(logits, idx, axis=1))
    return idx, (p / p.sum(axis=1, keepdims=True)).astype(np.float16)


def dense(oracle, c):
    """float64 [N, K] matrix and bias of a case, from the numpy twin of the dequantisation."""
    w = oracle.np_dequantise(c.w, T[c.w_type], c.scale, c.zp, ZT[c.zp_type], N=c.N, K=c.K, group_size=c.group_size)
    return np.asarray(w, np.float64), (np.zeros(c.N) if c.bias is None else c.bias.astype(np.float64))


@pytest.mark.parametrize("glu_type,act", [(1, torch.nn.functional.silu),
                                          (2, lambda t: torch.nn.functional.gelu(t, approximate="none")),
                                          (3, lambda t: torch.nn.functional.gelu(t, approximate="tanh"))])
def test_moe_reference_against_the_unfused_graph_in_float64(oracle, glu_type, act):
    E, H, I, M, top_k = 4, 64, 96, 9, 2
    gu, dn = make_layer(700, E, H, I)
    idx, routing = routed(701, M, E, top_k)
    x = np.random.default_rng(702).standard_normal((M, H)).astype(np.float16)
    got = oracle.moe_reference(x, routing, idx, [expert_args(c) for c in gu], [expert_args(c) for c in dn], glu_type)
    want = np.zeros((M, H))
    for m in range(M):
        for j in range(top_k):
            e = int(idx[m, j])
            wg, bg = dense(oracle, gu[e])
            wd, bd = dense(oracle, dn[e])
            y = wg @ x[m].astype(np.float64) + bg                      # gate rows first, then up rows
            h = act(torch.from_numpy(y[:I])).numpy() * y[I:]
            h = h.astype(np.float16).astype(np.float64)               # an f16 tensor between the projections
            want[m] += float(routing[m, j]) * (wd @ h + bd)
    assert got.shape == (M, H) and got.dtype == np.float32
    # f32 dot products against f64: agreement far inside the f16 rounding of h, which both sides apply -- except
    # where the two evaluations of act(g) u straddle an f16 rounding boundary (a few elements of 9 x 96 x 2)
    err = np.abs(got - want)
    assert np.median(err) < 1e-5 and err.max() < 5e-3 * np.abs(want).max(), (np.median(err), err.max())


def test_moe_reference_properties(oracle):
    E, H, I, M, top_k = 5, 32, 64, 12, 2
    gu, dn = make_layer(710, E, H, I, zt="none", wt="i4", bias=False)
    g, d = [expert_args(c) for c in gu], [expert_args(c) for c in dn]
    idx, routing = routed(711, M, E, top_k)
    x = np.random.default_rng(712).standard_normal((M, H)).astype(np.float16)
    y = oracle.moe_reference(x, routing, idx, g, d, 1)

    # one-hot routing: the row is the named expert's own output
    one = np.zeros_like(routing)
    one[:, 1] = 1
    y1 = oracle.moe_reference(x, one, idx, g, d, 1)
    for m in range(M):
        e = int(idx[m, 1])
        h = oracle.glu(oracle.fc_reference(x[m:m + 1], **g[e]), 1).astype(np.float16)
        assert np.array_equal(y1[m], oracle.fc_reference(h, **d[e])[0])

    # the order of a row's selections does not matter when the weights move with them
    ys = oracle.moe_reference(x, routing[:, ::-1], idx[:, ::-1], g, d, 1)
    assert np.allclose(ys, y, rtol=0, atol=1e-6 * np.abs(y).max())

    # linear in the routing weights (powers of two: exact)
    assert np.array_equal(oracle.moe_reference(x, routing * np.float16(2), idx, g, d, 1), 2 * y)

    # an expert that no row selects has no influence
    unused = [e for e in range(E) if not np.any(idx == e)]
    idx2 = idx.copy()
    if not unused:
        idx2[idx2 == E - 1] = 0          # free the last expert (a row may now name expert 0 twice: allowed)
        unused = [E - 1]
    base = oracle.moe_reference(x, routing, idx2, g, d, 1)
    g2, d2 = list(g), list(d)
    g2[unused[0]], d2[unused[0]] = g[(unused[0] + 1) % E], d[(unused[0] + 1) % E]
    assert np.array_equal(oracle.moe_reference(x, routing, idx2, g2, d2, 1), base)

    # no rows
    assert oracle.moe_reference(x[:0], routing[:0], idx[:0], g, d, 1).shape == (0, H)
