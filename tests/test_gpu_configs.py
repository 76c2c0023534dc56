"""GPU parity at the five benchmark configurations (real shapes).

Small-M cases are checked in full against the oracle.  Large-M cases are checked on a seeded sample of
rows against the oracle (all output channels), and over the full output through properties that do not
need the oracle: duplicated activation rows give duplicated output rows, and doubling the activations
doubles every output bit-exactly (a power-of-two scale commutes with every rounding on the path).
"""
import sys

import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc
from parity import REL_L2_MAX, T, ZT, check_parity, max_abs_limit, oracle_y

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


def sampled_check(oracle, req, w, c, rows, what, output_rounding_slack=False):
    """GPU on all rows; oracle on `rows` sampled rows, every output channel."""
    y = req.infer(w, c.x)
    info = req.last_kernel()
    rng = np.random.default_rng(99)
    pick = np.sort(rng.choice(c.M, size=min(rows, c.M), replace=False))
    ref = oracle_y(oracle, c, x=c.x[pick])
    r = check_parity(oracle, y[pick], ref, c.K, f"{what} {info}", output_rounding_slack=output_rounding_slack)
    say(f"   {what}: {info['name']} grid={info['grid']} split={info['split_k']} out={y.dtype} "
        f"rel-L2={r[0]:.2e} max-abs={r[1]:.2e}")
    return y


def test_config1_u4_asym(oracle, dev, req):
    say("config 1")
    c = datagen.config1()
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        assert w.tiled
        y = req.infer(w, c.x)
        assert req.last_kernel()["kernel"] == _lib.KERNEL_DECODE
        r = check_parity(oracle, y, oracle_y(oracle, c), c.K, "config1")
        say(f"   config1 rel-L2={r[0]:.2e} max-abs={r[1]:.2e} {req.last_kernel()}")
    finally:
        w.close()


@pytest.mark.parametrize("shape", list(datagen.LLAMA3_8B_SHAPES))
def test_config2_decode(oracle, dev, req, shape):
    say(f"config 2 {shape}")
    c = datagen.config2(shape, 32)
    w = fc.CompressedWeights.from_case(dev, c)
    ref = oracle_y(oracle, c)
    try:
        for M in (1, 4, 16, 32):
            y = req.infer(w, c.x[:M])
            info = req.last_kernel()
            assert info["kernel"] == _lib.KERNEL_DECODE
            r = check_parity(oracle, y, ref[:M], c.K, f"config2 {shape} M={M}")
            say(f"   M={M}: split={info['split_k']} rel-L2={r[0]:.2e} max-abs={r[1]:.2e}")
    finally:
        w.close()


@pytest.mark.parametrize("shape", list(datagen.LLAMA3_8B_SHAPES))
def test_config3_prefill(oracle, dev, req, shape):
    say(f"config 3 {shape}")
    c = datagen.config3(shape, 8192)
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        for M in (512, 2048, 8192):
            sub = datagen.FcCase(M, c.K, c.N, c.group_size, c.w_type, c.zp_type, c.w, c.scale, c.zp, c.x[:M])
            y = sampled_check(oracle, req, w, sub, 24, f"config3 {shape} M={M}")
            assert req.last_kernel()["kernel"] == _lib.KERNEL_PREFILL
            if M == 2048:
                # full-output properties
                y2 = req.infer(w, (sub.x * np.float16(2)))
                normal = np.abs(y.astype(np.float32)) >= 2.0 ** -13   # doubling a subnormal half rounds differently
                want = (y.astype(np.float32) * 2).astype(np.float16)
                bad = int(np.count_nonzero((want.view(np.uint16) != y2.view(np.uint16)) & normal))
                assert bad == 0, f"doubling the activations must double every output ({bad} differ)"
                assert np.all(np.abs(y2[~normal].astype(np.float32)) <= 2.0 ** -11)
                xdup = np.repeat(sub.x[:1], M, axis=0)
                yd = req.infer(w, xdup)
                assert np.all(yd.view(np.uint16) == yd[:1].view(np.uint16)), "equal rows must give equal outputs"
    finally:
        w.close()


@pytest.mark.parametrize("shape", list(datagen.LLAMA3_70B_SHAPES))
def test_config4_u8_per_channel(oracle, dev, req, shape):
    """Outputs of this distribution reach |y| > 128, where half a float16 ulp (0.0625) alone exceeds the max-abs
    bound, so the bound proper is checked on the f32 output_type (the kernel's arithmetic before the output
    cast); the f16 output must be exactly the rounding of that f32 output and meets the bound plus the cast's
    own half ulp."""
    say(f"config 4 {shape}")
    c = datagen.config4(shape, 1024)
    w16 = fc.CompressedWeights.from_case(dev, c)
    w32 = fc.CompressedWeights.from_case(dev, c, output_type="f32")
    try:
        for M, rows in ((1, 1), (32, 32), (1024, 12)):
            sub = datagen.FcCase(M, c.K, c.N, c.group_size, c.w_type, c.zp_type, c.w, c.scale, c.zp, c.x[:M])
            y32 = sampled_check(oracle, req, w32, sub, rows, f"config4 {shape} M={M}")
            assert y32.dtype == np.float32
            y16 = sampled_check(oracle, req, w16, sub, rows, f"config4 {shape} M={M}", output_rounding_slack=True)
            assert np.array_equal(y32.astype(np.float16).view(np.uint16), y16.view(np.uint16))
    finally:
        w16.close()
        w32.close()


def test_config5_moe_experts(oracle, dev, req):
    say("config 5")
    routes = datagen.moe_routing()
    assert sum(len(r) for r in routes) == 512
    rng = np.random.default_rng(7)
    for e, tokens in enumerate(routes):
        M = len(tokens)
        for which in ("gate", "up", "down"):
            c = datagen.config5_expert(e, which, M)
            w = fc.CompressedWeights.from_case(dev, c)
            try:
                y = req.infer(w, c.x)
                info = req.last_kernel()
                cols = np.sort(rng.choice(c.N, size=192, replace=False))
                ref = oracle_y(oracle, c, n_index=cols)
                r = check_parity(oracle, y[:, cols], ref, c.K, f"config5 expert {e} {which} M={M}")
                say(f"   expert {e} {which} M={M}: {info['name']} rel-L2={r[0]:.2e} max-abs={r[1]:.2e}")
            finally:
                w.close()


def test_config5_moe_block_real_shape(oracle, dev, req):
    """Config 5 as one call at its real shape: 8 experts 4096 -> 14336 -> 4096 (u4 asymmetric, groups of 128, SwiGLU
    fused into the gate / up node), 256 tokens, top-2 routing from datagen.moe_routing().  Sixteen sampled tokens are
    compared with oracle.moe_reference; the device-routed entry point (indices in device memory) must give the same
    bits as the host-routed one."""
    say("config 5 block")
    routes = datagen.moe_routing()
    tokens = 256
    indices = np.full((tokens, 2), -1, np.int32)
    for e, rows in enumerate(routes):
        for t in rows:
            indices[t, 0 if indices[t, 0] < 0 else 1] = e
    assert (indices >= 0).all()
    gu_cases, dn_cases, wg, wd = [], [], [], []
    try:
        for e in range(len(routes)):
            g, u = datagen.config5_expert(e, "gate", 1), datagen.config5_expert(e, "up", 1)
            gu_cases.append(datagen.FcCase(1, g.K, 2 * g.N, 128, "u4", "u4", np.concatenate([g.w, u.w]),
                                           np.concatenate([g.scale, u.scale]), np.concatenate([g.zp, u.zp]), g.x))
            dn_cases.append(datagen.config5_expert(e, "down", 1))
            wg.append(fc.CompressedWeights.from_case(dev, gu_cases[-1], glu="swish"))
            wd.append(fc.CompressedWeights.from_case(dev, dn_cases[-1]))
        rng = np.random.default_rng(55)
        x = rng.standard_normal((tokens, 4096)).astype(np.float16)
        rw = rng.uniform(0.2, 0.8, size=(tokens, 1))
        routing = np.concatenate([rw, 1.0 - rw], axis=1).astype(np.float16)
        say("   host-routed call")
        y_host = req.moe(wg, wd, x, routing, indices)
        info = req.last_kernel()
        say(f"   device-routed call ({info['name']})")
        y_dev = req.moe(wg, wd, x, routing, indices, device_indices=True)
        assert y_host.shape == (tokens, 4096) and y_host.dtype == np.float16
        assert np.array_equal(y_host.view(np.uint16), y_dev.view(np.uint16)), "host- and device-routed results differ"
        pick = np.sort(np.random.default_rng(56).choice(tokens, size=16, replace=False))

        def eargs(c):
            return dict(w=c.w, w_type=T[c.w_type], scale=c.scale, zp=c.zp, zp_type=ZT[c.zp_type], bias=None,
                        N=c.N, K=c.K, group_size=c.group_size)
        ref = oracle.moe_reference(x[pick], routing[pick], indices[pick], [eargs(c) for c in gu_cases],
                                   [eargs(c) for c in dn_cases], 1)
        y = y_host[pick].astype(np.float32)
        rl2, mab = oracle.rel_l2(y, ref), oracle.max_abs(y, ref)
        # two projections in a row: the down projection's bound counts twice (its own arithmetic and the error its
        # input carries), plus half an f16 ulp of the largest output
        limit = 2 * max_abs_limit(14336) + float(np.max(np.abs(ref))) * 2.0 ** -11
        say(f"   16 sampled tokens: rel-L2={rl2:.2e} max-abs={mab:.2e} (limit {limit:.2e})")
        assert rl2 <= 2 * REL_L2_MAX and mab <= limit
        assert np.all(np.isfinite(y_host.astype(np.float32)))
    finally:
        for w in wg + wd:
            w.close()
