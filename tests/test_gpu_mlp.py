"""GPU parity of the MLP node (gate / up projection with its gated linear unit, then the down projection, as one
object: the CPU plugin's LLMMLP, src/plugins/intel_cpu/src/nodes/llm_mlp.cpp:495-526) against the oracle's chain
glu(fc(x; gate_up)) -> f16 -> fc(.; down), and of its optional one-launch kernel (OVFCC_MLP_FUSED=1) against the two
launches the node runs as otherwise, bit for bit.  The unfused graph the reference's fusion pass matches is
src/plugins/intel_cpu/src/transformations/cpu_opset/x64/pass/mlp_fusion.cpp:48-120."""
import sys

import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc
from parity import REL_L2_MAX, max_abs_limit, oracle_y

pytestmark = pytest.mark.gpu

GLU = {"swish": 1, "gelu": 2, "gelu_tanh": 3}


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


def make_pair(seed, M, H, I, N2, wt, zt, bias):
    """gate / up case [2 I, H] (gate rows first) and down case [N2, I]."""
    cg = datagen.make_case(seed, M, H, 2 * I, wt, 128, zt, with_bias=bias)
    cd = datagen.make_case(seed + 1, 1, I, N2, wt, 128, zt, with_bias=bias)
    return cg, cd


def mlp_reference(o, cg, cd, kind, x):
    """The oracle's chain with the intermediate activations rounded to f16, as between two nodes."""
    h = o.glu(oracle_y(o, cg, x=x), GLU[kind], False).astype(np.float16)
    return oracle_y(o, cd, x=h), h.astype(np.float32)


def check_chain(o, y, ref, h, K2, what):
    y = np.asarray(y, np.float32)
    assert y.shape == ref.shape and np.all(np.isfinite(y)), what
    rl2, mab = o.rel_l2(y, ref), o.max_abs(y, ref)
    # the max-abs bound is stated for unit-variance activations; the intermediate row has its own scale
    limit = max_abs_limit(K2) * max(1.0, float(np.sqrt(np.mean(h * h)))) * 2.0 + float(np.max(np.abs(ref))) * 2.0 ** -11
    assert rl2 <= REL_L2_MAX, f"{what}: rel-L2 {rl2:.3e}"
    assert mab <= limit, f"{what}: max-abs {mab:.3e} > {limit:.3e}"


def build(dev, cg, cd, kind, out="f16"):
    wg = fc.CompressedWeights.from_case(dev, cg, glu=kind)
    wd = fc.CompressedWeights.from_case(dev, cd, output_type=out)
    node = fc.CompressedWeights.mlp(wg, wd)
    return wg, wd, node


SHAPES = [
    # H, I, N2, w_type, zp_type, bias, unit, output type
    (1024, 2048, 1024, "i4", "none", False, "swish", "f16"),   # one wave per tile: eight pair slots per workgroup
    (2048, 1024, 512, "u4", "u4", True, "swish", "f32"),       # zero-point tables on both nodes, fewer tiles than workgroups
    (4096, 3072, 256, "u4", "none", True, "gelu_tanh", "f16"),  # constant zero-point 0 with u4, 4 waves per tile, 3 down waves
    (8192, 1024, 4096, "i4", "none", False, "gelu", "f16"),    # eight waves per tile: one pair at a time
]


@pytest.mark.parametrize("H,I,N2,wt,zt,bias,kind,out", SHAPES)
def test_mlp_one_launch_against_oracle_and_two_launches(oracle, dev, req, monkeypatch, H, I, N2, wt, zt, bias, kind, out):
    monkeypatch.setenv("OVFCC_GEMV_C", "8")   # both nodes laid out for eight k-blocks per wave, whatever their size
    cg, cd = make_pair(8100 + H // 128 + I // 64, 4, H, I, N2, wt, zt, bias)
    wg, wd, node = build(dev, cg, cd, kind, out)
    try:
        for M in (1, 2, 3, 4):
            say(f"mlp {wt}/{zt} H={H} I={I} N2={N2} {kind} out={out} M={M}")
            x = cg.x[:M]
            ref, h = mlp_reference(oracle, cg, cd, kind, x)
            monkeypatch.setenv("OVFCC_MLP_FUSED", "1")
            y = req.infer(node, x)
            info = req.last_kernel()
            assert info["name"] == "fcc_mlp_gemv_w4" and info["block"] == 1024, info
            assert y.shape == (M, N2) and y.dtype == (np.float32 if out == "f32" else np.float16)
            check_chain(oracle, y, ref, h, I, f"one launch M={M} {info}")
            for _ in range(3):   # the counters return to zero; the sums do not depend on arrival order
                assert np.array_equal(req.infer(node, x).view(np.uint8), y.view(np.uint8))
            monkeypatch.setenv("OVFCC_MLP_FUSED", "0")
            y2 = req.infer(node, x)
            assert req.last_kernel()["name"] == "fcc_gemv_w4", req.last_kernel()
            assert np.array_equal(y2.view(np.uint8), y.view(np.uint8)), "one launch and two launches differ"
            # ... and the two separate nodes a host without the MLP node would run
            hh = req.infer(wg, x)
            y3 = req.infer(wd, hh)
            assert np.array_equal(y3.view(np.uint8), y.view(np.uint8))
    finally:
        for w in (wg, wd, node):
            w.close()


def test_mlp_llama3_8b_shape(oracle, dev, req, monkeypatch):
    """The benchmark's block: 4096 -> 14336 (gate, up; SwiGLU) -> 4096, i4 g128 symmetric, at the layout the planner
    gives the nodes by itself, through the one-launch kernel."""
    monkeypatch.setenv("OVFCC_MLP_FUSED", "1")
    H, I = 4096, 14336
    cg, cd = make_pair(8200, 4, H, I, H, "i4", "none", False)
    wg, wd, node = build(dev, cg, cd, "swish")
    try:
        for M in (1, 4):
            say(f"mlp llama-3-8b M={M}")
            x = cg.x[:M]
            y = req.infer(node, x)
            info = req.last_kernel()
            assert info["name"] == "fcc_mlp_gemv_w4", info
            ref, h = mlp_reference(oracle, cg, cd, "swish", x)
            check_chain(oracle, y, ref, h, I, f"M={M} {info}")
            y2 = req.infer(wd, req.infer(wg, x))
            assert np.array_equal(y2.view(np.uint8), y.view(np.uint8))
    finally:
        for w in (wg, wd, node):
            w.close()


@pytest.mark.parametrize("M", [5, 16, 64, 300])
def test_mlp_more_rows_run_as_two_launches(oracle, dev, req, M):
    H, I, N2 = 1024, 1024, 512
    cg, cd = make_pair(8300, M, H, I, N2, "u4", "u4", True)
    wg, wd, node = build(dev, cg, cd, "swish")
    try:
        say(f"mlp two launches M={M}")
        y = req.infer(node, cg.x)
        assert req.last_kernel()["name"] != "fcc_mlp_gemv_w4"
        ref, h = mlp_reference(oracle, cg, cd, "swish", cg.x)
        check_chain(oracle, y, ref, h, I, f"M={M}")
        assert np.array_equal(req.infer(wd, req.infer(wg, cg.x)).view(np.uint8), y.view(np.uint8))
    finally:
        for w in (wg, wd, node):
            w.close()


@pytest.mark.parametrize("fused", ["0", "1"])
def test_mlp_clone_and_device_buffers(oracle, dev, req, monkeypatch, fused):
    monkeypatch.setenv("OVFCC_MLP_FUSED", fused)
    monkeypatch.setenv("OVFCC_GEMV_C", "8")
    H, I, N2 = 1024, 2048, 1024
    cg, cd = make_pair(8400, 2, H, I, N2, "i4", "none", False)
    wg, wd, node = build(dev, cg, cd, "swish")
    twin = node.clone()
    try:
        assert node.device_bytes == wg.device_bytes + wd.device_bytes == twin.device_bytes
        y = req.infer(node, cg.x)
        x_dev, y_dev = dev.malloc(cg.x.nbytes), dev.malloc(2 * N2 * 2)
        dev.upload(x_dev, cg.x)
        req.infer_device(twin, x_dev, y_dev, 2)
        req.sync()
        assert np.array_equal(dev.download(y_dev, (2, N2), np.float16).view(np.uint8), y.view(np.uint8))
        dev.free(x_dev)
        dev.free(y_dev)
    finally:
        for w in (wg, wd, node, twin):
            w.close()


def test_mlp_wait_that_runs_out_is_reported(oracle, dev, req, monkeypatch):
    """The wait in the middle of the one-launch kernel is bounded.  With a limit of one poll most workgroups give up
    at once: the kernel still finishes, the call reports OVFCC_EDEVICE, and the next call works again."""
    monkeypatch.setenv("OVFCC_MLP_FUSED", "1")
    H, I = 4096, 14336
    cg, cd = make_pair(8500, 1, H, I, H, "i4", "none", False)
    wg, wd, node = build(dev, cg, cd, "swish")
    try:
        good = req.infer(node, cg.x)
        assert req.last_kernel()["name"] == "fcc_mlp_gemv_w4"
        monkeypatch.setenv("OVFCC_MLP_SPIN_LIMIT", "1")
        with pytest.raises(fc.OvfccError) as err:
            req.infer(node, cg.x)
        assert err.value.code == _lib.EDEVICE
        monkeypatch.delenv("OVFCC_MLP_SPIN_LIMIT")
        assert np.array_equal(req.infer(node, cg.x).view(np.uint8), good.view(np.uint8))
    finally:
        for w in (wg, wd, node):
            w.close()


def test_mlp_arguments():
    """Shape and kind checks of ovfcc_weights_mlp need a device for the nodes only."""
    d = fc.Device(0)
    try:
        cg, cd = make_pair(8600, 1, 256, 256, 128, "u4", "u4", False)
        plain = fc.CompressedWeights.from_case(d, cg)            # no gated linear unit
        wg = fc.CompressedWeights.from_case(d, cg, glu="swish")
        wd = fc.CompressedWeights.from_case(d, cd)
        wrong = fc.CompressedWeights.from_case(d, datagen.make_case(8601, 1, 384, 128, "u4", 128, "u4"))
        for a, b in ((plain, wd), (wg, wrong), (wg, wg)):
            with pytest.raises(fc.OvfccError) as err:
                fc.CompressedWeights.mlp(a, b)
            assert err.value.code == _lib.EINVAL
        node = fc.CompressedWeights.mlp(wg, wd)
        with pytest.raises(fc.OvfccError):
            fc.CompressedWeights.mlp(node, wd)
        for w in (plain, wg, wd, wrong, node):
            w.close()
    finally:
        d.close()
