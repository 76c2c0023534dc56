"""The shape matrix of the reference's own functional tests for this path
(src/plugins/intel_cpu/tests/functional/custom/subgraph_tests/src/x64/matmul_weights_decompression.cpp:37-66:
input_shapes_basic and input_shapes_amx) run through the C ABI against the oracle: every (K, N, group) with u8, u4
and i4 weights, full / scalar / absent zero-points, with and without bias, 3-D activations flattened to rows as the
CPU path does.  Those tests compare with an interpreter on random data; here the oracle stands in for it."""
import numpy as np
import pytest

from openvino_amd import datagen, fc
from parity import check_parity, oracle_y

pytestmark = pytest.mark.gpu

# (activation shapes, (K, N), group size or None for one group per channel)
REFERENCE_SHAPES = [
    ([(1, 4, 16), (10, 16, 16)], (16, 32), None),
    ([(1, 8, 16)], (16, 32), 4),
    ([(5, 40, 496)], (496, 240), None),
    ([(1, 4, 48)], (48, 256), None),
    ([(1, 11, 154)], (154, 77), 154),
    ([(10, 40, 480), (11, 40, 480)], (480, 256), None),
    ([(1, 4, 32)], (32, 256), None),
    ([(1, 16, 32)], (32, 64), None),
    ([(2, 4, 32)], (32, 65), None),
    ([(3, 12, 768)], (768, 1024), None),
    ([(3, 339, 577)], (577, 335), None),       # odd K and N: rows of the packed constants share bytes
    ([(1, 1, 256)], (256, 128), 64),
]


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


@pytest.mark.parametrize("zp_form", ["full", "scalar", "empty"])
@pytest.mark.parametrize("wt", ["u8", "u4", "i4"])
@pytest.mark.parametrize("shapes,kn,group", REFERENCE_SHAPES, ids=[f"{k}x{n}g{g}" for _, (k, n), g in REFERENCE_SHAPES])
def test_reference_functional_shapes(oracle, dev, req, shapes, kn, group, wt, zp_form):
    K, N = kn
    G = group or K
    if wt == "i4" and zp_form != "empty":
        pytest.skip("signed weights come without zero-points")
    zt = "none" if zp_form == "empty" else ("u4" if wt == "u4" else "u8")
    for bias in (False, True):
        c = datagen.make_case(1200 + K + N, 1, K, N, wt, G, zt, with_bias=bias)
        if zp_form == "scalar":
            c.zp, c.zp_scalar = np.array([7 if wt == "u4" else 121], np.uint8), True
        w = fc.CompressedWeights.from_case(dev, c)
        try:
            for shape in shapes:
                print(f"reference shape {shape} x ({K},{N}) G={G} {wt} zp={zp_form} bias={bias}", flush=True)
                x = np.random.default_rng(sum(shape)).standard_normal(shape).astype(np.float16)
                y = req.infer(w, x)                                  # leading dimensions flatten to rows
                assert y.shape == shape[:-1] + (N,)
                rows = x.reshape(-1, K)
                pick = np.arange(rows.shape[0]) if rows.shape[0] <= 64 else \
                    np.sort(np.random.default_rng(1).choice(rows.shape[0], 64, replace=False))
                ref = oracle_y(oracle, c, x=rows[pick])
                check_parity(oracle, y.reshape(-1, N)[pick], ref, K, f"{req.last_kernel()}", output_rounding_slack=True)
        finally:
            w.close()
