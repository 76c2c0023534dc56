"""GPU parity of GroupedMatMulCompressed (ovfcc_grouped_matmul_device) against the oracle, on the shapes and row
distributions of the reference's own functional test of the op
(src/plugins/intel_cpu/tests/functional/custom/single_layer_tests/instances/x64/grouped_matmul_compressed.cpp:21-33:
3-D x 3-D with a dynamic row count, 2-D x 3-D with tokens per expert that leave experts without rows; weights u8, i8,
u4, i4; zero-points per group, scalar, none), on a mixture-of-experts layer of the benchmark's proportions, and on
what the reference's arithmetic leaves to the caller: rows beyond the last offset, bad offsets."""
import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc
from parity import check_parity
from test_oracle_moe import expert_args

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


def make_groups(dev, seed, G, N, K, wt, zp_kind, group, out="f16"):
    """zp_kind: 'full' (one per channel and group), 'scalar', 'empty' -- the reference's DecompressionType."""
    zt = "none" if zp_kind == "empty" else ("u4" if wt in ("u4", "i4") else "u8")
    cases = []
    for g in range(G):
        c = datagen.make_case(seed + g, 1, K, N, wt, group, zt, scale_range=(0.01, 0.03),
                              zp_range=(100, 156) if zt == "u8" else None)
        if zp_kind == "scalar" and zt != "none":
            zp = np.array([7], dtype=np.uint8)
            c = datagen.FcCase(c.M, c.K, c.N, c.group_size, c.w_type, "u8", c.w, c.scale, zp, c.x, c.bias, zp_scalar=1)
        cases.append(c)
    return cases, [fc.CompressedWeights.from_case(dev, c, output_type=out) for c in cases]


def args_of(c):
    a = expert_args(c)
    a["zp_scalar"] = bool(getattr(c, "zp_scalar", 0))
    return a


# (G, N, K), row counts of the 3-D form, tokens per expert of the 2-D form
REFERENCE_SHAPES = [
    ((4, 256, 128), [8, 1, 16], [[8, 0, 8, 0], [0, 16, 0, 16], [4, 4, 0, 0], [4, 5, 3, 0], [0, 7, 6, 7]]),
    ((8, 512, 256), [4, 1], [[4, 2, 2, 2, 2, 2, 1, 1], [2, 6, 4, 4, 4, 4, 4, 4]]),
]


@pytest.mark.parametrize("shape,ms,tokens", REFERENCE_SHAPES)
@pytest.mark.parametrize("wt", ["u8", "i8", "u4", "i4"])
@pytest.mark.parametrize("zp_kind", ["full", "scalar", "empty"])
@pytest.mark.parametrize("group", [-1, 128])
def test_reference_functional_shapes(oracle, dev, req, shape, ms, tokens, wt, zp_kind, group):
    G, N, K = shape
    gs = K if group < 0 else group
    if gs > K:
        pytest.skip("group larger than K")
    cases, ws = make_groups(dev, 8100 + N, G, N, K, wt, zp_kind, gs, out="f32")
    groups = [args_of(c) for c in cases]
    rng = np.random.default_rng(8101)
    try:
        for M in ms:
            say(f"grouped 3-D {shape} {wt} zp={zp_kind} G={gs} M={M}")
            a = rng.uniform(-1, 1, size=(G, M, K)).astype(np.float16)
            y = req.grouped_matmul(ws, a, y_fill=77.0)
            assert y.shape == (G, M, N)
            check_parity(oracle, y.reshape(G * M, N), oracle.grouped_matmul_reference(a, groups).reshape(G * M, N), K,
                         f"3-D M={M}", output_rounding_slack=True)
        for tpe in tokens:
            say(f"grouped 2-D {shape} {wt} zp={zp_kind} G={gs} tokens={tpe}")
            offsets = np.cumsum(tpe).astype(np.int32)
            a = rng.uniform(-1, 1, size=(int(offsets[-1]), K)).astype(np.float16)
            y = req.grouped_matmul(ws, a, offsets, y_fill=77.0)
            check_parity(oracle, y, oracle.grouped_matmul_reference(a, groups, offsets), K, f"2-D {tpe}",
                         output_rounding_slack=True)
    finally:
        for w in ws:
            w.close()


@pytest.mark.parametrize("wt", ["u8", "i8"])
def test_reference_corner_shape_odd_k(oracle, dev, req, wt):
    """K = 77, N = 123 (the reference's corner case), 8-bit weights, one group per channel."""
    G, N, K = 4, 123, 77
    cases, ws = make_groups(dev, 8200, G, N, K, wt, "full", K, out="f32")
    groups = [args_of(c) for c in cases]
    rng = np.random.default_rng(8201)
    try:
        for tpe in ([4, 5, 3, 0], [0, 7, 6, 7]):
            offsets = np.cumsum(tpe).astype(np.int32)
            a = rng.uniform(-1, 1, size=(int(offsets[-1]), K)).astype(np.float16)
            # rows of A are 154 bytes: whichever kernel the library picks must not need more alignment than that
            y = req.grouped_matmul(ws, a, offsets)
            check_parity(oracle, y, oracle.grouped_matmul_reference(a, groups, offsets), K, f"corner {tpe}",
                         output_rounding_slack=True)
        a = rng.uniform(-1, 1, size=(G, 8, K)).astype(np.float16)
        y = req.grouped_matmul(ws, a)
        check_parity(oracle, y.reshape(-1, N), oracle.grouped_matmul_reference(a, groups).reshape(-1, N), K, "corner 3-D",
                     output_rounding_slack=True)
    finally:
        for w in ws:
            w.close()


def test_rows_beyond_the_last_offset_are_zero_and_bad_offsets_are_refused(oracle, dev, req):
    G, N, K = 4, 256, 128
    cases, ws = make_groups(dev, 8300, G, N, K, "u4", "full", 128)
    groups = [args_of(c) for c in cases]
    a = np.random.default_rng(8301).uniform(-1, 1, size=(20, K)).astype(np.float16)
    try:
        offsets = np.array([3, 3, 9, 14], np.int32)          # rows 14-19 belong to no group
        y = req.grouped_matmul(ws, a, offsets, y_fill=5.0)
        assert np.all(y[14:] == 0)
        check_parity(oracle, y, oracle.grouped_matmul_reference(a, groups, offsets), K, "tail", output_rounding_slack=True)
        y0 = req.grouped_matmul(ws, a, np.zeros(G, np.int32), y_fill=5.0)   # nobody has rows
        assert np.all(y0 == 0)
        for bad in ([3, 2, 9, 14], [3, 3, 9, 21], [-1, 3, 9, 14]):
            with pytest.raises(fc.OvfccError) as e:
                req.grouped_matmul(ws, a, np.array(bad, np.int32))
            assert e.value.code == _lib.EINVAL, bad
        assert req.grouped_matmul(ws, np.zeros((0, K), np.float16), np.zeros(G, np.int32)).shape == (0, N)
    finally:
        for w in ws:
            w.close()


def test_expert_layer_of_the_benchmarks_proportions(oracle, dev, req):
    """Eight experts of 1024 -> 3584 with 54-71 rows each (config 5 at a quarter of its width): the grouped prefill
    launch; the same bits on a second call; equal to the experts run one by one."""
    G, N, K = 8, 3584, 1024
    cases, ws = make_groups(dev, 8400, G, N, K, "u4", "full", 128)
    groups = [args_of(c) for c in cases]
    tpe = [65, 64, 54, 71, 70, 70, 56, 62]
    offsets = np.cumsum(tpe).astype(np.int32)
    a = np.random.default_rng(8401).standard_normal((int(offsets[-1]), K)).astype(np.float16)
    try:
        y = req.grouped_matmul(ws, a, offsets)
        say(f"   {req.last_kernel()}")
        assert "grouped" in req.last_kernel()["name"]
        check_parity(oracle, y, oracle.grouped_matmul_reference(a, groups, offsets), K, "expert layer",
                     output_rounding_slack=True)
        assert np.array_equal(req.grouped_matmul(ws, a, offsets).view(np.uint8), y.view(np.uint8))
        start = 0
        for g, end in enumerate(offsets.tolist()):
            one = req.infer(ws[g], a[start:end])
            assert oracle.rel_l2(y[start:end].astype(np.float32), one.astype(np.float32)) < 2e-3, g
            start = end
    finally:
        for w in ws:
            w.close()


@pytest.mark.parametrize("tpe,tail", [([65, 64, 54, 71, 70, 70, 56, 62], 0), ([0, 200, 0, 0, 3, 0, 129, 0], 9),
                                      ([1, 1, 1, 1, 1, 1, 1, 1], 0), ([0, 0, 0, 0, 0, 0, 0, 0], 5)])
def test_offsets_in_device_memory(oracle, dev, req, tpe, tail):
    """The same op with the offsets read on the device: against the oracle, and against the host-offset call; rows
    beyond the last offset are zeros; nothing waits for the stream in between."""
    G, N, K = 8, 1024, 512
    cases, ws = make_groups(dev, 8500, G, N, K, "u4", "scalar", 128)
    groups = [args_of(c) for c in cases]
    offsets = np.cumsum(tpe).astype(np.int32)
    rows = int(offsets[-1]) + tail
    a = np.random.default_rng(8501).standard_normal((rows, K)).astype(np.float16)
    try:
        y = req.grouped_matmul(ws, a, offsets, y_fill=3.0, device_offsets=True)
        say(f"   tokens {tpe} tail {tail}: {req.last_kernel()['name']}")
        assert req.last_kernel()["name"] == "fcc_prefill_async_grouped_w4"
        assert np.all(y[int(offsets[-1]):] == 0)
        check_parity(oracle, y, oracle.grouped_matmul_reference(a, groups, offsets), K, f"device offsets {tpe}",
                     output_rounding_slack=True)
        host = req.grouped_matmul(ws, a, offsets, y_fill=3.0)
        assert oracle.rel_l2(y.astype(np.float32), host.astype(np.float32)) < 2e-3 if rows else True
        assert np.array_equal(req.grouped_matmul(ws, a, offsets, device_offsets=True).view(np.uint8), y.view(np.uint8))
    finally:
        for w in ws:
            w.close()


def test_device_offsets_out_of_order_lose_rows_but_stay_inside(oracle, dev, req):
    """What the host form refuses cannot be checked without reading the offsets: a value below its predecessor or
    above the row count is taken as that bound."""
    G, N, K = 4, 512, 256
    cases, ws = make_groups(dev, 8600, G, N, K, "i4", "empty", 128)
    groups = [args_of(c) for c in cases]
    a = np.random.default_rng(8601).standard_normal((40, K)).astype(np.float16)
    try:
        y = req.grouped_matmul(ws, a, np.array([10, 5, 30, 99], np.int32), y_fill=2.0, device_offsets=True)
        clamped = np.array([10, 10, 30, 40], np.int32)
        check_parity(oracle, y, oracle.grouped_matmul_reference(a, groups, clamped), K, "clamped", output_rounding_slack=True)
        # 8-bit groups have no launch that reads its slices from memory
        c8, w8 = make_groups(dev, 8610, G, N, K, "u8", "full", K)
        try:
            with pytest.raises(fc.OvfccError) as e:
                req.grouped_matmul(w8, a, clamped, device_offsets=True)
            assert e.value.code == _lib.EUNSUPPORTED
        finally:
            for w in w8:
                w.close()
    finally:
        for w in ws:
            w.close()
