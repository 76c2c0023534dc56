"""The entry point that allocates nothing, ovfcc_fc_run_device_static, against ovfcc_fc_run_device: same kernels, so
the outputs must agree bit for bit -- on launches that split K (their partial tiles and arrival counters then live
in the fixed scratch array), on two calls in a row of which the second is smaller, across requests, and after the
array has been used by a different shape.  Launches beyond the array's size are refused with a clear error."""
import sys

import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def dev():
    d = fc.Device(0)
    yield d
    d.close()


def run_both(dev, req, w, x, out_bytes_per_el=2):
    """(static entry point, allocating entry point) outputs as raw bytes for x [M, K]."""
    M = x.shape[0]
    n_out = w.N_out
    x_ptr = dev.malloc(max(16, x.nbytes))
    ya, yb = dev.malloc(max(16, M * n_out * out_bytes_per_el)), dev.malloc(max(16, M * n_out * out_bytes_per_el))
    try:
        dev.upload(x_ptr, np.ascontiguousarray(x))
        req.infer_device_static(w, x_ptr, ya, M)
        info = req.last_kernel()
        req.infer_device(w, x_ptr, yb, M)
        req.sync()
        a = dev.download(ya, (M, n_out * out_bytes_per_el), np.uint8)
        b = dev.download(yb, (M, n_out * out_bytes_per_el), np.uint8)
        return a, b, info
    finally:
        for p in (x_ptr, ya, yb):
            dev.free(p)


def test_static_entry_point_matches_on_split_k_launches(oracle, dev):
    req = fc.InferRequest(dev)
    other = fc.InferRequest(dev)
    # a prefill launch that splits K (few tiles, long K), then smaller calls on the same node, then a decode launch
    # that splits K on a different shape, then the first shape again from another request
    c1 = datagen.make_case(9100, 512, 4096, 1024, "i4", 128, "none")
    c2 = datagen.make_case(9101, 24, 8192, 256, "u4", 128, "u4", with_bias=True)
    w1 = fc.CompressedWeights.from_case(dev, c1)
    w2 = fc.CompressedWeights.from_case(dev, c2)
    try:
        seen_split = 0
        for r, w, c, M in ((req, w1, c1, 512), (req, w1, c1, 300), (req, w1, c1, 1), (req, w2, c2, 24),
                           (req, w2, c2, 7), (other, w1, c1, 512), (req, w1, c1, 64)):
            a, b, info = run_both(dev, r, w, c.x[:M])
            say(f"static M={M} N={c.N} K={c.K}: {info['name']} split {info['split_k']}")
            seen_split += info["split_k"] > 1
            assert np.array_equal(a, b), (M, info)
        assert seen_split >= 3
        # and the result is the oracle's, not merely the same as the other entry point's
        from parity import check_parity, oracle_y
        x_ptr, y_ptr = dev.malloc(c1.x[:300].nbytes), dev.malloc(300 * c1.N * 2)
        dev.upload(x_ptr, np.ascontiguousarray(c1.x[:300]))
        req.infer_device_static(w1, x_ptr, y_ptr, 300)
        req.sync()
        y = dev.download(y_ptr, (300, c1.N), np.float16)
        pick = np.arange(0, 300, 37)
        check_parity(oracle, y[pick], oracle_y(oracle, c1, x=c1.x[pick]), c1.K, "static vs oracle")
        dev.free(x_ptr)
        dev.free(y_ptr)
    finally:
        w1.close()
        w2.close()
        req.close()
        other.close()


def test_static_entry_point_allocates_nothing_and_orders_its_streams(dev):
    """Free device memory reads the same before and after calls of the static entry point that split K (the
    allocating entry point, on a fresh request, does take memory for its partial tiles: the check can see an
    allocation).  And two requests -- two streams -- that call it back to back without waiting for each other share
    the one scratch array safely: each launch waits for the one before it, so every result equals the allocating
    entry point's."""
    c = datagen.make_case(9103, 512, 4096, 1024, "i4", 128, "none")
    w = fc.CompressedWeights.from_case(dev, c)
    M = 512
    n_bytes = M * c.N * 2
    x_ptr = dev.malloc(c.x.nbytes)
    ys = [dev.malloc(n_bytes) for _ in range(9)]
    a, b = fc.InferRequest(dev), fc.InferRequest(dev)
    try:
        dev.upload(x_ptr, np.ascontiguousarray(c.x))
        a.infer_device_static(w, x_ptr, ys[0], M)   # first use: whatever the runtime sets up lazily is in place
        a.sync()
        assert a.last_kernel()["split_k"] > 1
        free0 = dev.mem_info()[0]
        for i in range(4):
            a.infer_device_static(w, x_ptr, ys[2 * i], M)
            b.infer_device_static(w, x_ptr, ys[2 * i + 1], M)
        a.sync()
        b.sync()
        assert dev.mem_info()[0] == free0, "the static entry point changed the free device memory"
        fresh = fc.InferRequest(dev)
        fresh.infer_device(w, x_ptr, ys[8], M)
        fresh.sync()
        assert dev.mem_info()[0] < free0, "an allocation of partial tiles should show in the free memory"
        want = dev.download(ys[8], (M, c.N), np.uint16)
        for i in range(8):
            assert np.array_equal(dev.download(ys[i], (M, c.N), np.uint16), want), f"call {i}"
        fresh.close()
    finally:
        a.close()
        b.close()
        w.close()
        dev.free(x_ptr)
        for p_ in ys:
            dev.free(p_)


def test_static_entry_point_refuses_what_does_not_fit(dev):
    """Partial tiles beyond 32 MiB: a clear error instead of an allocation; M = 0 is fine."""
    req = fc.InferRequest(dev)
    c = datagen.make_case(9102, 1, 8192, 2048, "i4", 128, "none")
    w = fc.CompressedWeights.from_case(dev, c)
    M = 640   # 8 x 5 tiles of 128 x 256 with K split: 40 * split * 128 KiB of partial tiles
    x_ptr, y_ptr = dev.malloc(M * c.K * 2), dev.malloc(M * c.N * 2)
    try:
        req.infer_device_static(w, x_ptr, y_ptr, 0)
        req.force_kernel(_lib.KERNEL_PREFILL, 8)
        with pytest.raises(fc.OvfccError) as err:
            req.infer_device_static(w, x_ptr, y_ptr, M)
        assert "scratch" in str(err.value)
        req.force_kernel()
        req.sync()
    finally:
        dev.free(x_ptr)
        dev.free(y_ptr)
        w.close()
        req.close()
