"""Seeded random sweep through the C ABI: shapes, formats, epilogues, row counts, forced kernels and splits that no
hand-written case pairs up, each compared with the CPU oracle.  A refused combination must come back as an error code,
never as a wrong answer."""
import sys

import numpy as np
import pytest

from openvino_amd import _lib, datagen, fc
from parity import check_parity, glu_reference, oracle_y

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def dev():
    d = fc.Device(0)
    yield d
    d.close()


@pytest.mark.parametrize("seed", range(40))
def test_random_nodes(oracle, dev, seed, monkeypatch):
    rng = np.random.default_rng(7000 + seed)
    req = fc.InferRequest(dev)
    try:
        for _ in range(6):
            wt = str(rng.choice(["u4", "i4", "u8", "i8"]))
            zt = str(rng.choice(["none", "u4" if wt == "u4" else "u8"])) if wt in ("u4", "u8") else "none"
            K = int(rng.choice([128, 256, 384, 640, 1024, 200]))
            G = K if rng.random() < 0.3 else (int(rng.choice([128, 256])) if K % 256 == 0 else (128 if K % 128 == 0 else 50))
            if K % G:
                G = K
            if wt in ("u4", "i4") and K % 128 == 0 and rng.random() < 0.3:
                G = int(rng.choice([32, 64]))      # two or four groups per k-block
            N = int(rng.choice([16, 32, 48, 96, 128, 256, 272, 512, 768, 40]))
            glu = str(rng.choice(["none", "none", "swish", "gelu", "gelu_tanh"]))
            second = bool(rng.integers(0, 2)) if glu != "none" else False
            if glu != "none" and N % 2:
                glu = "none"
            bias = bool(rng.integers(0, 2))
            out = str(rng.choice(["f16", "f32"]))
            Mmax = int(rng.choice([1, 3, 7, 16, 33, 48, 50, 100, 129, 260]))
            if rng.random() < 0.5:
                monkeypatch.setenv("OVFCC_PREFILL_WIDE", "1")
            else:
                monkeypatch.delenv("OVFCC_PREFILL_WIDE", raising=False)
            c = datagen.make_case(int(rng.integers(1, 1 << 30)), Mmax, K, N, wt, G, zt, with_bias=bias)
            what = f"seed {seed}: {wt}/{zt} N={N} K={K} G={G} glu={glu}/{second} bias={bias} out={out} M={Mmax}"
            say(what)
            w = fc.CompressedWeights.from_case(dev, c, output_type=out, glu=None if glu == "none" else glu,
                                               glu_gate_second=second)
            try:
                if glu == "none":
                    ref, amp = oracle_y(oracle, c), 1.0
                else:
                    ref, amp = glu_reference(oracle, c, glu, second)
                for force, split in ((_lib.KERNEL_AUTO, 0), (int(rng.integers(1, 4)), int(rng.choice([0, 2, 5])))):
                    req.force_kernel(force, split)
                    try:
                        y = req.infer(w, c.x)
                    except fc.OvfccError as e:
                        assert force != _lib.KERNEL_AUTO, (what, str(e))     # the policy itself must always find a kernel
                        continue
                    info = req.last_kernel()
                    assert y.shape == ref.shape and y.dtype == (np.float32 if out == "f32" else np.float16)
                    check_parity(oracle, y, ref, K, f"{what} force={force}/{split} {info}", output_rounding_slack=True,
                                 limit_scale=amp)
                req.force_kernel()
                # the same node three times in a grouped run with ragged rows
                rows = [int(rng.integers(0, Mmax + 1)) for _ in range(3)]
                ys = req.infer_grouped([(w, c.x[:m]) for m in rows])
                for m, y in zip(rows, ys):
                    if m:
                        check_parity(oracle, y, ref[:m], K, f"{what} grouped rows={rows} {req.last_kernel()}",
                                     output_rounding_slack=True, limit_scale=amp)
            finally:
                req.force_kernel()
                w.close()
    finally:
        req.close()
