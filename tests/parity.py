"""Shared helpers of the GPU parity tests: run a case through the C ABI and compare with the oracle."""
import math

import numpy as np

from openvino_amd import _lib, datagen, fc

T = {"u4": 1, "i4": 2, "u8": 3, "i8": 4}
ZT = {"none": 0, "u4": 1, "u8": 3}

REL_L2_MAX = 1e-3                       # vs the fp32 dequantise-then-matmul oracle


def max_abs_limit(K: int) -> float:
    return 2e-2 * math.sqrt(K / 4096.0)


def oracle_y(o, c: datagen.FcCase, x=None, n_index=None, acc_f64=False):
    return o.fc_reference(c.x if x is None else x, c.w, T[c.w_type], c.scale, c.zp, ZT[c.zp_type], c.bias,
                          N=c.N, K=c.K, group_size=c.group_size, zp_scalar=c.zp_scalar, n_index=n_index,
                          acc_f64=acc_f64)


def check_parity(o, y_gpu, y_ref, K, what="", output_rounding_slack=False, limit_scale=1.0):
    """Both north-star bounds; returns (rel_l2, max_abs) for reporting.

    The max-abs bound 2e-2*sqrt(K/4096) is stated for the benchmark distributions.  Tests on other
    distributions (small K, large outputs) set output_rounding_slack, which adds half a float16 ulp of the
    largest reference output: the rounding of the f16 result itself, which no kernel can avoid."""
    y = np.asarray(y_gpu, dtype=np.float32)
    assert y.shape == y_ref.shape, (what, y.shape, y_ref.shape)
    assert np.all(np.isfinite(y)), what
    rl2 = o.rel_l2(y, y_ref)
    mab = o.max_abs(y, y_ref)
    limit = max_abs_limit(K) * limit_scale
    if output_rounding_slack and y_ref.size:
        limit += float(np.max(np.abs(y_ref))) * 2.0 ** -11
    assert rl2 <= REL_L2_MAX, f"{what}: rel-L2 {rl2:.3e} > {REL_L2_MAX}"
    assert mab <= limit, f"{what}: max-abs {mab:.3e} > {limit:.3e}"
    return rl2, mab


def glu_reference(o, c: datagen.FcCase, kind: str, gate_second=False, x=None):
    """Oracle of a node with a gated-linear-unit epilogue, and the factor by which the epilogue can amplify the
    north-star max-abs bound of the FullyConnected underneath: with out = act(g) u, |act'| <= 1.13 and
    |act(g)| <= |g|, an error d on g and u moves out by at most d (1.13 |u| + |g|)."""
    y = oracle_y(o, c, x=x)
    ref = o.glu(y, {"swish": 1, "gelu": 2, "gelu_tanh": 3}[kind], gate_second)
    return ref, 2.13 * max(1.0, float(np.max(np.abs(y))) if y.size else 1.0)


def run_case(dev, req, c: datagen.FcCase, x=None):
    w = fc.CompressedWeights.from_case(dev, c)
    try:
        return req.infer(w, c.x if x is None else x), req.last_kernel()
    finally:
        w.close()
