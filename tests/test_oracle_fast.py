"""The blocked, vectorised CPU port that the benchmark times as its CPU baseline (oracle/oracle_fast.c) against the
exact restatement: the same formula, a different order of the f32 sum."""
import numpy as np
import pytest

from openvino_amd import datagen


@pytest.mark.parametrize("wt,zt,G,K,N,bias", [("u4", "u4", 128, 512, 72, True), ("i4", "none", 128, 384, 33, False),
                                             ("u8", "u8", 256, 256, 40, True), ("i8", "none", 96, 96, 5, False),
                                             ("u4", "u8", 32, 160, 64, True)])
@pytest.mark.parametrize("M", [1, 3, 4, 9, 70])
def test_blocked_port_agrees_with_the_oracle(oracle, wt, zt, G, K, N, bias, M):
    c = datagen.make_case(1400 + M, M, K, N, wt, G, zt, with_bias=bias)
    T = oracle.TYPE_NAMES
    ref = oracle.fc_reference(c.x, c.w, T[wt], c.scale, c.zp, T[zt], c.bias, N=N, K=K, group_size=G)
    ref64 = oracle.fc_reference(c.x, c.w, T[wt], c.scale, c.zp, T[zt], c.bias, N=N, K=K, group_size=G, acc_f64=True)
    got = oracle.fc_reference(c.x, c.w, T[wt], c.scale, c.zp, T[zt], c.bias, N=N, K=K, group_size=G, blocked=True)
    assert got.shape == ref.shape
    # both f32 sums sit within summation-order distance of the f64 sum; the blocked one no further than the plain one
    assert oracle.rel_l2(got, ref64) < 1e-6
    assert oracle.rel_l2(got, ref64) <= 2 * oracle.rel_l2(ref, ref64) + 1e-7


def test_blocked_port_scalar_zero_point_and_rejections(oracle):
    c = datagen.make_case(1410, 6, 256, 48, "u4", 128, "u4")
    zp = np.array([9], np.uint8)
    a = oracle.fc_reference(c.x, c.w, oracle.U4, c.scale, zp, oracle.U8, None, N=48, K=256, group_size=128, zp_scalar=True)
    b = oracle.fc_reference(c.x, c.w, oracle.U4, c.scale, zp, oracle.U8, None, N=48, K=256, group_size=128, zp_scalar=True,
                            blocked=True)
    assert oracle.rel_l2(b, a) < 1e-6
    with pytest.raises(ValueError):
        oracle.fc_reference(c.x, c.w, oracle.U4, c.scale, None, oracle.NONE, None, N=48, K=256, group_size=128,
                            n_index=[1, 2], blocked=True)
