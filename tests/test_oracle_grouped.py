"""Pins of the oracle's GroupedMatMul (oracle.grouped_matmul_reference) that a plausible mistake fails: offsets read
as counts instead of cumulative ends, an empty group that shifts the groups after it, rows beyond the last offset
not zero, groups of the 3-D form multiplied with the wrong group's weights.  The expected numbers are worked out
here by the loops of the reference (src/core/reference/include/openvino/reference/grouped_matmul.hpp:17-88) over
integer matrices, not by the oracle's own code."""
import numpy as np

from oracle import oracle

G, N, K = 3, 2, 2
# B[g] as integers (u8 codes, scale 1, no zero-point): group g's matrix is [[g + 1, 2], [0, g + 3]]
B = np.array([[[g + 1, 2], [0, g + 3]] for g in range(G)], dtype=np.uint8)


def group_args(g):
    return dict(w=B[g].reshape(-1), w_type=oracle.U8, scale=np.ones((N, 1), np.float32), zp=None, zp_type=oracle.NONE,
                bias=None, N=N, K=K, group_size=K)


def loops_2d_3d(a, offsets):
    rows = a.shape[0]
    out = [[0.0] * N for _ in range(rows)]
    start = 0
    for g in range(G):
        end = int(offsets[g])
        for i in range(start, end):
            for j in range(N):
                for k in range(K):
                    out[i][j] += float(a[i][k]) * float(B[g][j][k])
        start = end
    return np.array(out, np.float32)


def test_offsets_are_cumulative_ends_and_a_group_may_be_empty():
    a = np.array([[1, 0], [0, 1], [1, 1], [2, -1]], dtype=np.float32)
    offsets = [2, 2, 3]      # group 0: rows 0-1, group 1: none, group 2: row 2, row 3: nobody's
    y = oracle.grouped_matmul_reference(a, [group_args(g) for g in range(G)], offsets)
    want = np.array([[1, 0], [2, 3], [5, 5], [0, 0]], dtype=np.float32)   # by hand from B above
    assert np.array_equal(loops_2d_3d(a, offsets), want)
    assert np.array_equal(y, want)


def test_all_rows_to_the_last_group_and_no_rows_at_all():
    a = np.array([[1, 2], [3, 4]], dtype=np.float32)
    y = oracle.grouped_matmul_reference(a, [group_args(g) for g in range(G)], [0, 0, 2])
    assert np.array_equal(y, np.array([[7, 10], [17, 20]], dtype=np.float32))   # B[2] = [[3, 2], [0, 5]]
    y0 = oracle.grouped_matmul_reference(np.zeros((0, K), np.float32), [group_args(g) for g in range(G)], [0, 0, 0])
    assert y0.shape == (0, N)


def test_three_d_form_pairs_group_g_with_weights_g():
    a = np.array([[[1, 1]], [[1, 1]], [[1, 1]]], dtype=np.float32)     # [G, 1, K]
    y = oracle.grouped_matmul_reference(a, [group_args(g) for g in range(G)])
    assert y.shape == (G, 1, N)
    assert np.array_equal(y[:, 0], np.array([[3, 3], [4, 4], [5, 5]], dtype=np.float32))


def test_against_the_loops_on_random_integers():
    rng = np.random.default_rng(4)
    for _ in range(20):
        rows = int(rng.integers(0, 9))
        a = rng.integers(-3, 4, size=(rows, K)).astype(np.float32)
        cuts = np.sort(rng.integers(0, rows + 1, size=G))
        y = oracle.grouped_matmul_reference(a, [group_args(g) for g in range(G)], cuts)
        assert np.array_equal(y, loops_2d_3d(a, cuts).reshape(rows, N)), (rows, cuts)
