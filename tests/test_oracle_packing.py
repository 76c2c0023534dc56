"""Pins the oracle's 4-bit element access against the reference's known-answer bytes
(src/core/tests/element_iterator_test.cpp, uint4.cpp, int4.cpp) and, where it was built,
against the reference's own element_iterator.hpp (oracle/_ref)."""
import numpy as np
import pytest

from golden_cases import packing_cases

CASES = packing_cases()


@pytest.mark.parametrize("case", CASES, ids=[c["id"] for c in CASES])
def test_known_answer(oracle, case):
    raw = np.array(case["bytes"], dtype=np.uint8)
    n = len(case["elements"])
    if case["op"] == "read":
        got = oracle.unpack_u4(raw, n) if case["type"] == "u4" else oracle.unpack_i4(raw, n)
        assert got.tolist() == case["elements"]
        got_np = oracle.np_unpack_nibbles(raw, n, case["type"] == "i4")
        assert got_np.tolist() == case["elements"]
    else:
        got = (oracle.pack_u4(np.array(case["elements"], np.uint8)) if case["type"] == "u4"
               else oracle.pack_i4(np.array(case["elements"], np.int8)))
        assert got.tolist() == case["bytes"]


def test_pack_unpack_round_trip(oracle):
    rng = np.random.default_rng(7)
    for n in (1, 2, 3, 17, 256, 4097):
        u = rng.integers(0, 16, n, dtype=np.uint8)
        assert np.array_equal(oracle.unpack_u4(oracle.pack_u4(u), n), u)
        i = rng.integers(-8, 8, n).astype(np.int8)
        assert np.array_equal(oracle.unpack_i4(oracle.pack_i4(i), n), i)
        # i4 and u4 views of the same bytes differ by the sign extension only
        b = oracle.pack_i4(i)
        assert np.array_equal(oracle.unpack_u4(b, n).astype(np.int16), np.where(i < 0, i + 16, i))


def test_against_reference_iterator(oracle):
    ref = oracle.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(11)
    for n in (1, 2, 3, 16, 33, 1000):
        raw = rng.integers(0, 256, (n + 1) // 2, dtype=np.uint8)
        u = np.empty(n, np.uint8)
        i = np.empty(n, np.int8)
        ref.ref_unpack_u4(raw.ctypes.data, n, u.ctypes.data)
        ref.ref_unpack_i4(raw.ctypes.data, n, i.ctypes.data)
        assert np.array_equal(oracle.unpack_u4(raw, n), u)
        assert np.array_equal(oracle.unpack_i4(raw, n), i)
        vals = rng.integers(0, 16, n, dtype=np.uint8)
        out = np.zeros((n + 1) // 2, np.uint8)
        ref.ref_pack_u4(vals.ctypes.data, n, out.ctypes.data)
        assert np.array_equal(oracle.pack_u4(vals), out)
        svals = rng.integers(-8, 8, n).astype(np.int8)
        out = np.zeros((n + 1) // 2, np.uint8)
        ref.ref_pack_i4(svals.ctypes.data, n, out.ctypes.data)
        assert np.array_equal(oracle.pack_i4(svals), out)
