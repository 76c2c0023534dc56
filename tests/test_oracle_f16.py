"""Pins the oracle's binary16 conversion: IEEE round-to-nearest-even, as
src/core/src/type/float16.cpp:32-140 implements it.  Checked against numpy.float16 (an
independent IEEE implementation), the exhaustive 65536-pattern round trip, hand-derived
ties, and the reference's own float16.cpp where oracle/_ref was built."""
import numpy as np
import pytest


def test_all_half_patterns_round_trip(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_bits_to_f32(bits)
    expect = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(expect)
    assert np.array_equal(f[~nan], expect[~nan])
    assert np.all(np.isnan(f[nan]))
    back = oracle.f32_to_f16_bits(f)
    assert np.array_equal(back[~nan], bits[~nan])


def test_known_roundings(oracle):
    cases = {
        1.0: 0x3C00, -2.0: 0xC000, 65504.0: 0x7BFF,
        65519.99: 0x7BFF,          # just below the overflow tie
        65520.0: 0x7C00,           # tie between 65504 and 2^16 rounds to even = inf
        1.0 + 2.0 ** -11: 0x3C00,  # tie, mantissa even: down
        1.0 + 3 * 2.0 ** -11: 0x3C02,  # tie, mantissa odd: up
        2.0 ** -24: 0x0001, 2.0 ** -25: 0x0000,  # tie to even at the smallest subnormal
        1.5 * 2.0 ** -24: 0x0002, 2.0 ** -14: 0x0400,
        (2.0 ** -14) * (1 - 2.0 ** -12): 0x0400,  # largest-subnormal side rounds up to the smallest normal
        0.0: 0x0000, 1e-45: 0x0000, float("inf"): 0x7C00, float("-inf"): 0xFC00,
    }
    x = np.array(list(cases.keys()), dtype=np.float32)
    got = oracle.f32_to_f16_bits(x)
    assert got.tolist() == list(cases.values())
    assert oracle.f32_to_f16_bits(np.array([-0.0], np.float32))[0] == 0x8000


def test_matches_numpy_on_random_floats(oracle):
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    # concentrate half of the samples on half's own range so ties and subnormals are hit
    x = bits.view(np.float32).copy()
    x[::2] = (rng.standard_normal(x[::2].size) * np.exp2(rng.integers(-26, 17, x[::2].size))).astype(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        expect = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16_bits(x), expect)


def test_against_reference_float16(oracle):
    ref = oracle.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(20000) * np.exp2(rng.integers(-27, 18, 20000))).astype(np.float32)
    x = np.concatenate([x, np.array([65504, 65520, 65519.9, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25, 0, -0.0,
                                     np.inf, -np.inf], np.float32)])
    ours = oracle.f32_to_f16_bits(x)
    theirs = np.array([ref.ref_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    # The reference's software routine is IEEE round-to-nearest-even except for one corner: when the
    # result is subnormal and rounding the float's significand to 11 bits carries into the exponent
    # (float mantissa >= 0x7FF000), float16.cpp:77-84 bumps the exponent and then shifts the
    # unrounded significand by the bumped exponent, doubling the result (e.g. 7.9986*2^-24 -> 0x0010
    # where IEEE, numpy and the GPU's conversion give 0x0008).  The oracle follows IEEE; outputs of
    # this path never sit in half's subnormal range at the tested configurations.
    subnormal_result = np.abs(x) < 2.0 ** -14
    carry = (x.view(np.uint32) & 0x7FFFFF) >= 0x7FF000
    quirk = subnormal_result & carry
    assert np.array_equal(ours[~quirk], theirs[~quirk])
    with np.errstate(over="ignore"):
        assert np.array_equal(ours, x.astype(np.float16).view(np.uint16))
    for h in list(range(0, 0x7C01)) + list(range(0x8000, 0xFC01)):
        assert oracle.lib().ovo_f16_to_f32(h) == ref.ref_f16_to_f32(h)
