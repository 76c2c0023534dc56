"""Pins the oracle's gated-linear-unit formula without retyping it: library routines (torch silu / gelu in float64),
algebraic identities, and the roles of the two halves."""
import numpy as np
import pytest
import torch


def t64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


@pytest.fixture(scope="module")
def data():
    rng = np.random.default_rng(2024)
    y = (rng.standard_normal((7, 2 * 24)) * 3).astype(np.float32)
    y[0, :6] = [0.0, -0.0, 20.0, -20.0, 88.0, -88.0]          # zero, saturation on both sides
    return y


LIB = {
    1: lambda g: torch.nn.functional.silu(g),
    2: lambda g: torch.nn.functional.gelu(g, approximate="none"),
    3: lambda g: torch.nn.functional.gelu(g, approximate="tanh"),
}


@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("gate_second", [False, True])
def test_glu_matches_library_activations(oracle, data, kind, gate_second):
    L = data.shape[1] // 2
    first, second = data[:, :L], data[:, L:]
    gate, up = (second, first) if gate_second else (first, second)
    want = (LIB[kind](t64(gate)) * t64(up)).numpy()
    got = oracle.glu(data, kind, gate_second)
    assert got.shape == (data.shape[0], L) and got.dtype == np.float32
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-12)  # tanh saturates to -1 at different x


@pytest.mark.parametrize("kind", [1, 2, 3])
def test_glu_identities(oracle, kind):
    """act(x) - act(-x) = x for all three activations (x sigma(x) + x sigma(-x) = x; Phi(x) + Phi(-x) = 1; tanh odd),
    act(0) = 0, and the up half enters linearly."""
    x = np.linspace(-9, 9, 37, dtype=np.float32).reshape(1, -1)
    one = np.ones_like(x)
    pos = oracle.glu(np.concatenate([x, one], axis=1), kind)
    neg = oracle.glu(np.concatenate([-x, one], axis=1), kind)
    np.testing.assert_allclose(pos - neg, x, rtol=0, atol=2e-6)
    assert oracle.glu(np.zeros((1, 2), np.float32), kind)[0, 0] == 0.0
    up = np.full_like(x, -2.5)
    np.testing.assert_allclose(oracle.glu(np.concatenate([x, up], axis=1), kind), -2.5 * pos, rtol=1e-6)


def test_glu_halves_and_rows(oracle):
    """One-hot probes: output f reads gate f and up f of its own row only."""
    L, M = 5, 3
    for m in range(M):
        for f in range(L):
            y = np.zeros((M, 2 * L), np.float32)
            y[m, f] = 1.0          # gate f
            y[m, L + f] = 4.0      # up f
            out = oracle.glu(y, 1)
            want = np.zeros((M, L), np.float32)
            want[m, f] = 4.0 / (1.0 + np.exp(-1.0))
            np.testing.assert_allclose(out, want, rtol=1e-6)
            assert np.count_nonzero(oracle.glu(y, 1, gate_second=True)) == 1   # roles swapped: silu(4) * 1
            np.testing.assert_allclose(oracle.glu(y, 1, gate_second=True)[m, f], 4.0 / (1.0 + np.exp(-4.0)), rtol=1e-6)
    with pytest.raises(ValueError):
        oracle.glu(np.zeros((1, 3), np.float32), 1)
    with pytest.raises(ValueError):
        oracle.glu(np.zeros((1, 4), np.float32), 0)
