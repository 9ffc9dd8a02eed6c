"""The gate adjoints of a diagonal have a finite horizon, so a band can be cut at any row.

Along a diagonal the gradient pass walks upwards with
    b(n) = A(n) + g(n+1) b(n+1),    h(n) = b(n) (S(n) + o(n)) - sum_{m=n..n+W} b(m) o(m),
where o(n) is the product of the W + 1 gates ending at n (zero while the window is not full).
h(n) depends on A(m) only for m <= n + W - 1 (the reference's O(W) form sums exactly those
terms: benchmarks/diagonal_recurrence.py:150-214), so the rows above a cut are reproduced by a
walk that starts W - 1 rows below the cut with b = 0 and an empty window sum.  This is what lets
the gradient kernel hand pieces of a long band to different waves; float64, no device.
"""

import numpy as np
import pytest


def forward(gates, window):
    n = len(gates)
    evidence = np.zeros(n)
    overflow = np.zeros(n)
    previous = 0.0
    for i in range(n):
        if i >= window:  # the W + 1 gates i - W .. i exist
            overflow[i] = np.prod(gates[i - window:i + 1])
        evidence[i] = gates[i] * (1.0 + previous) - overflow[i]
        previous = evidence[i]
    return evidence, overflow


def reverse_walk(gates, adjoint, evidence, overflow, window, start, stop):
    """Gate adjoints of rows stop .. start - 1, walking up from row start - 1 with b = 0."""

    n = len(gates)
    h = np.zeros(n)
    b_below, terms = 0.0, {}
    for i in range(start - 1, stop - 1, -1):
        gate_below = gates[i + 1] if i + 1 < n else 0.0
        b = adjoint[i] + (gate_below * b_below if i + 1 < start else 0.0)
        terms[i] = b * overflow[i]
        window_sum = sum(terms.get(m, 0.0) for m in range(i, i + window + 1))
        h[i] = b * (evidence[i] + overflow[i]) - window_sum
        b_below = b
    return h


def direct_adjoints(gates, adjoint, window):
    """dL/dlog g(n) by the definition S(m) = sum_{l=1..W} prod_{r<l} g(m - r)."""

    n = len(gates)
    h = np.zeros(n)
    for m in range(n):
        for length in range(1, min(window, m + 1) + 1):
            product = np.prod(gates[m - length + 1:m + 1])
            h[m - length + 1:m + 1] += adjoint[m] * product
    return h


@pytest.mark.parametrize("pattern", ["random", "all_match", "periodic"])
@pytest.mark.parametrize("window", [1, 3, 8, 40])
def test_a_walk_started_below_a_cut_reproduces_the_rows_above_it(pattern, window):
    rng = np.random.default_rng(7 + window)
    n = 60
    if pattern == "random":
        gates = np.exp(-rng.integers(0, 5, n) * 0.75)
    elif pattern == "all_match":
        gates = np.ones(n)
    else:
        gates = np.where(np.arange(n) % 7 == 3, np.exp(-1.5), 1.0)
    adjoint = rng.standard_normal(n)
    evidence, overflow = forward(gates, window)
    whole = reverse_walk(gates, adjoint, evidence, overflow, window, n, 0)
    # the recurrence itself against the definition
    np.testing.assert_allclose(whole, direct_adjoints(gates, adjoint, window), rtol=1e-10, atol=1e-12)
    for cut in (5, 16, 31, 47):
        halo_start = min(n, cut + window - 1)  # rows cut .. cut + W - 2 are the halo
        piece = reverse_walk(gates, adjoint, evidence, overflow, window, halo_start, 0)
        np.testing.assert_allclose(piece[:cut], whole[:cut], rtol=1e-10, atol=1e-12)
        # one row less of halo is not enough in general
        if pattern == "all_match" and cut + window - 1 < n and window > 2:
            short = reverse_walk(gates, adjoint, evidence, overflow, window, cut + window - 2, 0)
            assert not np.allclose(short[:cut], whole[:cut], rtol=1e-10, atol=1e-12)
