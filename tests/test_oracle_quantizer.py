"""Pins the oracle's Q8_0 activation quantizer (wick/src/backend/simd.rs:255-323).

The reference has no vector for the exact bits of this function, so the pin is the
committed numpy-float32 restatement (tests/golden/make_q8_0_quantizer_vectors.py)
plus the invariants the algorithm implies."""
import os

import numpy as np
import pytest

from conftest import GOLDEN


@pytest.fixture(scope="module")
def vectors():
    return np.load(os.path.join(GOLDEN, "q8_0_quantizer_vectors.npz"))


@pytest.mark.parametrize("name", ["normal", "wide", "edge"])
def test_matches_golden(oracle, vectors, name):
    x = vectors[f"{name}_x"]
    s, q = oracle.quantize_q8_0(x)
    assert np.array_equal(q, vectors[f"{name}_quants"])
    assert np.array_equal(s.view(np.uint32), vectors[f"{name}_scales"].view(np.uint32))


def test_ties_go_to_even(oracle):
    x = np.zeros(32, np.float32)
    x[:9] = [127.0, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 126.5]
    s, q = oracle.quantize_q8_0(x)
    assert s[0] == 1.0
    assert list(q[:9]) == [127, 0, 2, 2, 4, 0, -2, -2, 126]


def test_invariants(oracle):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(512 * 32) * np.exp(rng.uniform(-5, 5, 512 * 32))).astype(np.float32)
    s, q = oracle.quantize_q8_0(x)
    xb, qb = x.reshape(-1, 32), q.reshape(-1, 32).astype(np.int32)
    amax = np.abs(xb).max(axis=1)
    assert np.abs(qb).max() <= 127
    # the element of largest magnitude quantizes to +-127
    idx = np.abs(xb).argmax(axis=1)
    assert np.all(np.abs(qb[np.arange(len(idx)), idx]) == 127)
    # stored scale is f16(amax/127), widened
    d = (amax / np.float32(127)).astype(np.float32)
    assert np.array_equal(s, d.astype(np.float16).astype(np.float32))
    # reconstruction error at most half a step of the unrounded scale (plus rounding slack)
    err = np.abs(xb - qb * d[:, None])
    assert np.all(err <= d[:, None] * (0.5 + 1e-4))


def test_batch_layout(oracle):
    """scales[j*nb + b], quants[j*k + i] with a strided token-major source
    (wick/src/backend/simd.rs:683-685; wick/src/model/lfm2.rs:571-592)."""
    n, k, stride = 3, 64, 100
    x = oracle.fill_normal(9, 1.0, n * stride)
    s, q = oracle.quantize_q8_0_batch(x, n, k, stride)
    for j in range(n):
        sj, qj = oracle.quantize_q8_0(x[j * stride:j * stride + k])
        assert np.array_equal(s[j], sj) and np.array_equal(q[j], qj)
