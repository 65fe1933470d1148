"""Pins the arithmetic of the CPU oracle: squared distance, the lane-strided dot
product of the side test, the hyperplane, and the random-number helpers.

What fixes each function (none of these tests re-types the oracle's formula in
floating point):
  * closed forms with exactly representable inputs,
  * float64 evaluation within a rounding bound,
  * scipy's sqeuclidean,
  * the perpendicular-bisector identity  n.x < b  <=>  |x-p2|^2 < |x-p1|^2,
  * an exact rational emulation of binary32 that follows the reference's loops
    (sequential chain: compute_knn_from_buckets.cu:40-54; 32 lane-strided
    partials + xor butterfly: build_tree_check_points_side.cu:131-143,
    create_node.cu:122-135) -- this one fails if the summation order changes.
"""
from fractions import Fraction

import numpy as np
import pytest
from scipy.spatial.distance import cdist

import exact32 as e32


def test_sqdist_closed_forms(orc):
    a = np.zeros(3, np.float32)
    b = np.array([1, 2, 3], np.float32)
    assert orc.sqdist(a, b) == np.float32(14.0)
    assert orc.sqdist(b, b) == np.float32(0.0)
    # one dimension only
    assert orc.sqdist(np.array([2.5], np.float32), np.array([-1.5], np.float32)) == np.float32(16.0)
    # a dropped last term or an off-by-one in D would change this
    x = np.arange(1, 101, dtype=np.float32)
    assert orc.sqdist(x, np.zeros(100, np.float32)) == np.float32(338350.0)  # sum k^2, k=1..100 (exact in fp32)


@pytest.mark.parametrize("D", [1, 2, 7, 32, 33, 100, 257, 784])
def test_sqdist_against_float64_and_scipy(orc, rng, D):
    X = rng.standard_normal((12, D)).astype(np.float32)
    ref = cdist(X.astype(np.float64), X.astype(np.float64), "sqeuclidean")
    for i in range(12):
        for j in range(12):
            got = float(orc.sqdist(X[i], X[j]))
            assert got == float(orc.sqdist(X[j], X[i]))          # symmetric bit for bit
            assert abs(got - ref[i, j]) <= 1e-5 * ref[i, j] + 1e-30
            assert abs(orc.sqdist_f64(X[i], X[j]) - ref[i, j]) <= 1e-12 * max(ref[i, j], 1.0)


def _emulate_sqdist(a, b):
    acc = Fraction(0)
    for x, y in zip(a, b):
        d = e32.sub(e32.to_frac(x), e32.to_frac(y))
        acc = e32.fma(d, d, acc)
    return e32.as_f32(acc)


@pytest.mark.parametrize("D", [3, 32, 37, 100])
def test_sqdist_is_the_sequential_fma_chain(orc, rng, D):
    for _ in range(20):
        a = rng.random(D, dtype=np.float32)
        b = rng.random(D, dtype=np.float32)
        assert orc.sqdist(a, b) == _emulate_sqdist(a, b)


def _emulate_butterfly(p):
    m = 1
    while m < 32:
        p = [e32.add(p[l], p[l ^ m]) for l in range(32)]
        m <<= 1
    return p[0]


def _emulate_dot32(n, x):
    p = [Fraction(0)] * 32
    for d in range(len(n)):
        p[d % 32] = e32.fma(e32.to_frac(n[d]), e32.to_frac(x[d]), p[d % 32])
    return e32.as_f32(_emulate_butterfly(p))


@pytest.mark.parametrize("D", [1, 5, 32, 33, 100, 200])
def test_dot32_value_and_order(orc, rng, D):
    for _ in range(10):
        n = rng.standard_normal(D).astype(np.float32)
        x = rng.random(D, dtype=np.float32)
        got = orc.dot32(n, x)
        ref = float(np.dot(n.astype(np.float64), x.astype(np.float64)))
        scale = float(np.abs(n.astype(np.float64) * x.astype(np.float64)).sum())
        assert abs(float(got) - ref) <= 1e-6 * scale + 1e-30
        assert got == _emulate_dot32(n, x)


def test_dot32_closed_form(orc):
    n = np.ones(64, np.float32)
    x = np.arange(64, dtype=np.float32)
    assert orc.dot32(n, x) == np.float32(2016.0)
    e = np.zeros(40, np.float32)
    e[37] = 3.0
    assert orc.dot32(e, np.arange(40, dtype=np.float32)) == np.float32(111.0)   # picks element 37 only


def _emulate_hyperplane_offset(x1, x2):
    p = [Fraction(0)] * 32
    for d in range(len(x1)):
        t1, t2 = e32.to_frac(x1[d]), e32.to_frac(x2[d])
        nd = e32.sub(t1, t2)
        prod = e32.mul(nd, e32.add(t1, t2))
        p[d % 32] = e32.add(p[d % 32], e32.mul(prod, Fraction(1, 2)))
    return e32.as_f32(_emulate_butterfly(p))


@pytest.mark.parametrize("D", [2, 32, 45, 100])
def test_hyperplane(orc, rng, D):
    for _ in range(10):
        x1 = rng.random(D, dtype=np.float32)
        x2 = rng.random(D, dtype=np.float32)
        n, b = orc.hyperplane(x1, x2)
        assert np.array_equal(n, x1 - x2)
        closed = 0.5 * (np.dot(x1.astype(np.float64), x1.astype(np.float64)) - np.dot(x2.astype(np.float64), x2.astype(np.float64)))
        assert abs(float(b) - closed) <= 1e-5 * max(abs(closed), 1.0)
        assert b == _emulate_hyperplane_offset(x1, x2)
        # p1 is on the left (not "right"), p2 on the right
        assert not (orc.dot32(n, x1) < b)
        assert orc.dot32(n, x2) < b


def test_side_is_the_perpendicular_bisector(orc, rng):
    D = 24
    x1 = rng.random(D, dtype=np.float32)
    x2 = rng.random(D, dtype=np.float32)
    n, b = orc.hyperplane(x1, x2)
    checked = 0
    for _ in range(400):
        x = rng.random(D, dtype=np.float32)
        d1 = orc.sqdist_f64(x, x1)
        d2 = orc.sqdist_f64(x, x2)
        if abs(d1 - d2) < 1e-4:      # too close to the plane for a fp32 statement
            continue
        assert (orc.dot32(n, x) < b) == (d2 < d1)
        checked += 1
    assert checked > 300


def test_rng_helpers(orc):
    k = orc.root_key(0)
    assert k != orc.root_key(1)
    assert orc.child_key(k, 0) != orc.child_key(k, 1)
    assert orc.root_key(-1) != orc.root_key(2 ** 31 - 1)
    # draws are reproducible and spread over the range
    vals = [orc.draw(k, i) % 10 for i in range(2000)]
    hist = np.bincount(vals, minlength=10)
    assert hist.min() > 140 and hist.max() < 260
    assert orc.draw(k, 5) == orc.draw(k, 5)
    # the pair is distinct whenever it can be, and always in range
    for count in [1, 2, 3, 10, 1000]:
        for s in range(50):
            r1, r2 = orc.pick_pair(orc.root_key(s), count)
            assert 0 <= r1 < count and 0 <= r2 < count
            assert (r1 != r2) == (count >= 2)
