"""The oracle's query-set search (routing of query points through a tree, update of their rows from the leaf they
reach), pinned without the reference: a pure-Python restatement of the routing, the fact that a base point used as
a query must land in its own leaf, and brute force inside the reached leaves."""
import numpy as np
import pytest

import pyref
from util import rows_have_no_duplicates, recall


@pytest.mark.parametrize("N,NQ,D,MIN,MAX", [(300, 40, 3, 5, 12), (500, 60, 8, 9, 20), (64, 30, 2, 2, 4), (200, 25, 1, 4, 8)])
def test_routing_matches_python_restatement(orc, rng, N, NQ, D, MIN, MAX):
    X = rng.random((N, D), dtype=np.float32)
    Q = rng.random((NQ, D), dtype=np.float32)
    for seed in (0, 5):
        perm, qs, qz = orc.route_queries(X, Q, MIN, MAX, 5000, seed)
        want = pyref.route(orc, X, Q, MIN, MAX, 5000, seed)
        for q in range(NQ):
            assert sorted(perm[qs[q]:qs[q] + qz[q]].tolist()) == sorted(want[q])


def test_a_base_point_lands_in_its_own_leaf(orc, rng):
    X = rng.standard_normal((2000, 12)).astype(np.float32)
    perm, ls, lz, _ = orc.build_tree(X, 9, 18, 5000, 3)
    perm2, qs, qz = orc.route_queries(X, X, 9, 18, 5000, 3)
    assert np.array_equal(perm, perm2)
    leaf_of = np.empty(2000, np.int64)
    for s, z in zip(ls, lz):
        leaf_of[perm[s:s + z]] = s
    assert np.array_equal(qs, leaf_of)


def test_rows_are_exact_knn_of_the_reached_leaves(orc, rng):
    N, NQ, D, K = 1500, 200, 6, 5
    X = rng.random((N, D), dtype=np.float32)
    Q = rng.random((NQ, D), dtype=np.float32)
    T, MIN, MAX, seed = 3, 8, 16, 11
    qi, qd = orc.ann_forest(X, Q, K, T, MIN, MAX, 5000, seed)
    assert rows_have_no_duplicates(qi)
    for q in range(0, NQ, 7):
        cand = set()
        for t in range(T):
            perm, qs, qz = orc.route_queries(X, Q, MIN, MAX, 5000, seed + t)
            cand |= set(perm[qs[q]:qs[q] + qz[q]].tolist())
        cand = np.array(sorted(cand))
        d = np.array([orc.sqdist(Q[q], X[c]) for c in cand])
        order = np.lexsort((cand, d))[:K]
        got = np.lexsort((qi[q], qd[q]))
        assert np.array_equal(qd[q][got][:len(order)], d[order])           # same distances ...
        kth = d[order][-1]
        assert all(c in cand[d <= kth] for c in qi[q] if c >= 0)           # ... from candidates within the K-th
        for k in range(K):
            if qi[q, k] >= 0:
                assert qd[q, k] == orc.sqdist(Q[q], X[qi[q, k]])


def test_more_trees_never_hurt_and_reach_good_recall(orc, rng):
    N, NQ, D, K = 4000, 300, 8, 10
    X = rng.random((N, D), dtype=np.float32)
    Q = rng.random((NQ, D), dtype=np.float32)
    d2 = ((Q.astype(np.float64)[:, None, :] - X.astype(np.float64)[None, :, :]) ** 2).sum(2)
    ti = np.argsort(d2, axis=1, kind="stable")[:, :K]
    prev = -1.0
    qi = qd = None
    for T in (1, 4, 16):
        qi, qd = orc.ann_forest(X, Q, K, T, seed=2)
        r = recall(ti, qi)
        assert r >= prev
        prev = r
    assert prev > 0.6
    # chaining calls is the same as one call with the trees of both
    a_i, a_d = orc.ann_forest(X, Q, K, 2, seed=7)
    a_i, a_d = orc.ann_forest(X, Q, K, 3, seed=9, q_idx=a_i, q_dist=a_d)
    b_i, b_d = orc.ann_forest(X, Q, K, 2, seed=7)
    for t in range(3):
        b_i, b_d = orc.ann_forest(X, Q, K, 1, seed=9 + t, q_idx=b_i, q_dist=b_d)
    assert np.array_equal(np.sort(a_d, 1), np.sort(b_d, 1))
