"""Pins the oracle's bucket K-NN, exploration and forest against brute force,
set invariants and pure-Python restatements."""
import numpy as np
import pytest

import pyref
from util import assert_knn_equal, compare_knn, exact_knn_numpy, recall, rows_have_no_duplicates, sort_rows


@pytest.mark.parametrize("N,D,K", [(60, 3, 5), (200, 8, 16), (150, 33, 32), (120, 5, 90), (40, 2, 1)])
def test_one_bucket_with_all_points_is_exact_knn(orc, rng, N, D, K):
    """The special case that reduces to textbook brute force."""
    X = rng.random((N, D), dtype=np.float32)
    idx, dist = orc.init_lists(N, K)
    orc.bucket_knn(X, K, np.arange(N, dtype=np.int32), np.array([N], np.int32), idx, dist,
                   starts=np.array([0], np.int32))
    ti, td = exact_knn_numpy(X, K)
    bi, bd = orc.bruteforce(X, K)
    # the oracle's own brute force agrees with numpy's
    assert np.array_equal(np.sort(bi, 1), np.sort(ti, 1))
    assert np.allclose(bd, td, rtol=1e-9, atol=1e-12)
    keep = min(K, N)
    si, sd = sort_rows(idx, dist)
    assert np.array_equal(np.sort(si[:, :keep], 1), np.sort(ti[:, :keep], 1))
    assert np.allclose(sd[:, :keep], td[:, :keep], rtol=1e-5, atol=1e-7)
    if K > N:
        assert (si[:, N:] == -1).all() and np.isinf(sd[:, N:]).all()


@pytest.mark.parametrize("N,D,K,MIN,MAX", [(300, 4, 4, 5, 12), (500, 16, 8, 9, 18), (400, 7, 16, 17, 60)])
def test_bucket_knn_matches_python_restatement(orc, rng, N, D, K, MIN, MAX):
    X = rng.random((N, D), dtype=np.float32)
    idx, dist = orc.init_lists(N, K)
    pi, pd = idx.copy(), dist.copy()
    for seed in range(3):
        perm, ls, lz, _ = orc.build_tree(X, MIN, MAX, 5000, seed)
        orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
        pi, pd = pyref.bucket_knn(orc, X, K, [list(perm[s:s + z]) for s, z in zip(ls, lz)], pi, pd)
        assert_knn_equal(idx, dist, pi, pd)


def test_bucket_knn_invariants(orc, rng):
    N, D, K = 3000, 12, 10
    X = rng.random((N, D), dtype=np.float32)
    idx, dist = orc.init_lists(N, K)
    prev_max = dist.max(1).copy()
    for seed in range(6):
        perm, ls, lz, _ = orc.build_tree(X, K + 1, 2 * (K + 1), 5000, seed)
        orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
        assert rows_have_no_duplicates(idx)
        now_max = dist.max(1)
        assert (now_max <= prev_max).all()            # the row maximum never increases
        prev_max = now_max.copy()
        # idempotence: the same buckets again change nothing
        i2, d2 = idx.copy(), dist.copy()
        orc.bucket_knn(X, K, perm, lz, i2, d2, starts=ls)
        assert np.array_equal(i2, idx) and np.array_equal(d2, dist)
    assert (idx >= 0).all()                            # MIN = K+1 fills every row
    # stored distance == recomputed distance, self in slot 0
    for p in rng.choice(N, 100, replace=False):
        for k in range(K):
            assert dist[p, k] == orc.sqdist(X[p], X[idx[p, k]])
    assert (idx[:, 0] == np.arange(N)).all() and (dist[:, 0] == 0).all()


def test_padded_bucket_matrix_form(orc, rng):
    """stride form (bucket b = ids[b*stride : b*stride+size]) == offsets form."""
    N, D, K = 800, 6, 8
    X = rng.random((N, D), dtype=np.float32)
    perm, ls, lz, _ = orc.build_tree(X, 9, 30, 5000, 2)
    mc = int(lz.max())
    padded = np.full((len(lz), mc), -1, np.int32)
    for b, (s, z) in enumerate(zip(ls, lz)):
        padded[b, :z] = perm[s:s + z]
    i1, d1 = orc.init_lists(N, K)
    i2, d2 = orc.init_lists(N, K)
    orc.bucket_knn(X, K, perm, lz, i1, d1, starts=ls)
    orc.bucket_knn(X, K, padded.ravel(), lz, i2, d2, starts=None, stride=mc)
    assert np.array_equal(i1, i2) and np.array_equal(d1, d2)


@pytest.mark.parametrize("N,D,K", [(120, 3, 4), (250, 6, 8)])
def test_explore_matches_python_restatement(orc, rng, N, D, K):
    X = rng.random((N, D), dtype=np.float32)
    idx, dist = orc.forest(X, K, 2, nnef=0, seed=5)
    pi, pd = pyref.explore(orc, X, K, idx, dist)
    orc.explore(X, K, idx, dist)
    assert_knn_equal(idx, dist, pi, pd)


@pytest.mark.parametrize("N,D,K,trees,self_in", [(300, 5, 6, 2, True), (500, 9, 12, 1, True), (400, 3, 8, 2, False),
                                                 (350, 2, 10, 1, True)])
def test_explore_is_the_k_smallest_of_row_and_neighbours_of_neighbours(orc, rng, N, D, K, trees, self_in):
    """Set definition, no loop restated: after a pass the row of p holds the K smallest (distance, index) pairs of
    its old row joined with the rows (of the snapshot) of its old neighbours, p itself left out of what is offered.
    Distances come from an independent float64 evaluation rounded through the same fp32 chain (orc.sqdist is pinned
    by test_oracle_math.py); integer lattice points (the D = 2 case) make ties at the K-th distance common."""
    if D == 2:
        X = rng.integers(0, 7, size=(N, D)).astype(np.float32)
    else:
        X = rng.random((N, D), dtype=np.float32)
    idx, dist = orc.init_lists(N, K, self_in=self_in)
    for seed in range(trees):
        perm, ls, lz, _ = orc.build_tree(X, 4, 11, 5000, seed)      # small buckets: some rows stay partly empty
        orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
    old_i, old_d = idx.copy(), dist.copy()
    orc.explore(X, K, idx, dist)
    si, sd = sort_rows(idx, dist)
    for p in range(N):
        mine = {int(c): float(d) for c, d in zip(old_i[p], old_d[p]) if c >= 0}
        offered = set()
        for q in old_i[p]:
            if q >= 0:
                offered.update(int(c) for c in old_i[q] if c >= 0)
        offered.discard(p)
        for c in offered - set(mine):
            mine[c] = float(orc.sqdist(X[p], X[c]))
        want = sorted((d, c) for c, d in mine.items())[:K]
        got = [(float(d), int(c)) for d, c in zip(sd[p], si[p]) if c >= 0]
        assert got == want, "row %d" % p
        assert (si[p, len(want):] == -1).all()


def test_explore_with_empty_slots_and_without_self(orc, rng):
    """-1 neighbours are skipped (the reference reads out of range there) and a
    point is never offered to itself."""
    N, D, K = 200, 4, 12
    X = rng.random((N, D), dtype=np.float32)
    idx, dist = orc.init_lists(N, K, self_in=False)
    perm, ls, lz, _ = orc.build_tree(X, 4, 9, 5000, 0)       # buckets smaller than K+1: rows stay partly empty
    orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
    assert (idx < 0).any()
    pi, pd = pyref.explore(orc, X, K, idx, dist)
    orc.explore(X, K, idx, dist)
    assert_knn_equal(idx, dist, pi, pd)
    assert not (idx == np.arange(N)[:, None]).any()
    assert rows_have_no_duplicates(idx)


def test_explore_improves_recall_and_keeps_invariants(orc, rng):
    N, D, K = 4000, 8, 10
    X = rng.random((N, D), dtype=np.float32)
    ti, _ = orc.bruteforce(X, K)
    idx, dist = orc.forest(X, K, 3, nnef=0)
    r0 = recall(ti, idx)
    before = dist.max(1).copy()
    orc.explore(X, K, idx, dist)
    r1 = recall(ti, idx)
    assert r1 >= r0 and r1 > 0.5
    assert (dist.max(1) <= before).all()
    assert rows_have_no_duplicates(idx)
    for p in rng.choice(N, 50, replace=False):
        for k in range(K):
            assert dist[p, k] == orc.sqdist(X[p], X[idx[p, k]])


def test_forest_small_plumbing_config(orc):
    """BASELINE config 1: N=10,000, D=32, U[0,1), K=16, 4 trees, buckets 32/128,
    random_state 0, one exploration pass -- on the CPU path, against exact K-NN."""
    X = np.random.default_rng(0).random((10000, 32), dtype=np.float32)
    idx, dist, log = orc.forest(X, 16, 4, 32, 128, 5000, 0, 1, want_log=True)
    assert (idx >= 0).all() and rows_have_no_duplicates(idx)
    ti, _ = orc.bruteforce(X, 16)
    r = recall(ti, idx)
    assert 0.35 < r < 0.6          # measured 0.4469 with this seed
    # log layout: 16 series of n_trees values, then two scalars
    assert log.shape == (16 * 4 + 2,)
    depth, maxleaf, minleaf, leaves = log[0:4], log[4:8], log[8:12], log[12:16]
    assert (depth >= 7).all() and (maxleaf <= 128).all() and (minleaf >= 32).all()
    assert (leaves >= 10000 / 128).all() and (leaves <= 10000 / 32).all()
    # more trees can only help
    idx8, _ = orc.forest(X, 16, 8, 32, 128, 5000, 0, 1)
    assert recall(ti, idx8) > r


def test_forest_is_trees_then_explore(orc, rng):
    """The forest call equals the stage calls chained by hand with seeds seed+t."""
    N, D, K, T = 1500, 5, 6, 3
    X = rng.random((N, D), dtype=np.float32)
    fi, fd = orc.forest(X, K, T, 7, 14, 5000, 40, 2)
    idx, dist = orc.init_lists(N, K)
    for t in range(T):
        perm, ls, lz, _ = orc.build_tree(X, 7, 14, 5000, 40 + t)
        orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
    orc.explore(X, K, idx, dist)
    orc.explore(X, K, idx, dist)
    assert np.array_equal(fi, idx) and np.array_equal(fd, dist)


def test_forest_merges_into_existing_lists(orc, rng):
    """A second call starts from the lists it is given (reference RSFK.py:351-366)."""
    N, D, K = 1200, 6, 8
    X = rng.random((N, D), dtype=np.float32)
    i1, d1 = orc.forest(X, K, 2, seed=0, nnef=0)
    before = d1.max(1).copy()
    i2, d2 = orc.forest(X, K, 2, seed=10, nnef=0, knn_idx=i1.copy(), knn_dist=d1.copy())
    assert (d2.max(1) <= before).all()
    ia, da = orc.forest(X, K, 2, seed=0, nnef=0)
    idx, dist = ia, da
    for t in range(2):
        perm, ls, lz, _ = orc.build_tree(X, K + 1, 2 * (K + 1), 5000, 10 + t)
        orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
    bad_d, bad_i, _ = compare_knn(i2, d2, idx, dist)
    assert bad_d == 0 and bad_i == 0


def test_nan_distances_never_enter_a_row(orc):
    """Points with NaN coordinates: their distance to anything is NaN, which is below no row maximum."""
    rng = np.random.default_rng(5)
    N, D, K = 400, 6, 5
    X = rng.standard_normal((N, D)).astype(np.float32)
    bad = np.arange(0, N, 9)
    X[bad, 2] = np.nan
    idx, dist = orc.init_lists(N, K, self_in=True)
    perm, ls, lz, _ = orc.build_tree(X, K + 1, 2 * K + 2, 5000, 0)
    orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
    orc.explore(X, K, idx, dist)
    assert not np.isnan(dist).any()
    assert (idx[bad, 0] == bad).all() and (idx[bad, 1:] == -1).all()          # their rows keep only themselves
    good = np.setdiff1d(np.arange(N), bad)
    assert not np.isin(idx[good], bad).any()                                  # and nobody holds them


def _grid_points(n_side, D, rng):
    """Integer lattice points in shuffled order: every squared distance is a small integer (exact in fp32 in any
    summation order) and most of them are shared by many pairs."""
    axes = np.meshgrid(*[np.arange(n_side)] * D, indexing="ij")
    X = np.stack([a.ravel() for a in axes], 1).astype(np.float32)
    return X[rng.permutation(X.shape[0])]


@pytest.mark.parametrize("n_side,D,K", [(6, 2, 5), (4, 3, 9), (9, 2, 13)])
def test_ties_keep_the_smaller_index(orc, rng, n_side, D, K):
    """One bucket with all points of a lattice: the row must be the K smallest (distance, index) pairs -- an
    independent statement of the rule (integer arithmetic + lexsort), which a rule that keeps the first arrival, a
    comparison on the distance alone or a reversed index comparison all fail."""
    X = _grid_points(n_side, D, rng)
    N = X.shape[0]
    Xi = X.astype(np.int64)
    d2 = ((Xi[:, None, :] - Xi[None, :, :]) ** 2).sum(-1)
    order = np.lexsort((np.broadcast_to(np.arange(N), d2.shape), d2), axis=1)[:, :K]
    want_i = order.astype(np.int32)
    want_d = np.take_along_axis(d2, order, 1).astype(np.float32)
    idx, dist = orc.init_lists(N, K)
    orc.bucket_knn(X, K, np.arange(N, dtype=np.int32), np.array([N], np.int32), idx, dist, starts=np.array([0], np.int32))
    si, sd = sort_rows(idx, dist)
    assert np.array_equal(si, want_i) and np.array_equal(sd, want_d)


def test_result_does_not_depend_on_arrival_order(orc, rng):
    """Same buckets with their members in another order, and the trees in another order: identical rows,
    on data where almost every distance is tied with others."""
    X = _grid_points(7, 3, rng)                  # 343 points
    N, K = X.shape[0], 10
    trees = [orc.build_tree(X, K + 1, 2 * K + 2, 5000, seed) for seed in range(4)]
    ia, da = orc.init_lists(N, K)
    for perm, ls, lz, _ in trees:
        orc.bucket_knn(X, K, perm, lz, ia, da, starts=ls)
    ib, db = orc.init_lists(N, K)
    for perm, ls, lz, _ in reversed(trees):
        p2 = perm.copy()
        for s, z in zip(ls, lz):
            p2[s:s + z] = p2[s:s + z][rng.permutation(z)]
        orc.bucket_knn(X, K, p2, lz, ib, db, starts=ls)
    sa, sb = sort_rows(ia, da), sort_rows(ib, db)
    assert np.array_equal(sa[0], sb[0]) and np.array_equal(sa[1], sb[1])
    # exploration from the two (equal as sets, differently ordered) states agrees as well
    orc.explore(X, K, ia, da)
    orc.explore(X, K, ib, db)
    sa, sb = sort_rows(ia, da), sort_rows(ib, db)
    assert np.array_equal(sa[0], sb[0]) and np.array_equal(sa[1], sb[1])


def test_infinite_distance_never_enters(orc):
    """Coordinates so large that the squared distance overflows to +inf: such a candidate stays out of an empty
    slot (the reference's `dist >= max` test, compute_knn_from_buckets.cu:1215)."""
    X = np.zeros((6, 2), np.float32)
    X[3:] = 3e19
    idx, dist = orc.init_lists(6, 4)
    orc.bucket_knn(X, 4, np.arange(6, dtype=np.int32), np.array([6], np.int32), idx, dist, starts=np.array([0], np.int32))
    for p in range(6):
        mates = {0, 1, 2} if p < 3 else {3, 4, 5}
        assert set(idx[p][idx[p] >= 0]) == mates
        assert not np.isin(idx[p], list({0, 1, 2, 3, 4, 5} - mates)).any()


def _reference_rule_bucket(orc, X, K, bucket, idx, dist):
    """The reference's own rule, unordered rows and all (compute_knn_from_buckets.cu:1198-1286): every pair i < j of
    the bucket in the order of its diagonals; a candidate enters iff it is strictly below the row's maximum and is
    not in the row, and it overwrites the first slot that holds the maximum."""
    s = len(bucket)
    for diag in range(1, s):
        for i in range(s - diag):
            a, b = bucket[i], bucket[i + diag]
            d = orc.sqdist(X[a], X[b])
            for p, c in ((a, b), (b, a)):
                worst = int(np.argmax(dist[p]))
                if not d < dist[p, worst] or c in idx[p]:
                    continue
                idx[p, worst] = c
                dist[p, worst] = d


def test_rows_equal_those_of_the_reference_rule_where_nothing_ties(orc, rng):
    """The (distance, index) order of the rows differs from the reference's strict first-arrival rule only among
    points tied at a row's K-th distance: on points in general position (no two pair distances of a row equal) the
    rows, as sets, are the ones the reference's unordered replace-the-maximum rule produces."""
    N, D, K = 260, 6, 7
    X = rng.random((N, D), dtype=np.float32)
    idx, dist = orc.init_lists(N, K)
    ri, rd = idx.copy(), dist.copy()
    for seed in range(3):
        perm, ls, lz, _ = orc.build_tree(X, 8, 20, 5000, seed)
        orc.bucket_knn(X, K, perm, lz, idx, dist, starts=ls)
        for s, z in zip(ls, lz):
            _reference_rule_bucket(orc, X, K, [int(p) for p in perm[s:s + z]], ri, rd)
    # general position: no row holds two equal distances (so no tie can have been decided either way)
    sd = np.sort(rd, 1)
    assert (sd[:, 1:] != sd[:, :-1]).all()
    assert_knn_equal(idx, dist, ri, rd)
