"""Helpers shared by the tests: comparison of K-NN rows, partition
checks and a pure-Python restatement of the list update rule."""
import numpy as np


def sort_rows(idx, dist):
    order = np.lexsort((idx, dist), axis=1)
    return np.take_along_axis(idx, order, 1), np.take_along_axis(dist, order, 1)


def compare_knn(idx_a, dist_a, idx_b, dist_b, rtol=0.0):
    """Rows are compared as sets.  Returns (bad_dist, bad_idx, tie_idx):
    bad_dist = sorted distances that differ (beyond rtol; exact when rtol == 0),
    bad_idx  = index mismatches that are NOT among entries at the row's largest
               (K-th) distance, i.e. real disagreements,
    tie_idx  = index mismatches at the K-th distance (allowed: equal-distance ties).
    """
    ia, da = sort_rows(idx_a, dist_a)
    ib, db = sort_rows(idx_b, dist_b)
    both_inf = np.isinf(da) & np.isinf(db)
    if rtol == 0.0:
        deq = (da == db) | both_inf
    else:
        with np.errstate(invalid="ignore"):
            deq = (np.abs(da - db) <= rtol * np.maximum(np.abs(da), np.abs(db))) | both_inf
    mism = ia != ib
    kth = da[:, -1:]
    if rtol == 0.0:
        at_kth = (da == kth) | (np.isinf(da) & np.isinf(kth))
    else:
        with np.errstate(invalid="ignore"):
            at_kth = (np.abs(da - kth) <= rtol * np.abs(kth)) | (np.isinf(da) & np.isinf(kth))
    return int((~deq).sum()), int((mism & ~at_kth).sum()), int((mism & at_kth).sum())


def assert_knn_equal(idx_a, dist_a, idx_b, dist_b, rtol=0.0):
    """rtol == 0 (the bar for everything the library computes with the direct-difference chain): after sorting
    each row by (distance, index) the two results are identical, ties included -- rows are ordered by
    (distance, index) in the library and in the oracle, so nothing depends on the order of arrival.
    rtol > 0: distances within rtol, index mismatches only among entries at the row's K-th distance."""
    bad_d, bad_i, tie_i = compare_knn(idx_a, dist_a, idx_b, dist_b, rtol)
    assert bad_d == 0, "%d distances differ" % bad_d
    assert bad_i == 0, "%d indices differ away from the K-th distance" % bad_i
    if rtol == 0.0:
        assert tie_i == 0, "%d indices differ among entries tied at the K-th distance" % tie_i


def check_partition(perm, leaf_start, leaf_size, N, min_children=None, max_children=None):
    """Exact cover of 0..N-1 by contiguous leaf segments in ascending order."""
    assert np.array_equal(np.sort(perm), np.arange(N))
    assert leaf_size.sum() == N
    assert leaf_start[0] == 0
    assert np.array_equal(leaf_start[1:], np.cumsum(leaf_size)[:-1])
    if min_children is not None and N >= min_children:
        assert leaf_size.min() >= min_children
    if max_children is not None:
        assert leaf_size.max() <= max_children


def rows_have_no_duplicates(idx):
    s = np.sort(idx, axis=1)
    dup = (s[:, 1:] == s[:, :-1]) & (s[:, 1:] >= 0)
    return not dup.any()


def exact_knn_numpy(X, K):
    """Brute force with float64 Gram distances; ties -> smaller index."""
    Xd = X.astype(np.float64)
    sq = (Xd * Xd).sum(1)
    d2 = sq[:, None] + sq[None, :] - 2.0 * Xd @ Xd.T
    np.maximum(d2, 0.0, out=d2)
    np.fill_diagonal(d2, 0.0)
    order = np.lexsort((np.broadcast_to(np.arange(X.shape[0]), d2.shape), d2), axis=1)[:, :K]
    return order.astype(np.int32), np.take_along_axis(d2, order, 1)


def recall(true_idx, approx_idx):
    hits = 0
    for t, a in zip(true_idx, approx_idx):
        hits += np.intersect1d(t, a).size
    return hits / float(true_idx.shape[0] * true_idx.shape[1])


def baseline_points(config, N, seed=0):
    """The synthetic inputs of the benchmark configurations, at any number of rows:
    c2 uniform [0,1) D=100; c3 mixture of 64 isotropic Gaussians (centres uniform in [0,1]^256, sigma 0.1) D=256;
    c4 80 % exact zeros, the rest uniform in (0,1], D=784; c5 standard normal D=32."""
    rng = np.random.default_rng(seed)
    if config == "c2":
        return rng.random((N, 100), dtype=np.float32)
    if config == "c3":
        centres = rng.random((64, 256), dtype=np.float32)
        comp = rng.integers(64, size=N)
        return (centres[comp] + np.float32(0.1) * rng.standard_normal((N, 256), dtype=np.float32)).astype(np.float32)
    if config == "c4":
        X = np.float32(1.0) - rng.random((N, 784), dtype=np.float32)
        X[rng.random((N, 784), dtype=np.float32) < 0.8] = 0.0
        return X
    if config == "c5":
        return rng.standard_normal((N, 32), dtype=np.float32)
    raise ValueError(config)
