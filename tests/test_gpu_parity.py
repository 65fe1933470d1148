"""GPU parity tests: the HIP library, called through its C ABI, against the CPU
oracle on the same seeded inputs.

Bar: the tree partition (integer work) must be identical; K-NN rows, sorted by
(distance, index), must hold bit-identical distances and identical indices, ties
included (library and oracle order a row by (distance, index), so no result
depends on the order in which candidates arrive).
"""
import os

import numpy as np
import pytest

from util import (assert_knn_equal, baseline_points, check_partition, exact_knn_numpy, recall, rows_have_no_duplicates,
                  sort_rows)

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _say(*a):
    print(*a, flush=True)


# ---------------------------------------------------------------------------
# tree build
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("N,D,MIN,MAX,dist", [
    (1, 3, 2, 4, "u"), (5, 2, 2, 4, "u"), (40, 1, 3, 8, "u"), (700, 5, 9, 20, "u"),   # tail phase only
    (1024, 16, 33, 66, "u"), (1025, 16, 33, 66, "u"),                                  # around the wide/tail threshold
    (5000, 32, 33, 66, "u"), (30000, 100, 33, 66, "u"), (60000, 3, 64, 256, "n"),      # wide phase, several levels
    (20000, 33, 17, 34, "n"), (8000, 784, 91, 182, "sparse"),
])
@pytest.mark.parametrize("screen", ["auto", "q8", "bf16", "q8-256"])
def test_tree_partition_is_identical(gpu, orc, rng, monkeypatch, N, D, MIN, MAX, dist, screen):
    """screen: which low-precision copy the side tests are screened on (RSFK_TREE_SCREEN; "auto" chooses from the
    data).  The partition must be the one of the fp32 arithmetic whatever the screen.  "q8-256": the 8-bit screen with
    the subtrees below the wide levels finished by workgroups of 256 threads, as launches over many subtrees have it
    (RSFK_TAIL_BLOCK; the few subtrees of a test otherwise get workgroups of 1024)."""
    if screen == "q8-256":
        monkeypatch.setenv("RSFK_TREE_SCREEN", "q8")
        monkeypatch.setenv("RSFK_TAIL_BLOCK", "256")
    elif screen != "auto":
        monkeypatch.setenv("RSFK_TREE_SCREEN", screen)
    if dist == "u":
        X = rng.random((N, D), dtype=np.float32)
    elif dist == "n":
        X = rng.standard_normal((N, D)).astype(np.float32)
    else:
        X = np.where(rng.random((N, D)) < 0.8, 0.0, 1.0 - rng.random((N, D))).astype(np.float32)
    for seed in (0, 9):
        _say("tree", N, D, MIN, MAX, dist, seed)
        perm, ls, lz, st = orc.build_tree(X, MIN, MAX, 5000, seed)
        gperm, gls, glz, gst = gpu.build_tree(X, MIN, MAX, 5000, seed)
        check_partition(gperm, gls, glz, N)
        assert np.array_equal(gperm, perm)
        assert np.array_equal(gls, ls) and np.array_equal(glz, lz)
        assert list(gst) == [len(ls), st[0], st[1], st[2]]


def test_tree_edge_cases(gpu, orc, rng):
    # identical points: re-drawn until the depth limit, then one forced bucket
    X = np.ones((3000, 4), np.float32)
    _say("tree identical points")
    gperm, gls, glz, gst = gpu.build_tree(X, 5, 10, 30, 0)
    perm, ls, lz, st = orc.build_tree(X, 5, 10, 30, 0)
    assert list(glz) == [3000] == list(lz) and gst[1] == st[0] == 30
    # depth limits
    X = rng.random((5000, 6), dtype=np.float32)
    for depth in (1, 2, 5, 12):
        _say("tree depth limit", depth)
        g = gpu.build_tree(X, 5, 10, depth, 1)
        o = orc.build_tree(X, 5, 10, depth, 1)
        assert np.array_equal(g[0], o[0]) and np.array_equal(g[2], o[2]) and g[3][1] == o[3][0] <= depth
    # duplicated points mixed with distinct ones, N smaller than MIN
    X = np.repeat(rng.random((300, 3), dtype=np.float32), 7, axis=0)
    _say("tree duplicates")
    g = gpu.build_tree(X, 9, 20, 200, 4)
    o = orc.build_tree(X, 9, 20, 200, 4)
    assert np.array_equal(g[0], o[0]) and np.array_equal(g[2], o[2])
    X = rng.random((20, 3), dtype=np.float32)
    g = gpu.build_tree(X, 33, 66, 5000, 0)
    assert list(g[2]) == [20]


# ---------------------------------------------------------------------------
# bucket K-NN on a fixed partition
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("N,D,K,MIN,MAX", [
    (2000, 32, 16, 17, 34), (3000, 100, 32, 33, 66), (3000, 33, 8, 100, 300), (1500, 7, 90, 91, 182),
    (1200, 1, 4, 5, 10), (2500, 3, 1, 2, 4), (2000, 130, 64, 65, 130), (1500, 20, 65, 66, 140),
    (1800, 12, 200, 201, 420), (4000, 256, 32, 33, 66), (1500, 784, 90, 91, 182), (2000, 30, 32, 400, 1024),
    (2500, 10, 300, 301, 620), (4200, 6, 700, 701, 1500), (1600, 40, 1024, 400, 900),
])
@pytest.mark.parametrize("kernel", ["direct", "direct_per_bucket", "direct_per_64", "pairs_in_parts", "gram", "screen"])
def test_bucket_knn_matches_oracle(gpu, orc, rng, monkeypatch, N, D, K, MIN, MAX, kernel):
    """kernel: "direct" = fp32 chains for every pair, the buckets the specialised kernels leave through the pair of
    kernels that evaluates every pair once and hands the distances on through memory; "pairs_in_parts" = the same with
    1 MB of that memory, so that a launch goes in many parts (RSFK_BUCKET_PAIRS_MB=1), and without the kernel that keeps
    a bucket's points in LDS (RSFK_BUCKET_ROWS=0); "direct_per_bucket" / "direct_per_64" = the tiled kernels that need
    no working memory (RSFK_BUCKET_PAIRS=0), a workgroup per bucket or per 64 members of a bucket
    (RSFK_BUCKET_STRIP=0 / 1), also without the kernel for resident buckets; "gram" = the kernel that bounds the pair
    matrix on the matrix cores first and runs the chains only for the pairs that may enter a row (RSFK_GRAM_FROM=0);
    "screen" = the same idea in the two-wavefront kernel for buckets of up to 64 points (RSFK_BUCKET_SCREEN=always;
    other buckets, and K > 64, take the direct kernels)."""
    if kernel in ("direct_per_bucket", "direct_per_64", "pairs_in_parts"):
        if MAX <= 72 and K <= 64:
            pytest.skip("no bucket of this shape reaches the tiled kernels")
        monkeypatch.setenv("RSFK_BUCKET_ROWS", "0")
        if kernel == "pairs_in_parts":
            monkeypatch.setenv("RSFK_BUCKET_PAIRS_MB", "1")
        else:
            monkeypatch.setenv("RSFK_BUCKET_PAIRS", "0")
            monkeypatch.setenv("RSFK_BUCKET_STRIP", "0" if kernel == "direct_per_bucket" else "1")
    if kernel == "gram":
        monkeypatch.setenv("RSFK_GRAM_FROM", "0")
    if kernel == "screen":
        if K > 64 or MIN > 64:
            pytest.skip("no bucket of this shape reaches the screened small-bucket kernel")
        monkeypatch.setenv("RSFK_BUCKET_SCREEN", "always")
    X = rng.random((N, D), dtype=np.float32)
    oi, od = orc.init_lists(N, K)
    gi, gd = orc.init_lists(N, K)
    for seed in (3, 4):
        _say("bucket_knn", N, D, K, MIN, MAX, seed)
        perm, ls, lz, _ = orc.build_tree(X, MIN, MAX, 5000, seed)
        orc.bucket_knn(X, K, perm, lz, oi, od, starts=ls)
        gpu.bucket_knn(X, K, perm, lz, gi, gd, starts=ls)
        assert_knn_equal(gi, gd, oi, od)
        assert rows_have_no_duplicates(gi)


@pytest.mark.parametrize("N,D,K,MIN,MAX", [
    (4000, 32, 32, 64, 256), (3000, 48, 20, 80, 200), (2500, 16, 64, 70, 250), (3000, 64, 8, 65, 128),
    (2600, 32, 5, 30, 256),
])
def test_bucket_knn_resident_rows_matches_oracle(gpu, orc, rng, N, D, K, MIN, MAX):
    """Buckets of 73..256 low-dimensional points go to the kernel that keeps a bucket's points in LDS.  Three trees on
    the same rows of normally distributed points: in the second and third most candidates are above the last slot of
    the row they are offered to, and many of the others are points the row already holds."""
    X = rng.standard_normal((N, D)).astype(np.float32)
    oi, od = orc.init_lists(N, K)
    gi, gd = orc.init_lists(N, K)
    for seed in (3, 4, 5):
        _say("bucket_knn resident rows", N, D, K, MIN, MAX, seed)
        perm, ls, lz, _ = orc.build_tree(X, MIN, MAX, 5000, seed)
        orc.bucket_knn(X, K, perm, lz, oi, od, starts=ls)
        gpu.bucket_knn(X, K, perm, lz, gi, gd, starts=ls)
        assert_knn_equal(gi, gd, oi, od)
        assert rows_have_no_duplicates(gi)


@pytest.mark.parametrize("K", [20, 64])
@pytest.mark.parametrize("data", ["continuous", "grid", "mixed"])
@pytest.mark.parametrize("start", ["self", "empty", "self_far", "other"])
def test_bucket_knn_rows_that_start_new(gpu, orc, rng, start, data, K):
    """A row that holds at most the point itself is filled by counting, for every candidate, the candidates below it;
    two candidates at the same distance send the row to the insertions instead.  Rows start with the point itself,
    empty, with the point itself at a distance that is not 0, or with one other point (then they are not new); the points
    are continuous (no equal distances), on a small grid (nothing but equal distances and duplicates) or both.  Buckets
    of up to 72 points, so that both shapes of the small-bucket kernel run; with K = 64 the first tree does not fill
    the rows and the second finds rows that are neither new nor full."""
    N, D = 3000, 6
    X = rng.random((N, D), dtype=np.float32)
    if data == "grid":
        X = rng.integers(0, 3, (N, D)).astype(np.float32)
    elif data == "mixed":
        some = rng.random(N) < 0.05
        X[some] = rng.integers(0, 2, (int(some.sum()), D)).astype(np.float32)
    oi = np.full((N, K), -1, np.int32)
    od = np.full((N, K), np.inf, np.float32)
    if start in ("self", "self_far"):
        oi[:, 0] = np.arange(N)
        od[:, 0] = 0.0 if start == "self" else 0.3
    elif start == "other":
        # the point's partner in the pairs (0, 1), (2, 3), ... at its distance (a row must not hold a wrong distance:
        # an index could then leave the row and come back with another one, and the result would depend on the order)
        ti, td = orc.init_lists(N, 2)
        orc.bucket_knn(X, 2, np.arange(N, dtype=np.int32), np.full(N // 2, 2, np.int32), ti, td,
                       starts=np.arange(0, N, 2, dtype=np.int32))
        first_is_self = ti[:, 0] == np.arange(N)
        oi[:, 0] = np.where(first_is_self, ti[:, 1], ti[:, 0])
        od[:, 0] = np.where(first_is_self, td[:, 1], td[:, 0])
    gi, gd = oi.copy(), od.copy()
    for seed in (3, 4):
        _say("bucket_knn new rows", start, data, K, seed)
        perm, ls, lz, _ = orc.build_tree(X, 21, 72, 5000, seed)
        orc.bucket_knn(X, K, perm, lz, oi, od, starts=ls)
        gpu.bucket_knn(X, K, perm, lz, gi, gd, starts=ls)
        assert_knn_equal(gi, gd, oi, od)
        assert rows_have_no_duplicates(gi)


def test_bucket_knn_single_bucket_is_exact_knn(gpu, rng):
    """One bucket holding every point: the kernel must return exact K-NN."""
    for N, D, K in [(300, 8, 16), (700, 20, 32)]:
        _say("bucket_knn all-in-one", N, D, K)
        X = rng.random((N, D), dtype=np.float32)
        gi = np.full((N, K), -1, np.int32)
        gd = np.full((N, K), np.inf, np.float32)
        gi[:, 0] = np.arange(N)
        gd[:, 0] = 0
        gpu.bucket_knn(X, K, np.arange(N, dtype=np.int32), np.array([N], np.int32), gi, gd,
                       starts=np.array([0], np.int32))
        ti, td = exact_knn_numpy(X, K)
        si, sd = sort_rows(gi, gd)
        assert np.array_equal(np.sort(si, 1), np.sort(ti, 1))
        assert np.allclose(sd, td, rtol=1e-5, atol=1e-7)          # direct-difference path: 1e-5 relative


def test_bucket_knn_padded_matrix_ragged_and_empty(gpu, orc, rng):
    N, D, K = 1500, 10, 8
    X = rng.random((N, D), dtype=np.float32)
    perm, ls, lz, _ = orc.build_tree(X, 9, 40, 5000, 2)
    mc = int(lz.max())
    # padded matrix with two extra buckets of size 0 and 1 (never produce candidates)
    nb = len(lz) + 2
    padded = np.full((nb, mc), -1, np.int32)
    sizes = np.zeros(nb, np.int32)
    for b, (s, z) in enumerate(zip(ls, lz)):
        padded[b, :z] = perm[s:s + z]
        sizes[b] = z
    padded[nb - 1, 0] = 5
    sizes[nb - 1] = 1
    oi, od = orc.init_lists(N, K)
    gi, gd = orc.init_lists(N, K)
    orc.bucket_knn(X, K, padded.ravel(), sizes, oi, od, starts=None, stride=mc)
    _say("bucket_knn padded")
    gpu.bucket_knn(X, K, padded.ravel(), sizes, gi, gd, starts=None, stride=mc)
    assert_knn_equal(gi, gd, oi, od)
    # FLT_MAX instead of +inf in the empty slots (the reference's CLI initialisation)
    gi2 = np.full((N, K), -1, np.int32)
    gd2 = np.full((N, K), np.finfo(np.float32).max, np.float32)
    oi2, od2 = gi2.copy(), gd2.copy()
    orc.bucket_knn(X, K, perm, lz, oi2, od2, starts=ls)
    gpu.bucket_knn(X, K, perm, lz, gi2, gd2, starts=ls)
    assert_knn_equal(gi2, gd2, oi2, od2)
    # nothing to do
    gpu.bucket_knn(X, K, perm, np.zeros(0, np.int32), gi2, gd2, starts=np.zeros(0, np.int32))
    # bad ids are rejected on the host
    with pytest.raises(gpu.RsfkError):
        gpu.bucket_knn(X, K, np.array([0, 1, N], np.int32), np.array([3], np.int32), gi2, gd2,
                       starts=np.array([0], np.int32))


@pytest.mark.parametrize("memory_mb", [None, "1"])
def test_bucket_knn_padded_matrix_of_large_buckets(gpu, orc, rng, monkeypatch, memory_mb):
    """Buckets handed over as rows of a padded matrix (no table of starts) that reach the pair of kernels which passes
    a bucket's distances through working memory: all at once, and in parts of a few buckets (1 MB of that memory)."""
    if memory_mb:
        monkeypatch.setenv("RSFK_BUCKET_PAIRS_MB", memory_mb)
    N, D, K = 2600, 12, 70
    X = rng.random((N, D), dtype=np.float32)
    perm, ls, lz, _ = orc.build_tree(X, 71, 150, 5000, 8)
    mc = int(lz.max())
    nb = len(lz) + 1
    padded = np.full((nb, mc), -1, np.int32)
    sizes = np.zeros(nb, np.int32)                      # the bucket in the middle of the matrix is empty
    for b, (s, z) in enumerate(zip(ls, lz)):
        row = b if b < nb // 2 else b + 1
        padded[row, :z] = perm[s:s + z]
        sizes[row] = z
    oi, od = orc.init_lists(N, K)
    gi, gd = orc.init_lists(N, K)
    for _ in range(2):                                  # the second call finds rows that are full
        orc.bucket_knn(X, K, padded.ravel(), sizes, oi, od, starts=None, stride=mc)
        _say("bucket_knn padded, large buckets", memory_mb)
        gpu.bucket_knn(X, K, padded.ravel(), sizes, gi, gd, starts=None, stride=mc)
        assert_knn_equal(gi, gd, oi, od)


# ---------------------------------------------------------------------------
# exploration
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("join", ["join", "plain", "staged"])
@pytest.mark.parametrize("N,D,K,self_in", [(3000, 32, 16, True), (2000, 100, 32, True), (1500, 5, 8, False),
                                           (1200, 9, 90, True), (900, 3, 1, True), (2500, 20, 40, True),
                                           (1300, 6, 200, True), (40, 7, 33, True), (5000, 130, 12, True),
                                           (2200, 24, 64, True), (1600, 300, 100, True), (2600, 48, 20, True),
                                           (3000, 200, 32, True), (1100, 6, 300, True), (800, 5, 520, False)])
def test_explore_matches_oracle(gpu, orc, rng, monkeypatch, N, D, K, self_in, join):
    """Both ways of enumerating the candidates: the join over the reversed graph (default; with partly empty
    rows and a large K its marks overflow the small set; K above about 45 then takes the merge kernel that puts a
    whole workgroup on a point, and the general kernel finishes what is left; rows of more than 128 dimensions have
    their candidates taken nearer lower bounds first, several hundred per point at 3000 x 200 with K = 32),
    the same with the reversed graph made by the builder for large graphs (RSFK_REV_STAGED=1: two scatters staged in
    LDS, rows assembled in LDS), and every point for itself (RSFK_EXPLORE_JOIN=0)."""
    if join == "plain":
        monkeypatch.setenv("RSFK_EXPLORE_JOIN", "0")
    if join == "staged":
        if K > 256:
            pytest.skip("rows of more than 256 neighbours never take the join")
        monkeypatch.setenv("RSFK_REV_STAGED", "1")
    X = rng.random((N, D), dtype=np.float32)
    oi, od = orc.init_lists(N, K, self_in=self_in)
    MIN = max(2, K // 2)                 # buckets smaller than K+1 leave some rows partly empty
    for seed in range(2):
        perm, ls, lz, _ = orc.build_tree(X, MIN, 2 * MIN + 3, 5000, seed)
        orc.bucket_knn(X, K, perm, lz, oi, od, starts=ls)
    gi, gd = oi.copy(), od.copy()
    for _ in range(2):
        _say("explore", N, D, K, self_in)
        orc.explore(X, K, oi, od)
        gpu.explore(X, K, gi, gd, 1)
        assert_knn_equal(gi, gd, oi, od)
        assert rows_have_no_duplicates(gi)
    if not self_in:
        assert not (gi == np.arange(N)[:, None]).any()


# ---------------------------------------------------------------------------
# the whole call, through the entry points the Python package binds
# ---------------------------------------------------------------------------
def test_find_nearest_neighbors_small_plumbing_config(gpu, orc):
    """BASELINE config 1 through RSFK.find_nearest_neighbors."""
    import gpu_rsfk
    X = np.random.default_rng(0).random((10000, 32), dtype=np.float32)
    r = gpu_rsfk.RSFK(random_state=0)
    _say("forest C1")
    gi, gd = r.find_nearest_neighbors(X, 16, n_trees=4, min_tree_children=32, max_tree_children=128)
    oi, od, olog = orc.forest(X, 16, 4, 32, 128, 5000, 0, 1, want_log=True)
    assert_knn_equal(gi, gd, oi, od)
    ti, _ = orc.bruteforce(X, 16)
    assert abs(recall(ti, gi) - recall(ti, oi)) < 1e-9 and recall(ti, gi) > 0.35
    log = r.log_forest.data
    assert log["Tree Depth"] == [int(v) for v in olog[0:4]]
    assert log["Max Leaf Size"] == [int(v) for v in olog[4:8]]
    assert log["Min Leaf Size"] == [int(v) for v in olog[8:12]]
    assert log["Total Leaves"] == [int(v) for v in olog[12:16]]
    assert all(t > 0 for t in log["KNN Sets Updates"]) and r._last_search_time > 0
    # the phases that have a counterpart here carry their time: side tests, hyperplanes of the wide levels,
    # scatter (the reference's node update) and the kernel that finishes the small subtrees (its bucket creation)
    for name in ("Check Points Side Time", "Create Nodes Time", "Update Nodes Time", "Bucket Creation Time"):
        assert all(t > 0 for t in log[name]), name
        assert sum(log[name]) < sum(log["Total Tree Building Time"])
    assert (gi >= 0).all()


@pytest.mark.parametrize("N,D,K,T,kw", [
    (20000, 100, 32, 6, {}),
    (5000, 16, 8, 3, dict(min_tree_children=4, max_tree_children=9)),          # second call with K+1 .. 3(K+1)
    (6000, 24, 40, 3, dict(nn_exploring_factor=2)),
    (4000, 12, 10, 2, dict(point_in_self_neigh=False, nn_exploring_factor=0)),
    (9000, 12, 64, 6, dict(nn_exploring_factor=2)),     # rows of 64: the small set of the merge is tried on a sample first
    (4000, 10, 300, 2, dict(nn_exploring_factor=1)),                           # eight slots per lane
    (1400, 8, 520, 2, dict(nn_exploring_factor=1, min_tree_children=200, max_tree_children=500)),   # sixteen
])
@pytest.mark.parametrize("variant", ["default", "bucket_screen"])
def test_find_nearest_neighbors_matches_oracle(gpu, orc, rng, monkeypatch, N, D, K, T, kw, variant):
    import gpu_rsfk
    if variant == "bucket_screen":
        monkeypatch.setenv("RSFK_BUCKET_SCREEN", "100")     # every tree but the first through the screened small-bucket kernel
    X = rng.standard_normal((N, D)).astype(np.float32)
    r = gpu_rsfk.RSFK(random_state=17)
    _say("forest", N, D, K, T, kw)
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=T, **kw)
    mn = kw.get("min_tree_children", K + 1)
    mx = kw.get("max_tree_children", 2 * mn)
    nnef = kw.get("nn_exploring_factor", 1 if K <= 32 else 0)
    oi, od = orc.init_lists(N, K, self_in=kw.get("point_in_self_neigh", True))
    orc.forest(X, K, T, mn, mx, 5000, 17, nnef, knn_idx=oi, knn_dist=od)
    if mn < K + 1:
        orc.forest(X, K, 1, K + 1, 3 * (K + 1), 5000, 17, nnef, knn_idx=oi, knn_dist=od)
    assert_knn_equal(gi, gd, oi, od)


# The workloads of the benchmark configurations 3, 4 and 5 (clustered D=256; sparse D=784 with K=90 and one
# exploration pass, the only shape that runs the general bucket kernel with two slots per lane together with the
# workgroup-per-point exploration merge; standard normal D=32 with buckets of 64..256 points), as forest +
# exploration through the package against the oracle, at sizes the oracle finishes in seconds.
@pytest.mark.parametrize("config,N,K,T,kw", [
    ("c3", 24000, 32, 6, {}),
    ("c4", 9000, 90, 4, dict(nn_exploring_factor=1)),
    ("c5", 70000, 32, 5, dict(min_tree_children=64, max_tree_children=256)),
], ids=["config3_gmm64_d256_k32", "config4_sparse_d784_k90_explore", "config5_normal_d32_buckets64_256"])
@pytest.mark.parametrize("kernel", ["direct", "gram", "screen", "tiled"])
def test_baseline_config_workloads_match_oracle(gpu, orc, monkeypatch, config, N, K, T, kw, kernel):
    import gpu_rsfk
    if kernel == "tiled":
        if config != "c4":
            pytest.skip("no bucket of this configuration reaches the general kernel")
        monkeypatch.setenv("RSFK_BUCKET_PAIRS", "0")       # the forms of the general kernel that need no working memory
    if kernel == "gram":
        monkeypatch.setenv("RSFK_GRAM_FROM", "1")          # every tree but the first through the screened bucket kernel
    if kernel == "screen":
        if config != "c3":
            pytest.skip("no bucket of this configuration reaches the screened small-bucket kernel")
        monkeypatch.setenv("RSFK_BUCKET_SCREEN", "100")
    else:
        monkeypatch.setenv("RSFK_BUCKET_SCREEN", "never")
    X = baseline_points(config, N)
    r = gpu_rsfk.RSFK(random_state=0)
    _say("forest", config, N, X.shape[1], K, T, kw)
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=T, **kw)
    mn = kw.get("min_tree_children", K + 1)
    mx = kw.get("max_tree_children", 2 * mn)
    nnef = kw.get("nn_exploring_factor", 1 if K <= 32 else 0)
    assert nnef == 1
    oi, od, olog = orc.forest(X, K, T, mn, mx, 5000, 0, nnef, want_log=True)
    assert_knn_equal(gi, gd, oi, od)
    assert rows_have_no_duplicates(gi) and (gi >= 0).all()
    log = r.log_forest.data
    assert log["Total Leaves"] == [int(v) for v in olog[3 * T:4 * T]]
    assert log["Max Leaf Size"] == [int(v) for v in olog[1 * T:2 * T]]


# size-independent properties of the same three workloads at their full sizes
@pytest.mark.parametrize("config,N,K,T,mn,mx", [
    ("c3", 1000000, 32, 4, 33, 66),
    ("c4", 70000, 90, 10, 91, 182),
    ("c5", 10000000, 32, 3, 64, 256),
], ids=["config3_full_size", "config4_full_size", "config5_full_size"])
def test_baseline_config_properties_at_full_size(gpu, orc, config, N, K, T, mn, mx):
    import torch
    X = baseline_points(config, N)
    D = X.shape[1]
    dX = torch.from_numpy(X).cuda()
    idx = torch.full((N, K), -1, dtype=torch.int32, device="cuda")
    idx[:, 0] = torch.arange(N, dtype=torch.int32, device="cuda")
    dist = torch.full((N, K), float("inf"), dtype=torch.float32, device="cuda")
    dist[:, 0] = 0
    log = np.zeros(16 * T + 2, np.float32)
    _say("full size forest", config, N, D, K, T)
    gpu.knn_forest_device(T, K, N, D, mn, mx, 5000, 0, 0, 0, dX.data_ptr(), idx.data_ptr(), dist.data_ptr(), log)
    torch.cuda.synchronize()
    assert (log[1 * T:2 * T] <= mx).all() and (log[2 * T:3 * T] >= mn).all()
    assert (log[3 * T:4 * T] >= N / mx).all() and (log[3 * T:4 * T] <= N / mn).all()
    before = dist.max(1).values.clone()
    assert bool((idx >= 0).all()) and bool((idx < N).all())
    assert bool((dist[:, 1:] >= dist[:, :-1]).all())                 # rows come back ascending
    srt = torch.sort(idx, dim=1).values
    assert not bool((srt[:, 1:] == srt[:, :-1]).any())               # no point twice in a row
    del srt
    rng = np.random.default_rng(3)
    rows = rng.choice(N, 150, replace=False)
    hi, hd = idx[torch.from_numpy(rows).cuda()].cpu().numpy(), dist[torch.from_numpy(rows).cuda()].cpu().numpy()
    for r_, p in enumerate(rows):
        for k in range(0, K, 7):
            assert hd[r_, k] == orc.sqdist(X[p], X[hi[r_, k]])       # stored distance = distance of the stored neighbour
    # one exploration pass: the row maximum only falls, and sampled rows are what the oracle's rule gives from the
    # same graph (the K smallest (distance, index) of the old row and the neighbours of the old neighbours)
    old = idx.clone()
    scratch = torch.empty((N, K), dtype=torch.int32, device="cuda")
    _say("full size explore", config)
    gpu.explore_device(dX.data_ptr(), N, D, K, idx.data_ptr(), dist.data_ptr(), scratch.data_ptr())
    torch.cuda.synchronize()
    assert bool((dist.max(1).values <= before).all())
    for p in rows[:40]:
        orow = old[int(p)].cpu().numpy()
        cand = np.unique(np.concatenate([orow, old[torch.from_numpy(orow).long().cuda()].cpu().numpy().ravel()]))
        d = np.array([orc.sqdist(X[c], X[p]) for c in cand], np.float32)
        order = np.lexsort((cand, d))[:K]
        assert np.array_equal(idx[int(p)].cpu().numpy(), cand[order])
        assert np.array_equal(dist[int(p)].cpu().numpy(), d[order])


def test_reference_package_smoke_tests(gpu):
    """The two live smoke tests of the reference package (RSFK.py:841-903)."""
    import gpu_rsfk
    np.random.seed(0)
    _say("package test()")
    gpu_rsfk.test()


def test_cluster_by_sample_tree(gpu, orc, rng):
    import gpu_rsfk
    N, D = 4096, 99
    X = rng.random((N, D), dtype=np.float32)
    r = gpu_rsfk.RSFK(random_state=5)
    _say("cluster_by_sample_tree")
    total_leaves, max_child, nodes_buckets, bucket_sizes = r.cluster_by_sample_tree(
        X, min_tree_children=N // 30, max_tree_children=3 * (N // 30), verbose=0)
    perm, ls, lz, st = orc.build_tree(X, N // 30, 3 * (N // 30), 5000, 5)
    assert total_leaves == len(lz) and max_child == lz.max()
    assert nodes_buckets.shape == (total_leaves * max_child,) and np.array_equal(bucket_sizes, lz)
    nb = nodes_buckets.reshape(total_leaves, max_child)
    for b in range(total_leaves):
        assert np.array_equal(nb[b, :lz[b]], perm[ls[b]:ls[b] + lz[b]])
        assert (nb[b, lz[b]:] == -1).all()
    assert np.array_equal(np.sort(nb[nb >= 0]), np.arange(N))
    raw = r.cluster_by_sample_tree(X, min_tree_children=64, max_tree_children=256, verbose=0, numpy_result_format=False)
    assert raw[0].value > 0 and raw[1].value <= 256


def test_golden_vectors(gpu):
    g = np.load(os.path.join(ROOT, "tests", "golden", "small_knng.npz"))
    N, D, K, MIN, MAX, seed = [int(v) for v in g["params"]]
    X = g["X"]
    _say("golden")
    perm, ls, lz, st = gpu.build_tree(X, MIN, MAX, 5000, seed)
    assert np.array_equal(perm, g["perm"]) and np.array_equal(ls, g["leaf_start"]) and np.array_equal(lz, g["leaf_size"])
    gi = np.full((N, K), -1, np.int32)
    gd = np.full((N, K), np.inf, np.float32)
    gi[:, 0] = np.arange(N)
    gd[:, 0] = 0
    gpu.bucket_knn(X, K, perm, lz, gi, gd, starts=ls)
    assert_knn_equal(gi, gd, g["bucket_idx"], g["bucket_dist"])
    import gpu_rsfk
    fi, fd = gpu_rsfk.RSFK(seed).find_nearest_neighbors(X, K, n_trees=3, min_tree_children=MIN, max_tree_children=MAX)
    assert_knn_equal(fi, fd, g["forest_idx"], g["forest_dist"])
    qi, qd = gpu_rsfk.RSFK(seed).find_nearest_neighbors_ann(X, g["Q"], K, n_trees=3, min_tree_children=MIN,
                                                            max_tree_children=MAX, ensure_valid_indices=False)
    assert_knn_equal(qi, qd, g["ann_idx"], g["ann_dist"])
    indptr, cols, vals = gpu_rsfk.symmetric_knn_graph(g["forest_idx"], g["forest_dist"], drop_self=True)
    assert np.array_equal(indptr, g["csr_indptr"]) and np.array_equal(cols, g["csr_indices"])
    assert np.array_equal(vals, g["csr_data"])


# ---------------------------------------------------------------------------
# size-independent properties at a size the oracle is not run on
# ---------------------------------------------------------------------------
def test_properties_at_scale(gpu, orc):
    import torch
    N, D, K, T = 1000000, 100, 32, 8             # BASELINE config 2 at its full size
    rng = np.random.default_rng(0)
    X = rng.random((N, D), dtype=np.float32)
    dX = torch.from_numpy(X).cuda()
    idx = torch.full((N, K), -1, dtype=torch.int32, device="cuda")
    idx[:, 0] = torch.arange(N, dtype=torch.int32, device="cuda")
    dist = torch.full((N, K), float("inf"), dtype=torch.float32, device="cuda")
    dist[:, 0] = 0
    log = np.zeros(16 * T + 2, np.float32)
    _say("scale forest")
    gpu.knn_forest_device(T, K, N, D, K + 1, 2 * (K + 1), 5000, 0, 0, 0, dX.data_ptr(), idx.data_ptr(), dist.data_ptr(), log)
    torch.cuda.synchronize()
    gi, gd = idx.cpu().numpy(), dist.cpu().numpy()
    assert (gi >= 0).all() and (gi < N).all()
    assert rows_have_no_duplicates(gi)
    leaves = log[3 * T:4 * T]
    assert (log[1 * T:2 * T] <= 2 * (K + 1)).all() and (log[2 * T:3 * T] >= K + 1).all()
    assert (leaves >= N / (2 * (K + 1))).all() and (leaves <= N / (K + 1)).all()
    # stored distances are the distances of the stored neighbours
    rows = rng.choice(N, 300, replace=False)
    for p in rows:
        for k in range(0, K, 5):
            assert gd[p, k] == orc.sqdist(X[p], X[gi[p, k]])
    # one more identical forest cannot change anything (idempotence of the set update)
    before = gd.max(1).copy()
    _say("scale forest again")
    gpu.knn_forest_device(T, K, N, D, K + 1, 2 * (K + 1), 5000, 0, 0, 0, dX.data_ptr(), idx.data_ptr(), dist.data_ptr(), log)
    torch.cuda.synchronize()
    gi2, gd2 = idx.cpu().numpy(), dist.cpu().numpy()
    si, sd = sort_rows(gi, gd)
    si2, sd2 = sort_rows(gi2, gd2)
    assert np.array_equal(sd, sd2) and np.array_equal(si, si2)
    # exploration only lowers the row maximum, and the oracle agrees on a sample of rows
    scratch = torch.empty((N, K), dtype=torch.int32, device="cuda")
    _say("scale explore")
    gpu.explore_device(dX.data_ptr(), N, D, K, idx.data_ptr(), dist.data_ptr(), scratch.data_ptr())
    torch.cuda.synchronize()
    gi3, gd3 = idx.cpu().numpy(), dist.cpu().numpy()
    assert (gd3.max(1) <= before).all()
    assert rows_have_no_duplicates(gi3)
    # the oracle's exploration of a sample of rows, from the same graph: row p after the pass = the K smallest
    # (distance, index) of its old row and the neighbours of its old neighbours
    for p in rng.choice(N, 200, replace=False):
        cand = np.unique(np.concatenate([gi2[p], gi2[gi2[p]].ravel()]))
        cand = cand[cand != p] if p not in gi2[p] else cand
        d = np.array([orc.sqdist(X[c], X[p]) for c in cand], np.float32)
        order = np.lexsort((cand, d))[:K]
        assert np.array_equal(gi3[p], cand[order]) and np.array_equal(gd3[p], d[order])


# ---------------------------------------------------------------------------
# inputs chosen to stress the bfloat16 screens (tree side test, exploration)
# ---------------------------------------------------------------------------
def _hard_inputs(rng, kind, N, D):
    if kind == "offset":          # large common offset: bfloat16 keeps almost nothing of the differences
        return (1000.0 + rng.random((N, D))).astype(np.float32)
    if kind == "grid":            # coarse lattice: many points exactly on bisecting hyperplanes, many equal distances
        return rng.integers(0, 4, size=(N, D)).astype(np.float32)
    if kind == "tiny":            # values near the bottom of the normal range
        return (rng.random((N, D)) * 1e-30).astype(np.float32)
    if kind == "mixed":           # wildly different scales per dimension, both signs
        scale = np.logspace(-6, 6, D).astype(np.float32)
        return (rng.standard_normal((N, D)) * scale).astype(np.float32)
    if kind == "clusters":        # tight clusters: candidate distances crowd around the row maximum
        centres = rng.random((20, D))
        return (centres[rng.integers(20, size=N)] + 1e-3 * rng.standard_normal((N, D))).astype(np.float32)
    raise ValueError(kind)


@pytest.mark.parametrize("variant", ["default", "bucket_screen", "bucket_gram"])
@pytest.mark.parametrize("kind", ["offset", "grid", "tiny", "mixed", "clusters"])
def test_screens_never_change_a_result(gpu, orc, rng, monkeypatch, kind, variant):
    """The bfloat16 screens only skip work whose outcome is certain: trees, bucket K-NN and exploration on inputs
    that defeat a 8-bit mantissa must still be identical to the fp32 oracle.  "bucket_screen" also switches the
    buckets of up to 64 points to the two-wavefront kernel that bounds the pair matrix on the matrix cores
    (RSFK_BUCKET_SCREEN=always: every tree and the stage-level call), "bucket_gram" all buckets to the tiled kernel that
    does the same (RSFK_GRAM_FROM=0)."""
    import gpu_rsfk
    if variant == "bucket_screen":
        monkeypatch.setenv("RSFK_BUCKET_SCREEN", "always")
    if variant == "bucket_gram":
        monkeypatch.setenv("RSFK_GRAM_FROM", "0")
    N, D, K = 6000, 24, 10
    X = _hard_inputs(rng, kind, N, D)
    perm, ls, lz, st = orc.build_tree(X, K + 1, 2 * (K + 1), 300, 2)
    for screen in ("q8", "bf16"):
        _say("hard tree", kind, screen)
        monkeypatch.setenv("RSFK_TREE_SCREEN", screen)
        gperm, gls, glz, gst = gpu.build_tree(X, K + 1, 2 * (K + 1), 300, 2)
        assert np.array_equal(gperm, perm) and np.array_equal(glz, lz)
    monkeypatch.delenv("RSFK_TREE_SCREEN")
    _say("hard forest", kind)
    r = gpu_rsfk.RSFK(random_state=2)
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=3, max_tree_depth=300, nn_exploring_factor=2)
    oi, od = orc.forest(X, K, 3, K + 1, 2 * (K + 1), 300, 2, 2)
    assert_knn_equal(gi, gd, oi, od)          # "grid": equal distances everywhere, ties go to the smaller index
    assert rows_have_no_duplicates(gi)


@pytest.mark.parametrize("K,mn,mx,env,expected", [
    (16, 17, 34, {}, ["k_bucket_knn_auto"]),
    (16, 17, 34, {"RSFK_BUCKET_SCREEN": "never"}, ["k_bucket_knn_auto"]),
    (16, 17, 34, {"RSFK_BUCKET_SCREEN": "always"}, ["k_bucket_knn_auto"]),
    (16, 40, 100, {}, ["k_bucket_knn_auto", "k_bucket_knn_small<72>", "k_bucket_knn_rows"]),
    (90, 91, 182, {}, ["k_bucket_pairs + k_bucket_merge_pairs"]),
    (90, 91, 182, {"RSFK_BUCKET_PAIRS": "0"}, ["k_bucket_knn<per 64 members>"]),
    (90, 91, 182, {"RSFK_BUCKET_PAIRS": "0", "RSFK_BUCKET_STRIP": "0"}, ["k_bucket_knn<per bucket>"]),
    (90, 91, 182, {"RSFK_GRAM_FROM": "1"}, ["k_bucket_pairs + k_bucket_merge_pairs", "k_bucket_knn_gram"]),
])
def test_report_of_a_build_names_what_ran(gpu, rng, monkeypatch, K, mn, mx, env, expected):
    """rsfk_last_build_report: the kernels every tree's buckets went to, the counts the algorithmic bytes are made of
    and the seconds of the three steps, for the build that has just run."""
    import gpu_rsfk
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    N, D, T = 6000, 20, 3
    X = rng.random((N, D), dtype=np.float32)
    r = gpu_rsfk.RSFK(random_state=4)
    _say("report of a build", K, mn, mx, env)
    r.find_nearest_neighbors(X, K, n_trees=T, min_tree_children=mn, max_tree_children=mx, nn_exploring_factor=1)
    rep = gpu.last_build_report()
    assert (rep["N"], rep["D"], rep["K"], rep["n_trees"]) == (N, D, K, T)
    runs = rep["bucket_kernels"]
    assert runs[0][0] == 0 and runs[-1][1] == T - 1
    assert all(runs[i][1] + 1 == runs[i + 1][0] for i in range(len(runs) - 1))
    named = set(name for _, _, names in runs for name in names)
    assert named == set(expected), named
    assert len(rep["bucket_pair_share"]) == T and len(rep["bucket_screened"]) == T
    if "RSFK_BUCKET_SCREEN" in env:                     # the form of the kernel the trees took
        assert rep["bucket_screened"] == [1 if env["RSFK_BUCKET_SCREEN"] == "always" else 0] * T
    assert rep["tree_points_tested"] >= N * T and 0 <= rep["tree_points_undecided"] <= rep["tree_points_tested"]
    assert rep["explore_passes"] == 1 and rep["explore_exact_distances"] > 0
    assert rep["tree_seconds"] > 0 and rep["bucket_seconds"] > 0 and rep["explore_seconds"] > 0


def test_workspace_is_reused_and_can_be_released(gpu, rng):
    """Device buffers are kept between calls; releasing them changes nothing but the next call's allocations."""
    import gpu_rsfk
    from gpu_rsfk import capi
    X = rng.random((5000, 20), dtype=np.float32)
    a = gpu_rsfk.RSFK(random_state=4).find_nearest_neighbors(X, 12, n_trees=3)
    b = gpu_rsfk.RSFK(random_state=4).find_nearest_neighbors(X, 12, n_trees=3)      # served from the kept buffers
    capi.lib().rsfk_release_workspace()
    c = gpu_rsfk.RSFK(random_state=4).find_nearest_neighbors(X, 12, n_trees=3)
    for r in (b, c):
        assert_knn_equal(r[0], r[1], a[0], a[1])


def test_rows_come_back_sorted_and_unsorted_input_is_accepted(gpu, orc, rng):
    """Rows handed in unsorted (the reference keeps them unordered) are merged correctly; rows come back ascending."""
    N, D, K = 3000, 12, 16
    X = rng.random((N, D), dtype=np.float32)
    oi, od = orc.forest(X, K, 2, nnef=0, seed=3)              # oracle rows are in arrival order (unsorted)
    assert (np.diff(od, axis=1) < 0).any()
    gi, gd = oi.copy(), od.copy()
    perm, ls, lz, _ = orc.build_tree(X, K + 1, 2 * (K + 1), 5000, 77)
    orc.bucket_knn(X, K, perm, lz, oi, od, starts=ls)
    _say("unsorted rows in")
    gpu.bucket_knn(X, K, perm, lz, gi, gd, starts=ls)
    assert_knn_equal(gi, gd, oi, od)
    changed = (np.sort(gi, 1) != np.sort(oi.copy(), 1)).any(1)     # rows identical as sets
    assert not changed.any()
    gi2, gd2 = gi.copy(), gd.copy()
    gpu.explore(X, K, gi2, gd2, 1)
    assert (np.diff(gd2, axis=1) >= 0).all()                       # every row ascending after a full pass


# ---------------------------------------------------------------------------
# query-set search
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("N,NQ,D,MIN,MAX,dist", [
    (6000, 2500, 24, 9, 18, "normal"),
    (5000, 1, 130, 33, 66, "normal"),
    (3000, 777, 3, 5, 11, "grid"),           # many points on a hyperplane and duplicated points
    (20000, 4000, 64, 33, 66, "uniform"),
])
def test_queries_reach_the_leaf_the_oracle_routes_them_to(gpu, orc, rng, N, NQ, D, MIN, MAX, dist):
    """One tree and a row longer than any bucket: the row of a query is then exactly the bucket it was routed to."""
    import gpu_rsfk
    if dist == "grid":
        X = rng.integers(0, 6, (N, D)).astype(np.float32)
        Q = rng.integers(0, 6, (NQ, D)).astype(np.float32)
    elif dist == "uniform":
        X = rng.random((N, D), dtype=np.float32)
        Q = X[rng.permutation(N)[:NQ]].copy()           # queries that are base points: always on their own side
        Q[::2] += rng.standard_normal((len(Q[::2]), D)).astype(np.float32) * 0.01
    else:
        X = rng.standard_normal((N, D)).astype(np.float32)
        Q = rng.standard_normal((NQ, D)).astype(np.float32)
    perm, qs, qz = orc.route_queries(X, Q, MIN, MAX, 5000, 5)
    K = max(MAX, int(qz.max()))              # identical points cannot be split: such buckets stay above MAX
    assert (qz >= 1).all() and K <= 256
    r = gpu_rsfk.RSFK(random_state=5)
    _say("route", N, NQ, D, MIN, MAX, dist, K)
    gi, gd = r.find_nearest_neighbors_ann(X, Q, K, n_trees=1, min_tree_children=MIN, max_tree_children=MAX,
                                          ensure_valid_indices=False)
    for q in range(NQ):
        want = np.sort(perm[qs[q]:qs[q] + qz[q]])
        got = np.sort(gi[q][gi[q] >= 0])
        assert np.array_equal(got, want), (q, got, want)
    fin = gi >= 0
    assert np.isinf(gd[~fin]).all()
    d64 = ((X[gi[fin]].astype(np.float64) - np.repeat(Q, fin.sum(1), axis=0)) ** 2).sum(1)
    assert np.allclose(gd[fin], d64, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("N,NQ,D,K,T,kw", [
    (20000, 3000, 100, 32, 5, {}),
    (8000, 1500, 18, 8, 3, dict(min_tree_children=4, max_tree_children=9)),    # second call with K+1 .. 3(K+1)
    (9000, 500, 50, 100, 3, {}),
    (7000, 2000, 33, 200, 2, dict(min_tree_children=40, max_tree_children=90, ensure_valid_indices=False)),
    (300, 50, 7, 5, 4, {}),
    (6000, 800, 12, 300, 2, {}),
    (5000, 300, 9, 700, 2, {}),
])
def test_find_nearest_neighbors_ann_matches_oracle(gpu, orc, rng, N, NQ, D, K, T, kw):
    import gpu_rsfk
    X = rng.standard_normal((N, D)).astype(np.float32)
    Q = rng.standard_normal((NQ, D)).astype(np.float32)
    r = gpu_rsfk.RSFK(random_state=23)
    _say("ann", N, NQ, D, K, T, kw)
    gi, gd = r.find_nearest_neighbors_ann(X, Q, K, n_trees=T, **kw)
    mn = kw.get("min_tree_children", K + 1)
    mx = kw.get("max_tree_children", 2 * mn)
    oi, od = orc.ann_forest(X, Q, K, T, mn, mx, 5000, 23)
    if kw.get("ensure_valid_indices", True) and mn < K + 1:
        orc.ann_forest(X, Q, K, 1, K + 1, 3 * (K + 1), 5000, 23, q_idx=oi, q_dist=od)
    assert gi.shape == (NQ, K) and gi.dtype == np.int32 and gd.dtype == np.float32
    assert_knn_equal(gi, gd, oi, od)
    assert rows_have_no_duplicates(gi)
    assert r._last_search_time > 0


def test_ann_device_entry_point_merges_into_given_rows(gpu, capi, orc, rng):
    """Device-resident call, twice with different seeds on the same rows == the oracle doing the same."""
    import torch
    N, NQ, D, K = 12000, 2048, 40, 16
    X = rng.standard_normal((N, D)).astype(np.float32)
    Q = rng.standard_normal((NQ, D)).astype(np.float32)
    dX, dQ = torch.from_numpy(X).cuda(), torch.from_numpy(Q).cuda()
    idx = torch.full((NQ, K), -1, dtype=torch.int32, device="cuda")
    dist = torch.full((NQ, K), float("inf"), dtype=torch.float32, device="cuda")
    log = np.zeros(16 * 3 + 2, np.float32)
    _say("ann device", N, NQ, D, K)
    capi.knn_ann_device(3, K, N, NQ, D, K + 1, 2 * K + 2, 5000, 0, 7, dX.data_ptr(), dQ.data_ptr(),
                        idx.data_ptr(), dist.data_ptr(), log)
    capi.knn_ann_device(2, K, N, NQ, D, K + 1, 2 * K + 2, 5000, 0, 100, dX.data_ptr(), dQ.data_ptr(),
                        idx.data_ptr(), dist.data_ptr())
    torch.cuda.synchronize()
    oi, od = orc.ann_forest(X, Q, K, 3, K + 1, 2 * K + 2, 5000, 7)
    orc.ann_forest(X, Q, K, 2, K + 1, 2 * K + 2, 5000, 100, q_idx=oi, q_dist=od)
    assert_knn_equal(idx.cpu().numpy(), dist.cpu().numpy(), oi, od)
    assert (log[9:12] > 0).all() and log[48] > 0          # Total Leaves per tree, total seconds
    # the recorded index must not change the partition a plain tree build gives
    perm, ls, lz, st = capi.build_tree(X, K + 1, 2 * K + 2, 5000, 7)
    operm, ostarts, osizes, ost = orc.build_tree(X, K + 1, 2 * K + 2, 5000, 7)
    assert np.array_equal(perm, operm) and np.array_equal(lz, osizes) and int(log[9]) == len(osizes)
    # no queries: nothing to do, nothing touched
    capi.knn_ann_device(2, K, N, 0, D, K + 1, 2 * K + 2, 5000, 0, 1, dX.data_ptr(), dQ.data_ptr(),
                        idx.data_ptr(), dist.data_ptr())


def test_ann_recall_rises_with_the_number_of_trees(gpu, rng):
    import gpu_rsfk
    N, NQ, D, K = 30000, 2000, 16, 10
    X = rng.random((N, D), dtype=np.float32)
    Q = rng.random((NQ, D), dtype=np.float32)
    d2 = (Q ** 2).sum(1)[:, None] - 2.0 * Q @ X.T + (X ** 2).sum(1)[None, :]
    true = np.argsort(d2, axis=1)[:, :K]
    r = gpu_rsfk.RSFK(random_state=1)
    rec = []
    for T in (1, 8, 40):
        gi, _ = r.find_nearest_neighbors_ann(X, Q, K, n_trees=T)
        rec.append(np.mean([len(set(gi[q]) & set(true[q])) / K for q in range(NQ)]))
    _say("ann recall", rec)
    assert rec[0] < rec[1] < rec[2] and rec[2] > 0.5


# ---------------------------------------------------------------------------
# symmetrised graph export
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("N,K,drop_self", [(5000, 16, True), (3000, 100, False), (2000, 200, True), (1, 3, False),
                                           (700, 1, True), (900, 300, True), (700, 1000, False)])
def test_symmetric_graph_matches_oracle(gpu, orc, rng, N, K, drop_self):
    import gpu_rsfk
    idx = np.stack([rng.permutation(max(N, K + 1))[:K] for _ in range(N)]).astype(np.int32)
    idx[idx >= N] = -1                                           # only when N <= K: empty slots
    idx[:, 0] = np.arange(N)                                     # the point itself first, as the forest stores it
    for p in range(N):
        dup = np.flatnonzero(idx[p, 1:] == p) + 1
        idx[p, dup] = -1
    idx[rng.random((N, K)) < 0.02] = -1
    val = rng.random((N, K)).astype(np.float32)
    _say("symmetrize", N, K, drop_self)
    gp, gc, gv = gpu_rsfk.symmetric_knn_graph(idx, val, drop_self=drop_self)
    op, oc, ov = orc.symmetrize(idx, val, drop_self=drop_self)
    assert np.array_equal(gp, op) and np.array_equal(gc, oc)
    assert np.array_equal(gv, ov)          # a stored edge keeps its own value, an added one the value of its source
    gp2, gc2, gv2 = gpu_rsfk.symmetric_knn_graph(idx, None, drop_self=drop_self)
    assert np.array_equal(gp2, op) and np.array_equal(gc2, oc) and (gv2 == 0).all()


def test_symmetric_graph_of_a_built_graph(gpu, capi, orc, rng):
    """On a graph the library built (one distance value per pair) the export equals the oracle's bit for bit; device
    entry point with the two-call protocol (count, then fill)."""
    import torch
    import gpu_rsfk
    N, D, K = 30000, 20, 12
    X = rng.standard_normal((N, D)).astype(np.float32)
    gi, gd = gpu_rsfk.RSFK(random_state=2).find_nearest_neighbors(X, K, n_trees=6)
    op, oc, ov = orc.symmetrize(gi, gd, drop_self=True)
    di, dd = torch.from_numpy(gi).cuda(), torch.from_numpy(gd).cuda()
    indptr = torch.empty(N + 1, dtype=torch.int32, device="cuda")
    _say("symmetrize device", N, K)
    nnz = capi.symmetrize_device(di.data_ptr(), dd.data_ptr(), N, K, True, indptr.data_ptr(), 0, 0, 0)
    assert nnz == len(oc) and N * (K - 1) <= nnz <= 2 * N * (K - 1)
    cols = torch.empty(nnz, dtype=torch.int32, device="cuda")
    vals = torch.empty(nnz, dtype=torch.float32, device="cuda")
    assert capi.symmetrize_device(di.data_ptr(), dd.data_ptr(), N, K, True, indptr.data_ptr(), cols.data_ptr(),
                                  vals.data_ptr(), nnz) == nnz
    torch.cuda.synchronize()
    assert np.array_equal(indptr.cpu().numpy(), op) and np.array_equal(cols.cpu().numpy(), oc)
    assert np.array_equal(vals.cpu().numpy(), ov)
    with pytest.raises(RuntimeError, match="too small"):
        capi.symmetrize_device(di.data_ptr(), dd.data_ptr(), N, K, True, indptr.data_ptr(), cols.data_ptr(),
                               vals.data_ptr(), nnz - 1)
    S = gpu_rsfk.symmetric_knn_graph(gi, gd, as_scipy=True)
    assert S.shape == (N, N) and (abs(S - S.T)).nnz == 0 and S.diagonal().sum() == 0


@pytest.mark.parametrize("self_in", [True, False])
def test_rows_made_on_the_device_equal_uploaded_rows(gpu, rng, self_in):
    """find_nearest_neighbors lets the library make the initial rows; the reference's entry point with the rows
    uploaded must give the same arrays."""
    import gpu_rsfk
    N, D, K, T = 9000, 20, 12, 3
    X = rng.standard_normal((N, D)).astype(np.float32)
    r = gpu_rsfk.RSFK(random_state=4)
    _say("fresh rows", self_in)
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=T, point_in_self_neigh=self_in)
    hi = np.full((N, K), -1, np.int32)
    hd = np.full((N, K), np.inf, np.float32)
    if self_in:
        hi[:, 0] = np.arange(N, dtype=np.int32)
        hd[:, 0] = 0.0
    log = np.zeros(16 * T + 2, np.float32)
    r._lib.pymodule_rsfk_knn(T, K, N, D, K + 1, 2 * K + 2, 5000, 0, 4, 1, X, hi, hd, log)
    assert np.array_equal(gd, hd)
    assert_knn_equal(gi, gd, hi, hd)


@pytest.mark.parametrize("N,D,K", [(1500, 9000, 8), (1200, 20000, 6)])
def test_very_long_rows(gpu, orc, rng, N, D, K):
    """Rows far beyond what the LDS-resident fast paths take: the kernels with smaller working sets take over and the
    lists stay those of the oracle (forest with one exploration pass, and the query-set search)."""
    import gpu_rsfk
    X = rng.standard_normal((N, D)).astype(np.float32)
    r = gpu_rsfk.RSFK(random_state=3)
    _say("long rows", N, D, K)
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=1)
    oi, od = orc.forest(X, K, 1, K + 1, 2 * K + 2, 5000, 3, 1)
    assert_knn_equal(gi, gd, oi, od)
    Q = rng.standard_normal((200, D)).astype(np.float32)
    ai, ad = r.find_nearest_neighbors_ann(X, Q, K, n_trees=1)
    qi, qd = orc.ann_forest(X, Q, K, 1, K + 1, 2 * K + 2, 5000, 3)
    assert_knn_equal(ai, ad, qi, qd)


def test_points_with_nan_coordinates(gpu, orc, rng):
    """A NaN distance is below no row maximum: such points keep only themselves, nobody holds them, and the rest of
    the graph is the oracle's (same trees: a NaN side test sends the point left in both)."""
    import gpu_rsfk
    N, D, K, T = 6000, 10, 8, 3
    X = rng.standard_normal((N, D)).astype(np.float32)
    bad = np.arange(0, N, 7)
    X[bad] = np.nan
    _say("nan rows")
    gi, gd = gpu_rsfk.RSFK(random_state=3).find_nearest_neighbors(X, K, n_trees=T)
    oi, od = orc.init_lists(N, K, self_in=True)
    orc.forest(X, K, T, K + 1, 2 * K + 2, 5000, 3, 1, knn_idx=oi, knn_dist=od)
    assert not np.isnan(gd).any() and not np.isnan(od).any()
    assert (gi[bad, 0] == bad).all() and (gi[bad, 1:] == -1).all()
    assert_knn_equal(gi, gd, oi, od)


@pytest.mark.parametrize("K,D", [(8, 24), (5, 32), (20, 16)])
def test_points_with_nan_coordinates_in_large_buckets(gpu, orc, rng, K, D):
    """The same rule in the kernel that keeps a bucket's points in LDS (buckets of 80..256 low-dimensional points),
    with a third of the points NaN and K small: in the first two trees of a build nearly every candidate of a member
    is below its row's last slot, so the step that drops candidates by a histogram of their distances runs, and it
    must see the candidates with a NaN distance as absent."""
    import gpu_rsfk
    N, T = 9000, 3
    X = rng.standard_normal((N, D)).astype(np.float32)
    bad = np.arange(0, N, 3)
    X[bad, rng.integers(0, D, size=len(bad))] = np.nan
    _say("nan rows, large buckets", K, D)
    gi, gd = gpu_rsfk.RSFK(random_state=5).find_nearest_neighbors(X, K, n_trees=T, min_tree_children=80,
                                                                  max_tree_children=256, nn_exploring_factor=0)
    oi, od = orc.init_lists(N, K, self_in=True)
    orc.forest(X, K, T, 80, 256, 5000, 5, 0, knn_idx=oi, knn_dist=od)
    assert not np.isnan(gd).any() and not np.isnan(od).any()
    assert (gi[bad, 0] == bad).all() and (gi[bad, 1:] == -1).all()
    assert_knn_equal(gi, gd, oi, od)


def test_forest_in_several_batches(gpu, orc, rng, monkeypatch):
    """Trees are built a batch at a time (all at once when memory allows); two per batch must give the same graph,
    for the K-NN graph (buckets of both kinds, so both streams of the bucket step are in use) and the query search."""
    import gpu_rsfk
    monkeypatch.setenv("RSFK_TREE_BATCH", "2")
    N, D, K, T = 30000, 20, 32, 5
    X = rng.standard_normal((N, D)).astype(np.float32)
    Q = rng.standard_normal((2000, D)).astype(np.float32)
    r = gpu_rsfk.RSFK(random_state=9)
    _say("batches")
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=T)
    oi, od = orc.forest(X, K, T, K + 1, 2 * K + 2, 5000, 9, 1)
    assert_knn_equal(gi, gd, oi, od)
    assert r.log_forest.data["Total Leaves"] == [len(orc.build_tree(X, K + 1, 2 * K + 2, 5000, 9 + t)[2]) for t in range(T)]
    ai, ad = r.find_nearest_neighbors_ann(X, Q, K, n_trees=T)
    qi, qd = orc.ann_forest(X, Q, K, T, K + 1, 2 * K + 2, 5000, 9)
    assert_knn_equal(ai, ad, qi, qd)


def _random_case(seed):
    g = np.random.default_rng(1000 + seed)
    N = int(g.choice([37, 150, 700, 1300, 2600, 5200, 9000]))
    D = int(g.choice([1, 2, 3, 7, 16, 31, 32, 33, 64, 65, 100, 129, 257]))
    K = int(g.choice([1, 2, 5, 8, 16, 31, 32, 33, 48, 64, 65, 100]))
    T = int(g.integers(1, 5))
    MIN = int(g.choice([K + 1, max(2, K // 2), K + 7, 2 * K + 3]))
    MAX = int(2 * MIN + g.choice([0, 1, 5, MIN]))
    nnef = int(g.integers(0, 3))
    kind = str(g.choice(["normal", "uniform", "grid", "clusters"]))
    if kind == "normal":
        X = g.standard_normal((N, D))
    elif kind == "uniform":
        X = g.random((N, D)) * 100.0 - 30.0
    elif kind == "grid":
        X = g.integers(0, 4, (N, D)).astype(np.float64)          # many equal distances and duplicated points
    else:
        X = g.standard_normal((8, D))[g.integers(0, 8, N)] * 5.0 + 0.05 * g.standard_normal((N, D))
    return X.astype(np.float32), K, T, MIN, MAX, nnef, kind


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_match_oracle(gpu, orc, seed):
    """Seeded random shapes, bucket limits, numbers of exploration passes and kinds of data: K-NN graph, query-set
    search and graph export against the oracle.  On the grid data almost every distance is tied with others and
    points are duplicated: rows must still be identical, since ties are broken by index everywhere."""
    import gpu_rsfk
    X, K, T, MIN, MAX, nnef, kind = _random_case(seed)
    N, D = X.shape
    _say("random case", seed, N, D, K, T, MIN, MAX, nnef, kind)
    r = gpu_rsfk.RSFK(random_state=seed)
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=T, min_tree_children=MIN, max_tree_children=MAX,
                                      nn_exploring_factor=nnef, ensure_valid_indices=False)
    oi, od = orc.forest(X, K, T, MIN, MAX, 5000, seed, nnef)
    assert_knn_equal(gi, gd, oi, od)
    assert rows_have_no_duplicates(gi)
    Q = X[::3] + np.float32(0.125)
    ai, ad = r.find_nearest_neighbors_ann(X, Q, K, n_trees=T, min_tree_children=MIN, max_tree_children=MAX,
                                          ensure_valid_indices=False)
    qi, qd = orc.ann_forest(X, Q, K, T, MIN, MAX, 5000, seed)
    assert_knn_equal(ai, ad, qi, qd)
    ip, cc, vv = gpu_rsfk.symmetric_knn_graph(gi, gd, drop_self=bool(seed & 1))
    op, oc, ov = orc.symmetrize(gi, gd, drop_self=bool(seed & 1))
    assert np.array_equal(ip, op) and np.array_equal(cc, oc) and np.array_equal(vv, ov)


@pytest.mark.parametrize("N,D,K,nnef", [(1500, 3, 400, 1), (2400, 2, 1024, 0)])
def test_rows_of_many_neighbours_on_tied_data(gpu, orc, N, D, K, nnef):
    """Rows of more than 256 neighbours (eight and sixteen slots per lane) on grid data, where most distances are tied
    and points are duplicated: graph (with an exploration pass in the smaller case), query-set search and graph export."""
    import gpu_rsfk
    g = np.random.default_rng(K)
    X = g.integers(0, 6, (N, D)).astype(np.float32)
    _say("many neighbours, tied data", N, D, K)
    r = gpu_rsfk.RSFK(random_state=5)
    gi, gd = r.find_nearest_neighbors(X, K, n_trees=2, min_tree_children=K // 2, max_tree_children=K + 50,
                                      nn_exploring_factor=nnef, ensure_valid_indices=False)
    oi, od = orc.forest(X, K, 2, K // 2, K + 50, 5000, 5, nnef)
    assert_knn_equal(gi, gd, oi, od)
    assert rows_have_no_duplicates(gi)
    Q = X[::5] + np.float32(0.25)
    ai, ad = r.find_nearest_neighbors_ann(X, Q, K, n_trees=2, min_tree_children=K // 2, max_tree_children=K + 50,
                                          ensure_valid_indices=False)
    qi, qd = orc.ann_forest(X, Q, K, 2, K // 2, K + 50, 5000, 5)
    assert_knn_equal(ai, ad, qi, qd)
    ip, cc, vv = gpu_rsfk.symmetric_knn_graph(gi, gd, drop_self=True)
    op, oc, ov = orc.symmetrize(gi, gd, drop_self=True)
    assert np.array_equal(ip, op) and np.array_equal(cc, oc) and np.array_equal(vv, ov)
