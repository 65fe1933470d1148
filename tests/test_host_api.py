"""CPU-only tests of the host side: the shared library loads and exports every
symbol of include/rsfk.h, the Python layer mirrors the reference's interface
(signatures, defaults, error behaviour, log decoding), and the committed golden
vectors still come out of the oracle.  No compute call is made on the GPU
library here."""
import inspect
import os
import re

import numpy as np
import pytest

from util import sort_rows

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(capi):
    header = open(os.path.join(ROOT, "include", "rsfk.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(pymodule_\w+|rsfk_\w+)\s*\(", header))
    assert declared == set(capi.SYMBOLS), (declared ^ set(capi.SYMBOLS))
    L = capi.lib()
    for name in declared:
        assert getattr(L, name) is not None
    assert isinstance(L.rsfk_device_count(), int)
    assert L.rsfk_last_error() is not None


def test_python_layer_signatures_match_the_reference():
    """Names, order and defaults read off the reference's RSFK.py:209-217 and :541-546."""
    import gpu_rsfk
    sig = inspect.signature(gpu_rsfk.RSFK.find_nearest_neighbors)
    assert list(sig.parameters)[1:] == [
        "points", "num_nearest_neighbors", "n_trees", "max_tree_depth", "verbose", "min_tree_children",
        "max_tree_children", "ensure_valid_indices", "add_bit_random_motion", "random_motion_force",
        "nn_exploring_factor", "point_in_self_neigh"]
    d = {k: v.default for k, v in sig.parameters.items()}
    assert (d["n_trees"], d["max_tree_depth"], d["verbose"], d["min_tree_children"], d["max_tree_children"]) == (-1, 5000, 0, -1, -1)
    assert (d["ensure_valid_indices"], d["add_bit_random_motion"], d["random_motion_force"]) == (True, False, 1.0)
    assert (d["nn_exploring_factor"], d["point_in_self_neigh"]) == (-1, True)
    sig = inspect.signature(gpu_rsfk.RSFK.find_nearest_neighbors_ann)      # reference RSFK.py:371-378
    assert list(sig.parameters)[1:] == [
        "points", "query_points", "num_nearest_neighbors", "n_trees", "max_tree_depth", "verbose",
        "min_tree_children", "max_tree_children", "ensure_valid_indices", "add_bit_random_motion",
        "random_motion_force", "nn_exploring_factor"]
    d = {k: v.default for k, v in sig.parameters.items()}
    assert (d["n_trees"], d["max_tree_depth"], d["verbose"], d["min_tree_children"], d["max_tree_children"]) == (-1, 5000, 0, -1, -1)
    sig = inspect.signature(gpu_rsfk.RSFK.cluster_by_sample_tree)
    assert list(sig.parameters)[1:] == ["points", "max_tree_depth", "verbose", "min_tree_children",
                                        "max_tree_children", "add_bit_random_motion", "random_motion_force",
                                        "numpy_result_format"]
    d = {k: v.default for k, v in sig.parameters.items()}
    assert (d["max_tree_depth"], d["verbose"], d["min_tree_children"], d["max_tree_children"]) == (5000, 1, 32, 128)
    assert d["numpy_result_format"] is True
    assert inspect.signature(gpu_rsfk.RSFK.__init__).parameters["random_state"].default == 0
    assert hasattr(gpu_rsfk, "test")


def test_argument_errors_are_raised_before_the_library_is_called():
    import gpu_rsfk
    r = gpu_rsfk.RSFK(random_state=3.0)
    assert r.random_state == 3 and isinstance(r.random_state, int)
    X = np.zeros((10, 2), np.float32)
    with pytest.raises(Exception, match="max_tree_children must be at least 2\\*min_tree_children"):
        r.find_nearest_neighbors(X, 4, min_tree_children=8, max_tree_children=15)
    with pytest.raises(Exception, match="min_tree_children must be at least 1"):
        r.find_nearest_neighbors(X, 4, min_tree_children=-3)
    with pytest.raises(Exception, match="max_tree_children must be at least 2\\*min_tree_children"):
        r.cluster_by_sample_tree(X, min_tree_children=32, max_tree_children=63)
    with pytest.raises(Exception, match="min_tree_children must be at least 1"):
        r.cluster_by_sample_tree(X, min_tree_children=-1, max_tree_children=10)
    with pytest.raises(Exception, match="max_tree_children must be at least 2\\*min_tree_children"):
        r.find_nearest_neighbors_ann(X, X, 4, min_tree_children=8, max_tree_children=15)


def test_forest_log_decoding():
    from gpu_rsfk import ForestLog
    n = 3
    raw = np.arange(16 * n + 2, dtype=np.float32) + 0.4
    fl = ForestLog(raw)
    assert list(fl.data) == ForestLog.ATTR_NAMES and len(ForestLog.ATTR_NAMES) == 16
    assert fl.data["Tree Depth"] == [0, 1, 2]                      # rounded ints
    assert fl.data["Total Leaves"] == [9, 10, 11]
    assert np.allclose(fl.data["KNN Sets Updates"], raw[45:48])    # floats, series 15
    assert fl.total_forest_time == pytest.approx(48.4) and fl.exploration_time == pytest.approx(49.4)


def test_random_motion_is_small_and_in_place():
    from gpu_rsfk import random_motion
    np.random.seed(0)
    X = np.random.random((200, 3))
    Y = X.copy()
    random_motion(Y, 1.0)
    span = X.max(0) - X.min(0)
    assert (np.abs(Y - X) <= span / 200 + 1e-12).all() and not np.array_equal(X, Y)
    Z = X.copy()
    random_motion(Z, 0.0)
    assert np.array_equal(Z, X)


def test_n_trees_heuristic_closed_form(monkeypatch):
    """n_trees = max(ceil(N*D / (((min+max)/2) * 24913)), 50)  (reference RSFK.py:304-307)."""
    import gpu_rsfk
    seen = {}

    class FakeLib:
        def pymodule_rsfk_knn(self, n_trees, K, N, D, mn, mx, depth, verbose, seed, nnef, *arrays):
            seen.update(n_trees=n_trees, K=K, mn=mn, mx=mx, nnef=nnef, seed=seed, depth=depth)

    r = gpu_rsfk.RSFK(5)
    monkeypatch.setattr(r, "_lib", FakeLib())
    idx, dist = r.find_nearest_neighbors(np.zeros((1000, 10), np.float32), 32)
    assert seen == dict(n_trees=50, K=32, mn=33, mx=66, nnef=1, seed=5, depth=5000)
    assert idx.dtype == np.int32 and dist.dtype == np.float32 and idx.shape == (1000, 32)
    assert (idx[:, 0] == np.arange(1000)).all() and (idx[:, 1:] == -1).all()
    assert (dist[:, 0] == 0).all() and np.isinf(dist[:, 1:]).all()
    r.find_nearest_neighbors(np.zeros((300000, 784), np.float32), 90)
    assert seen["n_trees"] == int(np.ceil(300000 * 784 / (((91 + 182) / 2) * 24913))) == 70 and seen["nnef"] == 0
    # ensure_valid_indices: second call with one tree, min K+1, max 3(K+1), same seed
    calls = []

    class FakeLib2:
        def pymodule_rsfk_knn(self, *a):
            calls.append(a[:10])

    monkeypatch.setattr(r, "_lib", FakeLib2())
    r.find_nearest_neighbors(np.zeros((100, 4), np.float32), 8, n_trees=3, min_tree_children=4, max_tree_children=8,
                             point_in_self_neigh=False)
    assert calls[0][:7] == (3, 8, 100, 4, 4, 8, 5000) and calls[1][:7] == (1, 8, 100, 4, 9, 27, 5000)
    assert calls[0][8] == calls[1][8] == 5
    assert hasattr(r, "_last_search_time") and hasattr(r, "log_forest")


def test_golden_vectors_still_come_out_of_the_oracle(orc):
    g = np.load(os.path.join(ROOT, "tests", "golden", "small_knng.npz"))
    N, D, K, MIN, MAX, seed = [int(v) for v in g["params"]]
    X = g["X"]
    perm, ls, lz, st = orc.build_tree(X, MIN, MAX, 5000, seed)
    assert np.array_equal(perm, g["perm"]) and np.array_equal(ls, g["leaf_start"]) and np.array_equal(lz, g["leaf_size"])
    assert np.array_equal(st, g["tree_stats"])
    bi, bd = orc.init_lists(N, K)
    orc.bucket_knn(X, K, perm, lz, bi, bd, starts=ls)
    bi, bd = sort_rows(bi, bd)
    assert np.array_equal(bi, g["bucket_idx"]) and np.array_equal(bd, g["bucket_dist"])
    fi, fd = sort_rows(*orc.forest(X, K, 3, MIN, MAX, 5000, seed, 1))
    assert np.array_equal(fi, g["forest_idx"]) and np.array_equal(fd, g["forest_dist"])
    qi, qd = sort_rows(*orc.ann_forest(X, g["Q"], K, 3, MIN, MAX, 5000, seed))
    assert np.array_equal(qi, g["ann_idx"]) and np.array_equal(qd, g["ann_dist"])
    indptr, cols, vals = orc.symmetrize(g["forest_idx"], g["forest_dist"], drop_self=True)
    assert np.array_equal(indptr, g["csr_indptr"]) and np.array_equal(cols, g["csr_indices"])
    assert np.array_equal(vals, g["csr_data"])


def test_sizes_the_library_would_refuse_raise_in_python(capi):
    """K above 1024, no rows, negative n_trees: an exception before the call, not exit(1) inside the library."""
    import gpu_rsfk
    r = gpu_rsfk.RSFK(random_state=0)
    X = np.zeros((10, 3), np.float32)
    with pytest.raises(ValueError):
        r.find_nearest_neighbors(X, 1025)
    with pytest.raises(ValueError):
        r.find_nearest_neighbors(X, 0)
    with pytest.raises(ValueError):
        r.find_nearest_neighbors(np.zeros((0, 3), np.float32), 4)
    with pytest.raises(ValueError):
        r.find_nearest_neighbors(X, 4, n_trees=-5)
    with pytest.raises(ValueError):
        r.find_nearest_neighbors_ann(X, np.zeros((4, 2), np.float32), 4)
    with pytest.raises(ValueError):
        r.cluster_by_sample_tree(np.zeros((0, 3), np.float32))
