"""Python interface of the MI355X RSFK library.

Mirrors the public interface of the reference's ``python/gpu_rsfk/RSFK.py``
(class ``RSFK`` with ``find_nearest_neighbors`` and ``cluster_by_sample_tree``,
``ForestLog``, ``random_motion``): same method names, arguments, defaults and
error behaviour, so code written against the reference package runs unchanged.
The work is done by ``librsfk.so`` (hand-written HIP for gfx950) which is loaded
with ctypes from this package's directory, exactly where the reference looks for
it (RSFK.py:112-113 of the reference).  There is no CPU fallback: if the
library is missing, constructing ``RSFK`` raises.
"""
import ctypes
import os
import time

import numpy as np

_LIB_DIR = os.path.dirname(os.path.abspath(__file__))


def random_motion(points, random_motion_force):
    """Jitter every coordinate in place by ``force * U(-r, r)`` with
    ``r = (max - min) / N`` of that dimension (reference RSFK.py:40-66; uses the
    global numpy generator like the reference)."""
    N, D = points.shape
    for d in range(D):
        min_d = np.min(points[:, d])
        max_d = np.max(points[:, d])
        range_uniform = (max_d - min_d) / N
        points[:, d] = points[:, d] + random_motion_force * np.random.uniform(-range_uniform, range_uniform, N)


MAX_NEIGHBORS = 1024     # a K-NN row is held by one wavefront, up to sixteen slots per lane


def _check_sizes(points, K, n_trees=0):
    """The entry points of the reference's interface have no status return (a failure inside the library ends
    the process, as in the reference), so what the library would refuse is refused here, with an exception."""
    if points.ndim != 2 or points.shape[0] < 1 or points.shape[1] < 1:
        raise ValueError("points must be a matrix with at least one row and one column")
    if K is not None and not (1 <= K <= MAX_NEIGHBORS):
        raise ValueError("num_nearest_neighbors = {}: this library supports 1..{} neighbours".format(K, MAX_NEIGHBORS))
    if n_trees < 0:
        raise ValueError("n_trees must not be negative")


class ForestLog(object):
    """Per-tree series decoded from the ``float32[16*n_trees+2]`` log that the
    library fills (names and order: reference RSFK.py:71-88)."""

    ATTR_NAMES = [
        "Tree Depth",
        "Max Leaf Size",
        "Min Leaf Size",
        "Total Leaves",
        "Tree Initialization Time",
        "Total Tree Building Time",
        "Check Active Points Time",
        "Check Points Side Time",
        "Count New Nodes Time",
        "Dynamic Memory Allocation Time",
        "Preprocessing Split Points Time",
        "Create Nodes Time",
        "Update Nodes Time",
        "Bucket Creation Time",
        "End Tree Time",
        "KNN Sets Updates",
    ]
    INT_ATTRS = ["Tree Depth", "Max Leaf Size", "Min Leaf Size", "Total Leaves"]

    def __init__(self, data):
        self.data = {}
        n_trees = int((len(data) - 2) / 16)
        for i, attr in enumerate(self.ATTR_NAMES):
            values = data[i * n_trees:(i + 1) * n_trees]
            if attr in self.INT_ATTRS:
                values = [int(round(v)) for v in values]
            self.data[attr] = values
        # the two trailing scalars (reference rsfk.cu:2172-2173)
        self.total_forest_time = float(data[16 * n_trees]) if len(data) >= 16 * n_trees + 2 else 0.0
        self.exploration_time = float(data[16 * n_trees + 1]) if len(data) >= 16 * n_trees + 2 else 0.0


_f32_2d = np.ctypeslib.ndpointer(np.float32, ndim=2, flags='ALIGNED, CONTIGUOUS')
_i32_2d_w = np.ctypeslib.ndpointer(np.int32, ndim=2, flags='ALIGNED, CONTIGUOUS, WRITEABLE')
_f32_2d_w = np.ctypeslib.ndpointer(np.float32, ndim=2, flags='ALIGNED, CONTIGUOUS, WRITEABLE')
_f32_1d_w = np.ctypeslib.ndpointer(np.float32, ndim=1, flags='ALIGNED, CONTIGUOUS, WRITEABLE')


def load_library():
    """Load ``librsfk.so`` from the package directory and declare the three
    entry points the reference binds (RSFK.py:116-168)."""
    lib = np.ctypeslib.load_library('librsfk', _LIB_DIR)
    lib.pymodule_rsfk_knn.restype = None
    lib.pymodule_rsfk_knn.argtypes = [ctypes.c_int] * 10 + [_f32_2d, _i32_2d_w, _f32_2d_w, _f32_1d_w]
    lib.pymodule_rsfk_knn_ann.restype = None
    lib.pymodule_rsfk_knn_ann.argtypes = [ctypes.c_int] * 11 + [_f32_2d, _f32_2d, _i32_2d_w, _f32_2d_w, _f32_1d_w]
    lib.pymodule_cluster_by_sample_tree.restype = None
    lib.pymodule_cluster_by_sample_tree.argtypes = [ctypes.c_int] * 7 + [
        _f32_2d,
        ctypes.POINTER(ctypes.POINTER(ctypes.c_int)),
        ctypes.POINTER(ctypes.POINTER(ctypes.c_int)),
        ctypes.POINTER(ctypes.c_int),
        ctypes.POINTER(ctypes.c_int),
    ]
    # entry point of this library only: rows that start empty are made on the device instead of being uploaded
    if hasattr(lib, 'rsfk_knn_forest_fresh_host'):
        lib.rsfk_knn_forest_fresh_host.restype = ctypes.c_int
        lib.rsfk_knn_forest_fresh_host.argtypes = [ctypes.c_int] * 11 + [_f32_2d, _i32_2d_w, _f32_2d_w, _f32_1d_w]
        lib.rsfk_last_error.restype = ctypes.c_char_p
    return lib


class RSFK(object):
    def __init__(self, random_state=0):
        """
        Parameters
        ----------
        random_state : int
            Seed of the first tree; tree ``t`` of a forest uses ``random_state + t``.
        """
        self.random_state = int(random_state)
        self._path = _LIB_DIR
        self._lib = load_library()

    def find_nearest_neighbors(self, points, num_nearest_neighbors,
                               n_trees=-1, max_tree_depth=5000,
                               verbose=0, min_tree_children=-1,
                               max_tree_children=-1,
                               ensure_valid_indices=True,
                               add_bit_random_motion=False,
                               random_motion_force=1.0,
                               nn_exploring_factor=-1,
                               point_in_self_neigh=True):
        """Build the K-NN graph of ``points`` (reference RSFK.py:209-369).

        Parameters have the meaning and defaults of the reference:
        ``n_trees=-1`` picks ``max(ceil(N*D / (avg_bucket*24913)), 50)``;
        ``min_tree_children=-1`` means ``K+1``; ``max_tree_children=-1`` means
        ``2*min_tree_children`` and it must be at least that;
        ``nn_exploring_factor=-1`` means 1 pass if ``K <= 32`` else 0;
        ``ensure_valid_indices`` adds one tree with buckets of ``K+1 .. 3(K+1)``
        points when ``min_tree_children < K+1``; ``point_in_self_neigh`` puts the
        point itself (distance 0) in slot 0.

        Returns
        -------
        knn_indices : int32 ndarray (N, K), rows unordered, -1 = empty slot
        knn_squared_dist : float32 ndarray (N, K)
        """
        points = np.require(points, np.float32, ['CONTIGUOUS', 'ALIGNED'])

        max_tree_depth = int(max_tree_depth)
        verbose = int(verbose)
        max_tree_children = int(max_tree_children)
        min_tree_children = int(min_tree_children)
        N = points.shape[0]
        D = points.shape[1]
        K = int(num_nearest_neighbors)
        n_trees = int(n_trees)

        if nn_exploring_factor == -1:
            nn_exploring_factor = 1 if K <= 32 else 0

        if min_tree_children == -1:
            min_tree_children = K + 1
        if min_tree_children < 0:
            raise Exception('min_tree_children = {} \t => min_tree_children must be at least 1'.format(min_tree_children))
        if max_tree_children == -1:
            max_tree_children = 2 * min_tree_children
        if max_tree_children < 2 * min_tree_children:
            raise Exception('min_tree_children = {}, max_tree_children = {} \t => max_tree_children must be at least 2*min_tree_children'.format(min_tree_children, max_tree_children))

        if n_trees == -1:
            avg_bucket_size = (min_tree_children + max_tree_children) / 2
            n_trees = (N * D) / (avg_bucket_size * 24913)
            n_trees = max(np.ceil(n_trees), 50)
            if verbose > 0:
                print("Automatically setting n_trees to {}".format(n_trees))
        n_trees = int(n_trees)
        _check_sizes(points, K, n_trees)

        if add_bit_random_motion:
            random_motion(points, random_motion_force)
        points = np.require(points, np.float32, ['CONTIGUOUS', 'ALIGNED'])

        fresh = hasattr(self._lib, 'rsfk_knn_forest_fresh_host')
        if fresh:
            # the library makes the initial rows (empty, or the point itself in slot 0) on the device
            knn_indices = np.empty((N, K), dtype=np.int32)
            knn_squared_dist = np.empty((N, K), dtype=np.float32)
        else:
            knn_indices = np.full((N, K), -1, dtype=np.int32)
            knn_squared_dist = np.full((N, K), np.inf, dtype=np.float32)
            if point_in_self_neigh:
                knn_indices[:, 0] = np.arange(N, dtype=np.int32)
                knn_squared_dist[:, 0] = 0.0

        t_init = time.time()

        log_forest = np.zeros(n_trees * 16 + 2, dtype=np.float32)
        if fresh:
            rc = self._lib.rsfk_knn_forest_fresh_host(
                n_trees, K, N, D, min_tree_children, max_tree_children, max_tree_depth,
                verbose, self.random_state, int(nn_exploring_factor), int(bool(point_in_self_neigh)),
                points, knn_indices, knn_squared_dist, log_forest)
            if rc != 0:
                raise RuntimeError(self._lib.rsfk_last_error().decode('utf-8', 'replace'))
        else:
            self._lib.pymodule_rsfk_knn(
                n_trees, K, N, D, min_tree_children, max_tree_children, max_tree_depth,
                verbose, self.random_state, int(nn_exploring_factor),
                points, knn_indices, knn_squared_dist, log_forest)
        self.log_forest = ForestLog(log_forest)

        if ensure_valid_indices and min_tree_children < K + 1:
            log_extra = np.zeros(1 * 16 + 2, dtype=np.float32)
            self._lib.pymodule_rsfk_knn(
                1, K, N, D, K + 1, 3 * (K + 1), max_tree_depth,
                verbose, self.random_state, int(nn_exploring_factor),
                points, knn_indices, knn_squared_dist, log_extra)

        self._last_search_time = time.time() - t_init
        return knn_indices, knn_squared_dist

    def find_nearest_neighbors_ann(self, points, query_points, num_nearest_neighbors,
                                   n_trees=-1, max_tree_depth=5000,
                                   verbose=0, min_tree_children=-1,
                                   max_tree_children=-1,
                                   ensure_valid_indices=True,
                                   add_bit_random_motion=False,
                                   random_motion_force=1.0,
                                   nn_exploring_factor=-1):
        """Neighbours of ``query_points`` among ``points`` (reference RSFK.py:371-539).

        Every tree is built on ``points``; a query is routed to one bucket per tree
        and the points of that bucket are merged into its row.  Parameters and
        defaults as in ``find_nearest_neighbors``; ``nn_exploring_factor`` is passed
        on and ignored by the library, as in the reference.

        Returns
        -------
        knn_indices : int32 ndarray (NQ, K), indices into ``points``, -1 = empty slot
        knn_squared_dist : float32 ndarray (NQ, K)
        """
        points = np.require(points, np.float32, ['CONTIGUOUS', 'ALIGNED'])

        max_tree_depth = int(max_tree_depth)
        verbose = int(verbose)
        max_tree_children = int(max_tree_children)
        min_tree_children = int(min_tree_children)
        N = points.shape[0]
        NQ = query_points.shape[0]
        D = points.shape[1]
        K = int(num_nearest_neighbors)
        n_trees = int(n_trees)

        if nn_exploring_factor == -1:
            nn_exploring_factor = 1 if K <= 32 else 0

        if min_tree_children == -1:
            min_tree_children = K + 1
        if min_tree_children < 0:
            raise Exception('min_tree_children = {} \t => min_tree_children must be at least 1'.format(min_tree_children))
        if max_tree_children == -1:
            max_tree_children = 2 * min_tree_children
        if max_tree_children < 2 * min_tree_children:
            raise Exception('min_tree_children = {}, max_tree_children = {} \t => max_tree_children must be at least 2*min_tree_children'.format(min_tree_children, max_tree_children))

        if n_trees == -1:
            avg_bucket_size = (min_tree_children + max_tree_children) / 2
            n_trees = (N * D) / (avg_bucket_size * 24913)
            n_trees = max(np.ceil(n_trees), 50)
            if verbose > 0:
                print("Automatically setting n_trees to {}".format(n_trees))
        n_trees = int(n_trees)
        _check_sizes(points, K, n_trees)
        if query_points.ndim != 2 or query_points.shape[1] != D:
            raise ValueError("query_points must be a matrix with the columns of points")

        if add_bit_random_motion:
            random_motion(points, random_motion_force)
            random_motion(query_points, random_motion_force)
        points = np.require(points, np.float32, ['CONTIGUOUS', 'ALIGNED'])
        query_points = np.require(query_points, np.float32, ['CONTIGUOUS', 'ALIGNED'])

        knn_indices = np.full((NQ, K), -1, dtype=np.int32)
        knn_squared_dist = np.full((NQ, K), np.inf, dtype=np.float32)

        t_init = time.time()

        log_forest = np.zeros(n_trees * 16 + 2, dtype=np.float32)
        self._lib.pymodule_rsfk_knn_ann(
            n_trees, K, N, NQ, D, min_tree_children, max_tree_children, max_tree_depth,
            verbose, self.random_state, int(nn_exploring_factor),
            points, query_points, knn_indices, knn_squared_dist, log_forest)

        if ensure_valid_indices and min_tree_children < K + 1:
            log_extra = np.zeros(1 * 16 + 2, dtype=np.float32)
            self._lib.pymodule_rsfk_knn_ann(
                1, K, N, NQ, D, K + 1, 3 * (K + 1), max_tree_depth,
                verbose, self.random_state, int(nn_exploring_factor),
                points, query_points, knn_indices, knn_squared_dist, log_extra)

        self._last_search_time = time.time() - t_init
        return knn_indices, knn_squared_dist

    def cluster_by_sample_tree(self, points, max_tree_depth=5000,
                               verbose=1, min_tree_children=32,
                               max_tree_children=128,
                               add_bit_random_motion=False,
                               random_motion_force=1.0,
                               numpy_result_format=True):
        """Partition ``points`` with one random-sample tree (reference
        RSFK.py:541-644).

        Returns ``(total_leaves, max_child, nodes_buckets, bucket_sizes)``:
        ``nodes_buckets`` has ``total_leaves*max_child`` entries, bucket ``b`` is
        ``nodes_buckets[b*max_child : b*max_child + bucket_sizes[b]]`` and the rest
        of its row is -1.  With ``numpy_result_format=False`` the raw ctypes
        objects are returned, as in the reference.
        """
        points = np.require(points, np.float32, ['CONTIGUOUS', 'ALIGNED'])

        max_tree_depth = int(max_tree_depth)
        verbose = int(verbose)
        max_tree_children = int(max_tree_children)
        min_tree_children = int(min_tree_children)
        N = points.shape[0]
        D = points.shape[1]
        _check_sizes(points, None)

        if min_tree_children < 0:
            raise Exception('min_tree_children = {} \t => min_tree_children must be at least 1'.format(min_tree_children))
        if max_tree_children < 2 * min_tree_children:
            raise Exception('min_tree_children = {}, max_tree_children = {} \t => max_tree_children must be at least 2*min_tree_children'.format(min_tree_children, max_tree_children))

        if add_bit_random_motion:
            random_motion(points, random_motion_force)

        t_init = time.time()

        nodes_buckets = ctypes.POINTER(ctypes.c_int)()
        bucket_sizes = ctypes.POINTER(ctypes.c_int)()
        total_leaves = ctypes.c_int(0)
        max_child = ctypes.c_int(0)

        self._lib.pymodule_cluster_by_sample_tree(
            N, D, min_tree_children, max_tree_children, max_tree_depth, verbose, self.random_state,
            points,
            ctypes.byref(nodes_buckets), ctypes.byref(bucket_sizes),
            ctypes.byref(total_leaves), ctypes.byref(max_child))

        self._last_cluster_time = time.time() - t_init

        if numpy_result_format:
            total_leaves = int(total_leaves.value)
            max_child = int(max_child.value)
            nodes_buckets = np.ctypeslib.as_array(nodes_buckets, shape=(1, total_leaves * max_child))[0]
            bucket_sizes = np.ctypeslib.as_array(bucket_sizes, shape=(1, total_leaves))[0]

        return total_leaves, max_child, nodes_buckets, bucket_sizes


def _check_knn_graph_build():
    """A small K-NN graph with jittered input and two exploration passes: every slot must be filled
    (the property the reference's first built-in check asserts, RSFK.py:841-862)."""
    rng = np.random.default_rng(0)
    n, dim, k = 3000, 200, 30
    x = rng.random((n, dim))
    knn, _ = RSFK(random_state=0).find_nearest_neighbors(
        x, k, n_trees=10, max_tree_children=128, nn_exploring_factor=2, add_bit_random_motion=True,
        random_motion_force=0.01, verbose=2)
    empty = int((knn < 0).sum())
    if empty:
        raise Exception("%d empty neighbour slots in the K-NN graph" % empty)


def _check_single_tree_partition():
    """One random-sample tree on 4096 points of 99 dimensions: the call returns a partition
    (what the reference's second built-in check runs, RSFK.py:864-903) and it covers every point once."""
    rng = np.random.default_rng(1)
    n, dim = 4096, 99
    x = rng.random((n, dim))
    smallest = n // 30
    print("points: %d, dimensions: %d, bucket sizes: %d..%d" % (n, dim, smallest, 3 * smallest))
    leaves, widest, members, sizes = RSFK(random_state=0).cluster_by_sample_tree(
        x, min_tree_children=smallest, max_tree_children=3 * smallest, verbose=2)
    print("buckets: %d, largest: %d" % (leaves, widest))
    if int(sizes.sum()) != n or not np.array_equal(np.sort(members[members >= 0]), np.arange(n)):
        raise Exception("the buckets do not cover every point exactly once")


def test():
    """The package's built-in smoke run (same entry point as the reference's ``gpu_rsfk.test``)."""
    _check_knn_graph_build()
    _check_single_tree_partition()
