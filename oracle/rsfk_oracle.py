"""ctypes binding of the CPU oracle (``librsfk_oracle.so``).

TEST INFRASTRUCTURE: imported only by the tests, by ``__graft_entry__.smoke``
and by the CPU-baseline leg of ``bench.py``.  The GPU package never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librsfk_oracle.so")

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile the oracle with the Makefile next to this file."""
    src = os.path.join(_HERE, "rsfk_oracle.c")
    stale = os.path.exists(_SO) and os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_SO)
    if force or stale or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "librsfk_oracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        L.rsfk_or_root_key.restype = ctypes.c_uint64
        L.rsfk_or_root_key.argtypes = [ctypes.c_int]
        L.rsfk_or_child_key.restype = ctypes.c_uint64
        L.rsfk_or_child_key.argtypes = [ctypes.c_uint64, ctypes.c_int]
        L.rsfk_or_draw.restype = ctypes.c_uint32
        L.rsfk_or_draw.argtypes = [ctypes.c_uint64, ctypes.c_uint32]
        L.rsfk_or_pick_pair.restype = None
        L.rsfk_or_pick_pair.argtypes = [ctypes.c_uint64, ctypes.c_int,
                                        ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.rsfk_or_sqdist.restype = ctypes.c_float
        L.rsfk_or_sqdist.argtypes = [_f32p, _f32p, ctypes.c_int]
        L.rsfk_or_sqdist_f64.restype = ctypes.c_double
        L.rsfk_or_sqdist_f64.argtypes = [_f32p, _f32p, ctypes.c_int]
        L.rsfk_or_dot32.restype = ctypes.c_float
        L.rsfk_or_dot32.argtypes = [_f32p, _f32p, ctypes.c_int]
        L.rsfk_or_hyperplane.restype = ctypes.c_float
        L.rsfk_or_hyperplane.argtypes = [_f32p, _f32p, ctypes.c_int, _f32p]
        L.rsfk_or_build_tree.restype = ctypes.c_int
        L.rsfk_or_build_tree.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int, _i32p, _i32p, _i32p, ctypes.c_int, _i32p]
        L.rsfk_or_bucket_knn.restype = None
        L.rsfk_or_bucket_knn.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p,
                                         ctypes.c_void_p, _i32p, ctypes.c_int, ctypes.c_int, _i32p, _f32p]
        L.rsfk_or_explore.restype = None
        L.rsfk_or_explore.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p, _f32p]
        L.rsfk_or_forest.restype = ctypes.c_int
        L.rsfk_or_forest.argtypes = [ctypes.c_int] * 9 + [_f32p, _i32p, _f32p, ctypes.c_void_p]
        L.rsfk_or_route_queries.restype = ctypes.c_int
        L.rsfk_or_route_queries.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_int, _f32p, ctypes.c_int, _i32p, _i32p, _i32p]
        L.rsfk_or_ann_forest.restype = ctypes.c_int
        L.rsfk_or_ann_forest.argtypes = [ctypes.c_int] * 9 + [_f32p, _f32p, _i32p, _f32p]
        L.rsfk_or_symmetrize.restype = ctypes.c_longlong
        L.rsfk_or_symmetrize.argtypes = [_i32p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p,
                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_longlong]
        L.rsfk_or_bruteforce.restype = None
        L.rsfk_or_bruteforce.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                         ctypes.c_int, _i32p, _f64p]
        L.rsfk_or_num_threads.restype = ctypes.c_int
        L.rsfk_or_set_num_threads.argtypes = [ctypes.c_int]
        _lib = L
    return _lib


def _pts(points):
    return np.require(points, np.float32, ["C_CONTIGUOUS", "ALIGNED"])


def root_key(seed):
    return int(lib().rsfk_or_root_key(int(seed)))


def child_key(key, side):
    return int(lib().rsfk_or_child_key(ctypes.c_uint64(key), int(side)))


def draw(key, i):
    return int(lib().rsfk_or_draw(ctypes.c_uint64(key), int(i)))


def pick_pair(key, count):
    a, b = ctypes.c_int(), ctypes.c_int()
    lib().rsfk_or_pick_pair(ctypes.c_uint64(key), int(count), ctypes.byref(a), ctypes.byref(b))
    return a.value, b.value


def sqdist(a, b):
    a, b = _pts(a), _pts(b)
    return np.float32(lib().rsfk_or_sqdist(a, b, a.shape[0]))


def sqdist_f64(a, b):
    a, b = _pts(a), _pts(b)
    return float(lib().rsfk_or_sqdist_f64(a, b, a.shape[0]))


def dot32(n, x):
    n, x = _pts(n), _pts(x)
    return np.float32(lib().rsfk_or_dot32(n, x, n.shape[0]))


def hyperplane(x1, x2):
    x1, x2 = _pts(x1), _pts(x2)
    n = np.empty_like(x1)
    b = lib().rsfk_or_hyperplane(x1, x2, x1.shape[0], n)
    return n, np.float32(b)


def build_tree(points, min_children, max_children, max_depth=5000, seed=0):
    """-> perm, leaf_start, leaf_size, stats(levels, max leaf, min leaf)"""
    points = _pts(points)
    N, D = points.shape
    cap = N // max(min_children, 1) + 2
    perm = np.empty(N, np.int32)
    ls = np.empty(cap, np.int32)
    lz = np.empty(cap, np.int32)
    stats = np.zeros(3, np.int32)
    n = lib().rsfk_or_build_tree(points, N, D, int(min_children), int(max_children), int(max_depth),
                                 int(seed), perm, ls, lz, cap, stats)
    if n < 0:
        raise RuntimeError("oracle: leaf capacity exceeded")
    return perm, ls[:n].copy(), lz[:n].copy(), stats


def bucket_knn(points, K, ids, sizes, knn_idx, knn_dist, starts=None, stride=0):
    """In-place update of knn_idx / knn_dist with the given buckets."""
    points = _pts(points)
    N, D = points.shape
    ids = np.ascontiguousarray(ids, np.int32)
    sizes = np.ascontiguousarray(sizes, np.int32)
    sp = None
    if starts is not None:
        starts = np.ascontiguousarray(starts, np.int32)
        sp = starts.ctypes.data_as(ctypes.c_void_p)
    assert knn_idx.dtype == np.int32 and knn_dist.dtype == np.float32
    lib().rsfk_or_bucket_knn(points, N, D, int(K), ids, sp, sizes, len(sizes), int(stride), knn_idx, knn_dist)


def explore(points, K, knn_idx, knn_dist):
    points = _pts(points)
    N, D = points.shape
    lib().rsfk_or_explore(points, N, D, int(K), knn_idx, knn_dist)


def init_lists(N, K, self_in=True):
    idx = np.full((N, K), -1, np.int32)
    dist = np.full((N, K), np.inf, np.float32)
    if self_in:
        idx[:, 0] = np.arange(N, dtype=np.int32)
        dist[:, 0] = 0.0
    return idx, dist


def forest(points, K, n_trees, min_children=-1, max_children=-1, max_depth=5000, seed=0, nnef=1,
           knn_idx=None, knn_dist=None, want_log=False):
    points = _pts(points)
    N, D = points.shape
    if min_children == -1:
        min_children = K + 1
    if max_children == -1:
        max_children = 2 * min_children
    if knn_idx is None:
        knn_idx, knn_dist = init_lists(N, K)
    log = np.zeros(16 * n_trees + 2, np.float32)
    rc = lib().rsfk_or_forest(int(n_trees), int(K), N, D, int(min_children), int(max_children), int(max_depth),
                              int(seed), int(nnef), points, knn_idx, knn_dist,
                              log.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise RuntimeError("oracle forest failed")
    if want_log:
        return knn_idx, knn_dist, log
    return knn_idx, knn_dist


def route_queries(points, queries, min_children, max_children, max_depth=5000, seed=0):
    """One tree on the points; -> perm, start and size (segments of perm) of the leaf every query ends in."""
    points, queries = _pts(points), _pts(queries)
    N, D = points.shape
    NQ = queries.shape[0]
    perm = np.empty(N, np.int32)
    qs = np.full(NQ, -1, np.int32)
    qz = np.full(NQ, -1, np.int32)
    lib().rsfk_or_route_queries(points, N, D, int(min_children), int(max_children), int(max_depth), int(seed),
                                queries, NQ, perm, qs, qz)
    return perm, qs, qz


def ann_forest(points, queries, K, n_trees, min_children=-1, max_children=-1, max_depth=5000, seed=0,
               q_idx=None, q_dist=None):
    """Query-set search; rows start empty (-1, +inf) unless given."""
    points, queries = _pts(points), _pts(queries)
    N, D = points.shape
    NQ = queries.shape[0]
    if min_children == -1:
        min_children = K + 1
    if max_children == -1:
        max_children = 2 * min_children
    if q_idx is None:
        q_idx, q_dist = init_lists(NQ, K, self_in=False)
    rc = lib().rsfk_or_ann_forest(int(n_trees), int(K), N, NQ, D, int(min_children), int(max_children),
                                  int(max_depth), int(seed), points, queries, q_idx, q_dist)
    if rc != 0:
        raise RuntimeError("oracle query search failed")
    return q_idx, q_dist


def symmetrize(knn_idx, knn_dist=None, drop_self=False):
    """Symmetrised graph in CSR form -> indptr (N+1), indices, data (columns ascending inside a row)."""
    knn_idx = np.ascontiguousarray(knn_idx, np.int32)
    N, K = knn_idx.shape
    dp = None
    if knn_dist is not None:
        knn_dist = np.ascontiguousarray(knn_dist, np.float32)
        dp = knn_dist.ctypes.data_as(ctypes.c_void_p)
    indptr = np.empty(N + 1, np.int32)
    nnz = lib().rsfk_or_symmetrize(knn_idx, dp, N, K, int(bool(drop_self)), indptr, None, None, 0)
    cols = np.empty(max(nnz, 1), np.int32)
    vals = np.empty(max(nnz, 1), np.float32)
    got = lib().rsfk_or_symmetrize(knn_idx, dp, N, K, int(bool(drop_self)), indptr,
                                   cols.ctypes.data_as(ctypes.c_void_p), vals.ctypes.data_as(ctypes.c_void_p), nnz)
    if got != nnz:
        raise RuntimeError("oracle symmetrize failed")
    return indptr, cols[:nnz], vals[:nnz]


def bruteforce(points, K, queries=None):
    points = _pts(points)
    N, D = points.shape
    if queries is None:
        nq, qp = N, None
    else:
        queries = np.ascontiguousarray(queries, np.int32)
        nq, qp = len(queries), queries.ctypes.data_as(ctypes.c_void_p)
    oi = np.empty((nq, K), np.int32)
    od = np.empty((nq, K), np.float64)
    lib().rsfk_or_bruteforce(points, N, D, int(K), qp, nq, oi, od)
    return oi, od


def num_threads():
    return int(lib().rsfk_or_num_threads())


def set_num_threads(n):
    lib().rsfk_or_set_num_threads(int(n))


def recall(true_idx, approx_idx):
    """sum_rows |set(true) & set(approx)| / (rows*K)  (examples/utils/knn_compare.py:46-65)."""
    t = np.sort(np.asarray(true_idx), axis=1)
    a = np.sort(np.asarray(approx_idx), axis=1)
    hits = 0
    for r in range(t.shape[0]):
        hits += np.intersect1d(t[r], a[r], assume_unique=False).size
    return hits / float(t.shape[0] * t.shape[1])
