"""ctypes declarations of every entry point of ``librsfk.so`` (see
``include/rsfk.h``), plus thin numpy / raw-pointer helpers for the stage-level
calls.  Device pointers are passed as plain integers (for example
``tensor.data_ptr()``); this module does not import torch."""
import ctypes
import os

import numpy as np

_LIB_DIR = os.path.dirname(os.path.abspath(__file__))
_f32 = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i32 = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_vp = ctypes.c_void_p
_ci = ctypes.c_int

# name -> (restype, argtypes); the complete list of exported symbols
SYMBOLS = {
    "pymodule_rsfk_knn": (None, [_ci] * 10 + [_vp, _vp, _vp, _vp]),
    "pymodule_rsfk_knn_ann": (None, [_ci] * 11 + [_vp, _vp, _vp, _vp, _vp]),
    "pymodule_cluster_by_sample_tree": (None, [_ci] * 7 + [_vp, _vp, _vp, _vp, _vp]),
    "rsfk_knn_forest_device": (_ci, [_ci] * 10 + [_vp, _vp, _vp, _vp, _vp]),
    "rsfk_knn_ann_device": (_ci, [_ci] * 10 + [_vp, _vp, _vp, _vp, _vp, _vp]),
    "rsfk_knn_forest_fresh_host": (_ci, [_ci] * 11 + [_vp, _vp, _vp, _vp]),
    "rsfk_symmetrize_device": (_ci, [_vp, _vp, _ci, _ci, _ci, _vp, _vp, _vp, ctypes.c_longlong, _vp, _vp]),
    "rsfk_symmetrize_count_noalloc": (_ci, [_vp, _ci, _ci, _ci, _vp, _vp, _vp]),
    "rsfk_symmetrize_host": (_ci, [_vp, _vp, _ci, _ci, _ci, _vp, _vp, _vp, ctypes.c_longlong, _vp]),
    "rsfk_bucket_knn_device": (_ci, [_vp, _ci, _ci, _ci, _vp, _vp, _vp, _ci, _ci, _vp, _vp, _vp]),
    "rsfk_explore_device": (_ci, [_vp, _ci, _ci, _ci, _vp, _vp, _vp, _vp]),
    "rsfk_build_tree_host": (_ci, [_f32, _ci, _ci, _ci, _ci, _ci, _ci, _i32, _i32, _i32, _ci, _i32]),
    "rsfk_bucket_knn_host": (_ci, [_f32, _ci, _ci, _ci, _i32, _ci, _vp, _i32, _ci, _ci, _i32, _f32]),
    "rsfk_explore_host": (_ci, [_f32, _ci, _ci, _ci, _i32, _f32, _ci]),
    "rsfk_last_error": (ctypes.c_char_p, []),
    "rsfk_last_build_report": (_ci, [ctypes.c_char_p, _ci]),
    "rsfk_device_count": (_ci, []),
    "rsfk_release_workspace": (None, []),
}

_lib = None


def lib():
    """The loaded library.  Raises OSError when ``librsfk.so`` has not been built."""
    global _lib
    if _lib is None:
        L = ctypes.CDLL(os.path.join(_LIB_DIR, "librsfk.so"))
        for name, (res, args) in SYMBOLS.items():
            f = getattr(L, name)
            f.restype = res
            f.argtypes = args
        _lib = L
    return _lib


class RsfkError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise RsfkError(lib().rsfk_last_error().decode("utf-8", "replace"))


def _pts(points):
    return np.require(points, np.float32, ["C_CONTIGUOUS", "ALIGNED"])


def build_tree(points, min_children, max_children, max_depth=5000, seed=0):
    """One tree on the GPU -> (perm, leaf_start, leaf_size, stats[4])."""
    points = _pts(points)
    N, D = points.shape
    cap = N // max(int(min_children), 1) + 2
    perm = np.empty(N, np.int32)
    ls = np.empty(cap, np.int32)
    lz = np.empty(cap, np.int32)
    stats = np.zeros(4, np.int32)
    n = lib().rsfk_build_tree_host(points, N, D, int(min_children), int(max_children), int(max_depth), int(seed),
                                   perm, ls, lz, cap, stats)
    if n < 0:
        raise RsfkError(lib().rsfk_last_error().decode("utf-8", "replace"))
    return perm, ls[:n].copy(), lz[:n].copy(), stats


def bucket_knn(points, K, ids, sizes, knn_idx, knn_dist, starts=None, stride=0):
    """In-place bucket K-NN update on the GPU (host arrays in and out)."""
    points = _pts(points)
    N, D = points.shape
    ids = np.ascontiguousarray(ids, np.int32)
    sizes = np.ascontiguousarray(sizes, np.int32)
    sp = None
    if starts is not None:
        starts = np.ascontiguousarray(starts, np.int32)
        sp = starts.ctypes.data_as(_vp)
    _check(lib().rsfk_bucket_knn_host(points, N, D, int(K), ids, len(ids), sp, sizes, len(sizes), int(stride),
                                      knn_idx, knn_dist))


def explore(points, K, knn_idx, knn_dist, passes=1):
    points = _pts(points)
    N, D = points.shape
    _check(lib().rsfk_explore_host(points, N, D, int(K), knn_idx, knn_dist, int(passes)))


def knn_forest_device(n_trees, K, N, D, min_children, max_children, max_depth, verbose, seed, nnef,
                      d_points, d_idx, d_dist, log=None, stream=0):
    """Whole K-NN-graph build on device-resident buffers (integer addresses)."""
    lp = None if log is None else log.ctypes.data_as(_vp)
    _check(lib().rsfk_knn_forest_device(int(n_trees), int(K), int(N), int(D), int(min_children), int(max_children),
                                        int(max_depth), int(verbose), int(seed), int(nnef),
                                        _vp(d_points), _vp(d_idx), _vp(d_dist), lp, _vp(stream)))


def knn_ann_device(n_trees, K, N, NQ, D, min_children, max_children, max_depth, verbose, seed,
                   d_points, d_queries, d_idx, d_dist, log=None, stream=0):
    """Query-set search on device-resident buffers (integer addresses); rows NQ x K are merged into."""
    lp = None if log is None else log.ctypes.data_as(_vp)
    _check(lib().rsfk_knn_ann_device(int(n_trees), int(K), int(N), int(NQ), int(D), int(min_children),
                                     int(max_children), int(max_depth), int(verbose), int(seed),
                                     _vp(d_points), _vp(d_queries), _vp(d_idx), _vp(d_dist), lp, _vp(stream)))


def symmetrize(knn_idx, knn_dist=None, drop_self=False):
    """Symmetrised K-NN graph in CSR form -> indptr (N+1), indices, data; columns ascend inside a row."""
    knn_idx = np.ascontiguousarray(knn_idx, np.int32)
    N, K = knn_idx.shape
    dp = None
    if knn_dist is not None:
        knn_dist = np.ascontiguousarray(knn_dist, np.float32)
        if knn_dist.shape != knn_idx.shape:
            raise ValueError("knn_dist must have the shape of knn_idx")
        dp = knn_dist.ctypes.data_as(_vp)
    indptr = np.empty(N + 1, np.int32)
    nnz = ctypes.c_longlong(0)
    _check(lib().rsfk_symmetrize_host(knn_idx.ctypes.data_as(_vp), dp, N, K, int(bool(drop_self)),
                                      indptr.ctypes.data_as(_vp), None, None, 0, ctypes.byref(nnz)))
    n = int(nnz.value)
    cols = np.empty(n, np.int32)
    vals = np.empty(n, np.float32)
    if n:
        _check(lib().rsfk_symmetrize_host(knn_idx.ctypes.data_as(_vp), dp, N, K, int(bool(drop_self)),
                                          indptr.ctypes.data_as(_vp), cols.ctypes.data_as(_vp),
                                          vals.ctypes.data_as(_vp), n, ctypes.byref(nnz)))
    return indptr, cols, vals


def symmetrize_device(d_idx, d_dist, N, K, drop_self, d_indptr, d_cols, d_vals, capacity, stream=0):
    """Device-resident form (integer addresses; d_cols = d_vals = 0 for the count only) -> number of entries."""
    nnz = ctypes.c_longlong(0)
    _check(lib().rsfk_symmetrize_device(_vp(d_idx), _vp(d_dist) if d_dist else None, int(N), int(K), int(bool(drop_self)),
                                        _vp(d_indptr), _vp(d_cols) if d_cols else None, _vp(d_vals) if d_vals else None,
                                        int(capacity), ctypes.byref(nnz), _vp(stream)))
    return int(nnz.value)


def last_build_report():
    """What the last K-NN-graph build of this process did (kernels per tree, counts, seconds) as a dict."""
    import json
    buf = ctypes.create_string_buffer(1 << 16)
    lib().rsfk_last_build_report(buf, len(buf))
    return json.loads(buf.value.decode())


def symmetrize_count_noalloc(d_idx, N, K, drop_self, d_indptr, stream=0, fetch_count=True):
    """Row offsets and number of entries of the symmetrised graph without any allocation in the library (fixed
    working memory: N <= 2^20, N * K <= 2^25) -> number of entries.  fetch_count=False: the library only enqueues
    its kernels (no copy to the host, no synchronisation); the count is d_indptr[N] on the device and None is returned."""
    nnz = ctypes.c_longlong(0)
    _check(lib().rsfk_symmetrize_count_noalloc(_vp(d_idx), int(N), int(K), int(bool(drop_self)), _vp(d_indptr),
                                               ctypes.byref(nnz) if fetch_count else None, _vp(stream)))
    return int(nnz.value) if fetch_count else None


def bucket_knn_device(d_points, N, D, K, d_ids, d_starts, d_sizes, n_buckets, stride, d_idx, d_dist, stream=0):
    _check(lib().rsfk_bucket_knn_device(_vp(d_points), int(N), int(D), int(K), _vp(d_ids),
                                        _vp(d_starts) if d_starts else None, _vp(d_sizes), int(n_buckets),
                                        int(stride), _vp(d_idx), _vp(d_dist), _vp(stream)))


def explore_device(d_points, N, D, K, d_idx, d_dist, d_scratch, stream=0):
    _check(lib().rsfk_explore_device(_vp(d_points), int(N), int(D), int(K), _vp(d_idx), _vp(d_dist),
                                     _vp(d_scratch), _vp(stream)))
