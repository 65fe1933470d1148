"""Pure-Python restatements used to pin the oracle's control flow on small
inputs.  They are written from the rules, not from the oracle's C code:

  tree    : split / min-size merge / leaf rules of
            src/kernels/build_tree_update_parents.cu:64-75,106-134 and the
            pair draw per (node, side) of build_tree_create_nodes.cu:86-104,
            expressed recursively over Python lists;
  insert  : "replace the maximum iff below it and not present"
            (compute_knn_from_buckets.cu:1215-1230), with rows ordered by
            (distance, index) so that ties at the K-th distance keep the smaller index;
  explore : nearest_neighbors_exploring.cu:70-141;
  route   : the descent of a query point through a tree (src/rsfk.cu:262-356,
            build_tree_update_parents_ann.cu:141-151): side test where the node has
            two children, the only child otherwise.

The random draws and the fp32 side test are taken from the oracle's exported
helpers (pick_pair / hyperplane / dot32), which have their own tests.
"""
import numpy as np


def tree(orc, X, MIN, MAX, MAX_DEPTH, seed):
    """-> list of buckets (lists of ids) in left-to-right order, and the number of levels."""
    buckets = []
    levels = [1]

    def rec(members, draw_from, key, depth, leaf):
        levels[0] = max(levels[0], depth + 1)
        if leaf or depth >= MAX_DEPTH - 1:
            buckets.append(list(members))
            return
        r1, r2 = orc.pick_pair(key, len(draw_from))
        n, b = orc.hyperplane(X[draw_from[r1]], X[draw_from[r2]])
        left = [p for p in members if not (orc.dot32(n, X[p]) < b)]
        right = [p for p in members if orc.dot32(n, X[p]) < b]
        kl, kr = orc.child_key(key, 0), orc.child_key(key, 1)
        c = len(members)
        if not left or not right:
            only = left if left else right
            rec(only, only, kl if left else kr, depth + 1, c <= MAX - 2)
        elif min(len(left), len(right)) < MIN:
            whole = left + right
            if len(left) >= len(right):
                rec(whole, left, kl, depth + 1, c <= MAX)
            else:
                rec(whole, right, kr, depth + 1, c <= MAX)
        else:
            rec(left, left, kl, depth + 1, len(left) <= MAX - 2)
            rec(right, right, kr, depth + 1, len(right) <= MAX - 2)

    import sys
    old = sys.getrecursionlimit()
    sys.setrecursionlimit(max(old, MAX_DEPTH + 1000))
    try:
        ids = list(range(X.shape[0]))
        rec(ids, ids, orc.root_key(seed), 0, False)
    finally:
        sys.setrecursionlimit(old)
    return buckets, levels[0]


def route(orc, X, Q, MIN, MAX, MAX_DEPTH, seed):
    """-> for every query the bucket (list of ids of X) it ends in.  The tree is the one of `tree` above; a query
    is carried along the recursion instead of being routed afterwards."""
    out = [None] * Q.shape[0]

    def rec(members, draw_from, key, depth, leaf, queries):
        if leaf or depth >= MAX_DEPTH - 1:
            for q in queries:
                out[q] = list(members)
            return
        r1, r2 = orc.pick_pair(key, len(draw_from))
        n, b = orc.hyperplane(X[draw_from[r1]], X[draw_from[r2]])
        left = [p for p in members if not (orc.dot32(n, X[p]) < b)]
        right = [p for p in members if orc.dot32(n, X[p]) < b]
        kl, kr = orc.child_key(key, 0), orc.child_key(key, 1)
        c = len(members)
        if not left or not right:
            only = left if left else right
            rec(only, only, kl if left else kr, depth + 1, c <= MAX - 2, queries)
        elif min(len(left), len(right)) < MIN:
            whole = left + right
            if len(left) >= len(right):
                rec(whole, left, kl, depth + 1, c <= MAX, queries)
            else:
                rec(whole, right, kr, depth + 1, c <= MAX, queries)
        else:
            ql = [q for q in queries if not (orc.dot32(n, Q[q]) < b)]
            qr = [q for q in queries if orc.dot32(n, Q[q]) < b]
            rec(left, left, kl, depth + 1, len(left) <= MAX - 2, ql)
            rec(right, right, kr, depth + 1, len(right) <= MAX - 2, qr)

    import sys
    old = sys.getrecursionlimit()
    sys.setrecursionlimit(max(old, MAX_DEPTH + 1000))
    try:
        ids = list(range(X.shape[0]))
        rec(ids, ids, orc.root_key(seed), 0, False, list(range(Q.shape[0])))
    finally:
        sys.setrecursionlimit(old)
    return out


def insert(idx_row, dist_row, c, d):
    """One candidate against one row (lists, modified in place)."""
    m = max(range(len(dist_row)), key=lambda j: (dist_row[j], idx_row[j]))     # largest (distance, index)
    if not (d < float("inf")) or not ((d, c) < (dist_row[m], idx_row[m])):
        return False
    if c in idx_row:
        return False
    idx_row[m] = c
    dist_row[m] = d
    return True


def bucket_knn(orc, X, K, buckets, idx, dist):
    """All pairs of every bucket, both directions; arrival order is free
    (results are compared as sets)."""
    idx = [list(r) for r in idx]
    dist = [list(r) for r in dist]
    for b in buckets:
        for i in range(len(b)):
            for j in range(i + 1, len(b)):
                d = orc.sqdist(X[b[i]], X[b[j]])
                insert(idx[b[i]], dist[b[i]], b[j], d)
                insert(idx[b[j]], dist[b[j]], b[i], d)
    return np.array(idx, np.int32), np.array(dist, np.float32)


def explore(orc, X, K, idx, dist):
    old = np.array(idx).copy()
    idx = [list(r) for r in idx]
    dist = [list(r) for r in dist]
    N = X.shape[0]
    for p in range(N):
        for i in range(K):
            q = old[p][i]
            if q < 0:
                continue
            for k in range(K):
                c = old[q][k]
                if c < 0 or c == p:
                    continue
                insert(idx[p], dist[p], int(c), orc.sqdist(X[c], X[p]))
    return np.array(idx, np.int32), np.array(dist, np.float32)
