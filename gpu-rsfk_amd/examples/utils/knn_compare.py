"""Quality measures of an approximate K-NN graph and an exact ground truth computed on the CPU.

Same measures as the reference's examples/utils/knn_compare.py:46-94 (get_nne_rate, create_recall_eps); the ground
truth there comes from FAISS or from files, here from a brute force in float64 on a sample of the points.
"""
import numpy as np


def get_nne_rate(real_indices, indices, real_dist=None, dist=None, random_state=0, max_k=32, verbose=0):
    """Fraction of the true neighbours that were found: sum_p |true(p) & found(p)| / (N * max_k)."""
    total = 0
    for x, y in zip(real_indices, indices):
        total += len(set(x.tolist()).intersection(y.tolist()))
    return float(total) / (len(real_indices) * max_k)


def create_recall_eps(eps):
    """Recall-eps: a found neighbour counts when its distance is within (1 + eps) of the true K-th distance."""
    def get_recall_eps(real_indices, indices, real_dist, dist, random_state=0, max_k=32, verbose=0):
        total = 0
        for dx, dy in zip(real_dist, dist):
            total += int(np.sum(dy <= np.max(dx) * (1.0 + eps)))
        return float(total) / (len(real_indices) * max_k)
    return get_recall_eps


def exact_knn(points, queries, K, include_self=True, chunk=512):
    """Exact K nearest neighbours (squared Euclidean, float64) of points[queries]; ties -> smaller index.

    Returns indices (len(queries), K) and squared distances."""
    X = np.asarray(points, np.float64)
    sq = (X * X).sum(1)
    out_i = np.empty((len(queries), K), np.int64)
    out_d = np.empty((len(queries), K), np.float64)
    for a in range(0, len(queries), chunk):
        q = np.asarray(queries[a:a + chunk])
        d2 = sq[q][:, None] - 2.0 * (X[q] @ X.T) + sq[None, :]
        np.maximum(d2, 0.0, out=d2)
        d2[np.arange(len(q)), q] = 0.0 if include_self else np.inf
        part = np.argpartition(d2, K - 1, axis=1)[:, :K]
        pd = np.take_along_axis(d2, part, 1)
        order = np.lexsort((part, pd), axis=1)
        out_i[a:a + chunk] = np.take_along_axis(part, order, 1)
        out_d[a:a + chunk] = np.take_along_axis(pd, order, 1)
    return out_i, out_d
