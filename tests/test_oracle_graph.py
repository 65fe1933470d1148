"""The oracle's symmetrised-graph export against scipy.sparse and a hand-written case (CPU only)."""
import numpy as np
import pytest
from scipy.sparse import csr_matrix


def _directed(idx, val, N):
    rows = np.repeat(np.arange(N), idx.shape[1])
    ok = (idx.ravel() >= 0) & (idx.ravel() < N)
    return csr_matrix((val.ravel()[ok], (rows[ok], idx.ravel()[ok])), shape=(N, N))


def test_hand_written_case(orc):
    # 0 <-> 1 mutual; 0 -> 2, 2 -> 3 and 3 -> 4 one way; 4 stores itself and an empty slot
    idx = np.array([[1, 2], [0, -1], [3, 0 + 5], [4, 4 + 5], [4, -1]], np.int32)     # 5, 9: out of range -> no edge
    d = np.array([[1.0, 2.0], [1.0, 9.0], [3.0, 9.0], [4.0, 9.0], [0.0, 9.0]], np.float32)
    indptr, cols, vals = orc.symmetrize(idx, d)
    rows = [list(zip(cols[indptr[p]:indptr[p + 1]].tolist(), vals[indptr[p]:indptr[p + 1]].tolist())) for p in range(5)]
    assert rows == [[(1, 1.0), (2, 2.0)], [(0, 1.0)], [(0, 2.0), (3, 3.0)], [(2, 3.0), (4, 4.0)], [(3, 4.0), (4, 0.0)]]
    indptr, cols, vals = orc.symmetrize(idx, d, drop_self=True)
    assert cols[indptr[4]:indptr[5]].tolist() == [3] and indptr[5] == 8
    indptr, cols, vals = orc.symmetrize(idx)                 # no distances: zeros
    assert (vals == 0).all() and indptr[5] == 9


@pytest.mark.parametrize("N,K,seed", [(200, 5, 0), (1000, 12, 1), (64, 63, 2)])
def test_equals_scipy_maximum_of_graph_and_transpose(orc, N, K, seed):
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((N, 4)).astype(np.float32)
    d2 = ((X[:, None, :] - X[None, :, :]) ** 2).sum(-1).astype(np.float32)
    d2 = np.minimum(d2, d2.T)                                # one value per pair, as the library guarantees
    idx = np.argsort(d2 + np.eye(N, dtype=np.float32) * 1e9, axis=1)[:, :K].astype(np.int32)   # no self edges
    idx[rng.random((N, K)) < 0.05] = -1                      # some empty slots
    val = np.take_along_axis(d2, np.maximum(idx, 0), 1) + 1.0    # strictly positive: scipy drops explicit zeros
    indptr, cols, vals = orc.symmetrize(idx, val)
    A = _directed(idx, val, N)
    S = A.maximum(A.T).tocsr()
    S.sort_indices()
    assert np.array_equal(indptr, S.indptr) and np.array_equal(cols, S.indices) and np.array_equal(vals, S.data)
    # symmetric, no duplicates, count-only call agrees
    G = csr_matrix((vals, cols, indptr), shape=(N, N))
    assert (abs(G - G.T)).nnz == 0
    assert all(len(set(cols[indptr[p]:indptr[p + 1]])) == indptr[p + 1] - indptr[p] for p in range(N))


def test_self_edges_kept_or_dropped(orc):
    rng = np.random.default_rng(3)
    N, K = 300, 6
    idx = np.stack([rng.permutation(N)[:K] for _ in range(N)]).astype(np.int32)
    idx[:, 0] = np.arange(N)                                 # the point itself, as find_nearest_neighbors stores it
    for p in range(N):                                       # no second copy of p further right
        idx[p, 1:][idx[p, 1:] == p] = (p + 1) % N if (p + 1) % N not in idx[p] else -1
    val = rng.random((N, K)).astype(np.float32)
    ip0, c0, v0 = orc.symmetrize(idx, val, drop_self=False)
    ip1, c1, v1 = orc.symmetrize(idx, val, drop_self=True)
    assert ip0[-1] == ip1[-1] + N
    for p in range(N):
        r0 = c0[ip0[p]:ip0[p + 1]].tolist()
        r1 = c1[ip1[p]:ip1[p + 1]].tolist()
        assert p in r0 and p not in r1 and [c for c in r0 if c != p] == r1
