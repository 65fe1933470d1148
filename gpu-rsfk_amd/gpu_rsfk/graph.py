"""Export of a K-NN graph for the pipelines that consume it (t-SNE, UMAP, spectral methods)."""
import numpy as np

from . import capi


def symmetric_knn_graph(knn_indices, knn_squared_dist=None, drop_self=True, as_scipy=False):
    """Symmetrised K-NN graph in compressed-row (CSR) form, built on the GPU.

    Row ``p`` holds every neighbour stored for ``p`` and every point that stores ``p``
    as a neighbour, each once, with the squared distance of the pair; the columns of
    a row ascend.  The reference keeps this step as commented-out kernels beside its
    spectral experiment (``src/rsfk.cu:1229-1299``).

    Parameters
    ----------
    knn_indices : int32 array (N, K); slots that are negative or >= N are no edges
    knn_squared_dist : float32 array (N, K) or None (the values are then zero)
    drop_self : remove ``p`` from its own row (``find_nearest_neighbors`` stores it by default)
    as_scipy : return a ``scipy.sparse.csr_matrix`` instead of the three arrays

    Returns
    -------
    indptr (N + 1, int32), indices (nnz, int32), data (nnz, float32)
    """
    knn_indices = np.require(knn_indices, np.int32, ['CONTIGUOUS', 'ALIGNED'])
    if knn_indices.ndim != 2:
        raise ValueError("knn_indices must be a matrix (points x neighbours)")
    indptr, indices, data = capi.symmetrize(knn_indices, knn_squared_dist, drop_self)
    if as_scipy:
        from scipy.sparse import csr_matrix
        n = knn_indices.shape[0]
        return csr_matrix((data, indices, indptr), shape=(n, n))
    return indptr, indices, data
