"""Command-line run of the forest on generated data, the counterpart of the reference's stand-alone program
(`main`, src/rsfk.cu:2230-2295):

    python -m gpu_rsfk <Total of points> <Dimensions> <Max Depth> <Verbose> <Dataset ID>

Dataset ID 0 = SPLITED_LINE (point i has all coordinates i, the upper half shifted by N/2), 1 = UNIFORM_SQUARE
(integer coordinates drawn from [0, N)).  As there: K = 32, buckets of 33..66 points, 5 trees, no exploration, rows
start empty.  Prints the time of the call and the per-tree log.
"""
import sys
import time

import numpy as np

from . import capi
from .RSFK import ForestLog


def generate(N, D, dataset_id, seed=0):
    if dataset_id == 0:
        l = np.arange(N)
        return np.repeat((l + (l > N // 2) * (N // 2))[:, None], D, axis=1).astype(np.float32)
    if dataset_id == 1:
        return np.random.RandomState(seed).randint(0, N, (N, D)).astype(np.float32)
    raise SystemExit("Dataset ID must be 0 (SPLITED_LINE) or 1 (UNIFORM_SQUARE)")


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) < 5:
        print("Error. run with python -m gpu_rsfk <Total of points> <Dimensions> <Max Depth> <Verbose> <Dataset ID>")
        return 1
    N, D, max_depth, verbose, ds = (int(a) for a in argv[:5])
    K, n_trees, random_seed, nn_exploring_factor = 32, 5, 0, 0
    points = generate(N, D, ds, random_seed)
    knn_indices = np.full((N, K), -1, np.int32)
    knn_sqr_distances = np.full((N, K), np.finfo(np.float32).max, np.float32)
    log = np.zeros(16 * n_trees + 2, np.float32)
    L = capi.lib()
    t0 = time.time()
    L.pymodule_rsfk_knn(n_trees, K, N, D, K + 1, 2 * (K + 1), max_depth, verbose, random_seed, nn_exploring_factor,
                        points.ctypes.data, knn_indices.ctypes.data, knn_sqr_distances.ctypes.data, log.ctypes.data)
    dt = time.time() - t0
    fl = ForestLog(log)
    filled = float((knn_indices >= 0).mean())
    print("N = {}, D = {}, K = {}, trees = {}: {:.4f} s ({:.0f} points/s), {:.1f} % of the slots filled".format(
        N, D, K, n_trees, dt, N / dt, 100.0 * filled))
    print("Tree Depth: {}".format(fl.data["Tree Depth"]))
    print("Total Leaves: {}".format(fl.data["Total Leaves"]))
    return 0


if __name__ == "__main__":
    sys.exit(main())
