"""Synthetic data sets for the example scripts (the reference's examples/datasets.py loads MNIST, CIFAR and others
from files and the network; none of them is available offline) and a loader for .npy files."""
import numpy as np

SYNTHETIC = ("UNIFORM", "NORMAL", "GMM64", "SPLITED_LINE", "UNIFORM_SQUARE")


def get_dataset_options():
    return list(SYNTHETIC)


def load_dataset(name, n=20000, d=32, seed=0):
    """-> (dataX float32 (n, d), dataY int labels).  `name` is one of SYNTHETIC or the path of a .npy matrix."""
    rng = np.random.RandomState(seed)
    if name.endswith(".npy"):
        X = np.load(name, allow_pickle=False).astype(np.float32)
        return np.ascontiguousarray(X.reshape(len(X), -1)), np.zeros(len(X), np.int64)
    if name == "UNIFORM":
        return rng.random_sample((n, d)).astype(np.float32), np.zeros(n, np.int64)
    if name == "NORMAL":
        return rng.standard_normal((n, d)).astype(np.float32), np.zeros(n, np.int64)
    if name == "GMM64":
        centres = rng.standard_normal((64, d)) * 4.0
        y = rng.randint(0, 64, n)
        return (centres[y] + rng.standard_normal((n, d))).astype(np.float32), y
    if name == "SPLITED_LINE":           # the generators of the reference's command-line program, src/rsfk.cu:2262-2282
        l = np.arange(n)
        X = np.repeat((l + (l > n // 2) * (n // 2))[:, None], d, axis=1).astype(np.float32)
        return X, (l > n // 2).astype(np.int64)
    if name == "UNIFORM_SQUARE":
        return rng.randint(0, n, (n, d)).astype(np.float32), (rng.randint(0, n, n) > n // 2).astype(np.int64)
    raise ValueError("unknown data set {}".format(name))
