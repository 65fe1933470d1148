"""Example scripts and the command-line program: quality measures and ground truth on the CPU, the sweep and the CLI
on the GPU."""
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "gpu-rsfk_amd", "examples"))
sys.path.insert(0, os.path.join(ROOT, "gpu-rsfk_amd"))


def test_quality_measures_closed_forms():
    from utils.knn_compare import get_nne_rate, create_recall_eps
    real = np.array([[0, 1, 2, 3], [4, 5, 6, 7]])
    found = np.array([[3, 2, 9, 8], [7, 6, 5, 4]])
    assert get_nne_rate(real, found, max_k=4) == pytest.approx((2 + 4) / 8)
    rd = np.array([[0.0, 1.0, 2.0, 4.0], [0.0, 1.0, 1.0, 1.0]])
    fd = np.array([[0.0, 4.0, 4.03, 4.05], [1.0, 1.0, 1.02, 0.5]])
    assert create_recall_eps(0.01)(real, found, rd, fd, max_k=4) == pytest.approx((3 + 3) / 8)
    assert create_recall_eps(0.0)(real, found, rd, fd, max_k=4) == pytest.approx((2 + 3) / 8)


def test_exact_knn_against_scipy():
    from scipy.spatial.distance import cdist
    from utils.knn_compare import exact_knn
    rng = np.random.default_rng(0)
    X = rng.standard_normal((700, 9)).astype(np.float32)
    q = np.array([0, 5, 699, 123])
    idx, d = exact_knn(X, q, 6, chunk=3)
    full = cdist(X[q].astype(np.float64), X.astype(np.float64), "sqeuclidean")
    want = np.argsort(full, axis=1, kind="stable")[:, :6]
    assert np.array_equal(idx, want) and (idx[:, 0] == q).all()
    assert np.allclose(d, np.take_along_axis(full, want, 1), atol=1e-9)
    idx2, _ = exact_knn(X, q, 6, include_self=False)
    assert np.array_equal(idx2[:, :5], want[:, 1:])


def test_datasets_and_parser(tmp_path):
    from synthetic_datasets import load_dataset, get_dataset_options
    import knn_experiment1
    for name in get_dataset_options():
        X, y = load_dataset(name, 300, 5)
        assert X.shape == (300, 5) and X.dtype == np.float32 and len(y) == 300
    X, _ = load_dataset("SPLITED_LINE", 10, 2)
    assert X[:, 0].tolist() == [0, 1, 2, 3, 4, 5, 11, 12, 13, 14]        # upper half shifted by N/2 (rsfk.cu:2276)
    np.save(tmp_path / "m.npy", np.arange(12, dtype=np.float64).reshape(4, 3))
    X, _ = load_dataset(str(tmp_path / "m.npy"))
    assert X.shape == (4, 3) and X.dtype == np.float32
    a = knn_experiment1.build_parser().parse_args([])
    assert (a.name, a.path, a.n_neighbors, a.mntc, a.mxtc, a.recall_eps_val) == ("exp1", ".", 32, -1, -1, 0.01)
    assert a.nnexp_factor_list == [0, 1, 2] and a.n_trees_list == list(range(1, 29, 2))     # knn_experiment1.py:54-60
    from gpu_rsfk.__main__ import generate, main
    assert generate(8, 3, 0).tolist()[5] == [9.0, 9.0, 9.0] and generate(50, 4, 1).max() < 50
    assert main(["10", "2"]) == 1                                        # too few arguments, as rsfk.cu:2232-2235


@pytest.mark.gpu
def test_sweep_quality_rises_with_trees_and_exploration(gpu, tmp_path):
    import knn_experiment1
    args = knn_experiment1.build_parser().parse_args(
        ["--test_rsfk", "-d", "GMM64", "--n_points", "20000", "--dims", "24", "-k", "16", "-t", "1", "4", "12", "-e", "0", "1",
         "--gt_queries", "1500", "-p", str(tmp_path), "-n", "sweep", "--sanity_check"])
    print("sweep", flush=True)
    res = knn_experiment1.run(args)
    assert len(res) == 2 and res[0]["method"] == "RSFK" and res[1]["method"] == "RSFK (NN exploring factor = 1)"
    for r in res:
        q = r["quality_list"]
        assert q[0] < q[1] < q[2] <= 1.0 and all(t > 0 for t in r["time_list"])
    # (with one tree there is nothing new to explore; every call perturbs the data afresh, so that pair is noise)
    assert all(a < b for a, b in zip(res[0]["quality_list"][1:], res[1]["quality_list"][1:]))
    assert res[1]["quality_list"][-1] > 0.9
    assert json.load(open(tmp_path / "sweep.json"))[0]["parameter_list"] == [1, 4, 12]
    args = knn_experiment1.build_parser().parse_args(
        ["--test_rsfk", "-d", "UNIFORM", "--n_points", "5000", "--dims", "8", "-k", "8", "-t", "2", "-e", "0",
         "--quality", "recall_eps", "--skip_save", "--gt_queries", "0"])
    res = knn_experiment1.run(args)
    assert res[0]["quality_name"] == "recall_eps_0.01" and 0 < res[0]["quality_list"][0] <= 1.0


@pytest.mark.gpu
def test_command_line_program(gpu, capsys):
    from gpu_rsfk.__main__ import main
    print("cli", flush=True)
    assert main(["20000", "16", "5000", "0", "1"]) == 0
    out = capsys.readouterr().out
    assert "N = 20000, D = 16, K = 32, trees = 5" in out and "Total Leaves" in out
    assert main(["3000", "4", "5000", "0", "0"]) == 0
