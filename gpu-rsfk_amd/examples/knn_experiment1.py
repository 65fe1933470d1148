"""Quality and time of the K-NN graph as a function of the number of trees and of the exploration passes.

The sweep of the reference's examples/knn_experiment1.py:200-262 (same options, same calls of
RSFK.find_nearest_neighbors, same quality measures), with an exact CPU brute force on a sample of the points as the
ground truth instead of FAISS, and synthetic data or a .npy matrix instead of the downloaded data sets.  Writes
<path>/<name>.json.

    python knn_experiment1.py --test_rsfk -d GMM64 --n_points 100000 --dims 64 -k 32 -t 1 3 5 9 17 -e 0 1
"""
import argparse
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from gpu_rsfk.RSFK import RSFK                                          # noqa: E402
from synthetic_datasets import load_dataset, get_dataset_options                  # noqa: E402
from utils.knn_compare import get_nne_rate, create_recall_eps, exact_knn  # noqa: E402


def build_parser():
    parser = argparse.ArgumentParser(description="Parameters used to init experiments")
    parser.add_argument("-n", "--name", help="Experiment name used to create json log", type=str, default="exp1")
    parser.add_argument("-p", "--path", help="Experiment path used to create json log", type=str, default=".")
    parser.add_argument("-v", "--rsfk_verbose", help="RSFK verbose level", type=int, default=0)
    parser.add_argument("-k", "--n_neighbors", help="Number of neighbors (K) used in KNN", type=int, default=32)
    parser.add_argument("--mntc", help="Min Tree Children parameter in RSFK", type=int, default=-1)
    parser.add_argument("--mxtc", help="Max Tree Children parameter in RSFK", type=int, default=-1)
    parser.add_argument("-d", "--dataset", help="Dataset name ({}) or a .npy file".format(", ".join(get_dataset_options())),
                        type=str, default="GMM64")
    parser.add_argument("--n_points", help="Points of a synthetic dataset", type=int, default=20000)
    parser.add_argument("--dims", help="Dimensions of a synthetic dataset", type=int, default=32)
    parser.add_argument("--quality", choices=["nne", "recall_eps"], default="nne")
    parser.add_argument("--recall_eps_val", help="Recall-e value", type=float, default=0.01)
    parser.add_argument("--gt_queries", help="Points the exact ground truth is computed for (0 = all)", type=int,
                        default=5000)
    parser.add_argument("-e", "--nnexp_factor_list", type=int, nargs="+", default=[0, 1, 2],
                        help="Nearest Neighbors Exploring factor list to test")
    parser.add_argument("-t", "--n_trees_list", type=int, nargs="+", default=[x for x in range(1, 29, 2)],
                        help="List of total of trees to test")
    parser.add_argument("--skip_save", action="store_true", default=False, help="Doesnt change log file")
    parser.add_argument("--test_rsfk", action="store_true", default=False, help="Test Random Projection Forest KNN")
    parser.add_argument("--sanity_check", action="store_true", default=False, help="Fail on empty neighbour slots")
    return parser


def run(args):
    K = args.n_neighbors
    if args.quality == "nne":
        quality_function, quality_name = get_nne_rate, "nne"
    else:
        quality_function = create_recall_eps(args.recall_eps_val)
        quality_name = "recall_eps_{}".format(args.recall_eps_val)

    dataX, _ = load_dataset(args.dataset, args.n_points, args.dims)
    print("dataX.shape: {}".format(dataX.shape))
    print("K = {}".format(K))
    N = len(dataX)
    rng = np.random.RandomState(0)
    sample = np.arange(N) if args.gt_queries <= 0 or args.gt_queries >= N else np.sort(rng.permutation(N)[:args.gt_queries])
    t0 = time.time()
    real_indices, real_sqd_dist = exact_knn(dataX, sample, K)
    print("Exact K-NN of {} points on the CPU: {:.2f} s".format(len(sample), time.time() - t0))

    results = []
    if args.test_rsfk:
        for nnef in args.nnexp_factor_list:
            if args.mxtc == -1:
                method = "RSFK" + (" (NN exploring factor = {})".format(nnef) if nnef > 0 else "")
            else:
                method = "RSFK MNTC{} MXTC{}".format(args.mntc, args.mxtc) + \
                         (" (NN exploring factor = {})".format(nnef) if nnef > 0 else "")
            print("Testing knn method: {}".format(method))
            quality_list, time_list = [], []
            for n_trees in args.n_trees_list:
                rsfk = RSFK(random_state=0)
                indices, dist = rsfk.find_nearest_neighbors(dataX.copy(), K,
                                                            min_tree_children=args.mntc,
                                                            max_tree_children=args.mxtc,
                                                            max_tree_depth=5000,
                                                            n_trees=n_trees,
                                                            random_motion_force=0.1,
                                                            ensure_valid_indices=True,
                                                            nn_exploring_factor=nnef,
                                                            add_bit_random_motion=True,
                                                            verbose=args.rsfk_verbose)
                t = rsfk._last_search_time                       # data initialisation is not counted
                q = quality_function(real_indices, indices[sample], real_sqd_dist, dist[sample], max_k=K)
                time_list.append(t)
                quality_list.append(q)
                print("RSFK Time: {}".format(t), flush=True)
                print("RSFK NNP: {}".format(q), flush=True)
                print("")
                if args.sanity_check:
                    negative_indices = int(np.sum(indices == -1))
                    if negative_indices > 0:
                        raise Exception("{} Negative indices".format(negative_indices))
            results.append({"dataset": args.dataset, "K": K, "method": method, "parameter": "n_trees",
                            "parameter_list": list(args.n_trees_list), "quality_name": quality_name,
                            "quality_list": quality_list, "time_list": time_list})
    if not args.skip_save:
        os.makedirs(args.path, exist_ok=True)
        with open(os.path.join(args.path, args.name + ".json"), "w") as f:
            json.dump(results, f, indent=1)
    return results


if __name__ == "__main__":
    run(build_parser().parse_args())
