"""Benchmark of the K-NN-graph build on one MI355X.

A step is one complete build (forest of random-sample trees with bucket K-NN,
then the exploration passes) on inputs that are already resident in HBM, through
the C-ABI entry point ``rsfk_knn_forest_device``.  Default workload: BASELINE
config 2, N=1,000,000 x D=100 uniform points, K=32, 50 trees, one exploration
pass, buckets 33..66; ``--config c1..c5`` selects any of the five.  Prints one
JSON line.  ``host_call_seconds`` is the region the reference times
(``RSFK._last_search_time``: host arrays in, host arrays out).

``value`` times the device-resident build (``timed_region``).  Three roofline objects, one per subsystem:
``roofline`` (bucket K-NN, the metric's kernel), ``roofline_tree`` (tree build: sum over the levels of the points of
the nodes that are split, times the bytes of a screening row and of the permutation entry read and written by the side
test and by the scatter, plus the fp32 rows of the points the screen leaves to the exact test, plus the permutation
written once) and ``roofline_explore`` (one pass: the fp32 rows of the candidates that get an exact distance, the
K^2 ids of the neighbours' rows and the K-NN row read and written); the counts come from the library's report of
the build (``rsfk_last_build_report``), as do the names of the bucket kernels that ran.

The first roofline object is for the bucket K-NN step: algorithmic bytes per launch
(one launch = one tree) = N*(4D + 4 + 16K) -- every point row gathered once, every
id read once, every K-NN row (index + distance) read once and written once --
or, where the arithmetic intensity is above the machine balance, 3 D P flops
(P = pairs of the tree's buckets), divided by the average duration of a launch
measured with HIP events recorded on the launching stream inside the library
(they come back in the per-tree log).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "gpu-rsfk_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0


def make_points(N, D, workload, seed=0):
    rng = np.random.default_rng(seed)
    if workload == "uniform":
        return rng.random((N, D), dtype=np.float32)
    if workload == "normal":
        return rng.standard_normal((N, D), dtype=np.float32)
    if workload == "gmm64":
        centres = rng.random((64, D), dtype=np.float32)
        comp = rng.integers(64, size=N)
        return (centres[comp] + 0.1 * rng.standard_normal((N, D), dtype=np.float32)).astype(np.float32)
    if workload == "sparse":
        X = 1.0 - rng.random((N, D), dtype=np.float32)
        X[rng.random((N, D), dtype=np.float32) < 0.8] = 0.0
        return X
    raise SystemExit("unknown workload %r" % workload)


def exact_knn_sample(torch, dX, queries, K, chunk=65536):
    """Exact K-NN of the query rows against all rows (float64 on the GPU)."""
    q = dX[queries].double()
    qn = (q * q).sum(1)
    nq = q.shape[0]
    best_d = torch.full((nq, K), float("inf"), dtype=torch.float64, device=dX.device)
    best_i = torch.full((nq, K), -1, dtype=torch.int64, device=dX.device)
    for s in range(0, dX.shape[0], chunk):
        xb = dX[s:s + chunk].double()
        d2 = qn[:, None] + (xb * xb).sum(1)[None, :] - 2.0 * (q @ xb.T)
        ids = torch.arange(s, s + xb.shape[0], device=dX.device)[None, :].expand(nq, -1)
        dd = torch.cat([best_d, d2], 1)
        ii = torch.cat([best_i, ids], 1)
        best_d, o = torch.topk(dd, K, dim=1, largest=False)
        best_i = torch.gather(ii, 1, o)
    return best_i


def _base(metric, value, unit, args, sec_per_step, workload):
    return {"metric": metric, "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 3), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": {"workload": workload}}


def bench_ann(args):
    """Query-set search: a step = n_trees trees built on the points, every query routed and merged per tree."""
    import torch
    from gpu_rsfk import capi
    from gpu_rsfk.RSFK import ForestLog
    if not torch.cuda.is_available() or capi.lib().rsfk_device_count() < 1:
        raise SystemExit("bench.py: no GPU visible")
    N, D, K, T = args.n, args.d, args.k, args.trees
    NQ = N if args.queries < 0 else args.queries
    mn = K + 1 if args.min_children < 0 else args.min_children
    mx = 2 * mn if args.max_children < 0 else args.max_children
    both = make_points(N + NQ, D, args.workload)           # points and queries from one distribution
    X, Q = np.ascontiguousarray(both[:N]), np.ascontiguousarray(both[N:])
    del both
    dX, dQ = torch.from_numpy(X).cuda(), torch.from_numpy(Q).cuda()
    idx = torch.empty((NQ, K), dtype=torch.int32, device="cuda")
    dist = torch.empty((NQ, K), dtype=torch.float32, device="cuda")
    logs = []

    def step(keep):
        idx.fill_(-1)
        dist.fill_(float("inf"))
        log = np.zeros(16 * T + 2, np.float32)
        capi.knn_ann_device(T, K, N, NQ, D, mn, mx, 5000, 0, 0, dX.data_ptr(), dQ.data_ptr(), idx.data_ptr(),
                            dist.data_ptr(), log)
        if keep:
            logs.append(log)

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(True)
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / max(args.steps, 1)

    nq = min(args.recall_queries, NQ)
    sel = torch.from_numpy(np.random.default_rng(1).choice(NQ, nq, replace=False)).cuda()
    best_d = torch.full((nq, K), float("inf"), device="cuda", dtype=torch.float64)
    best_i = torch.full((nq, K), -1, device="cuda", dtype=torch.int64)
    q64 = dQ[sel].double()
    for a in range(0, N, 65536):
        xs = dX[a:a + 65536].double()
        dd = torch.cat([best_d, torch.cdist(q64, xs) ** 2], 1)
        ii = torch.cat([best_i, torch.arange(a, a + xs.shape[0], device="cuda").expand(nq, -1)], 1)
        best_d, o = torch.topk(dd, K, dim=1, largest=False)
        best_i = torch.gather(ii, 1, o)
    hits = (idx[sel].long()[:, :, None] == best_i[:, None, :]).any(2).sum().item()

    upd_s = float(np.mean([np.mean(ForestLog(l).data["KNN Sets Updates"]) for l in logs])) if logs and T > 0 else 0.0
    alg_bytes = float(N) * 4 * D + float(NQ) * (4 * D + 16 * K)
    achieved = alg_bytes / upd_s / 1e9 if upd_s > 0 else 0.0
    cpu = None
    if args.cpu_sample > 0:
        from oracle import rsfk_oracle as orc
        ns, nqs = min(args.cpu_sample, N), min(args.cpu_sample, NQ)
        c0 = time.perf_counter()
        orc.ann_forest(np.ascontiguousarray(X[:ns]), np.ascontiguousarray(Q[:nqs]), K, T, mn, mx, 5000, 0)
        cs = time.perf_counter() - c0
        cpu = {"value": round(nqs / cs, 1), "unit": "queries/s", "cores": orc.num_threads(), "kind": "port",
               "seconds": round(cs, 3),
               "sample": "first %d points and first %d queries of the same workload, same D, K, %d trees, OpenMP" % (ns, nqs, T)}
    out = _base("ann_queries_per_sec", NQ / sec, "queries/s", args, sec,
                "%s N=%d NQ=%d D=%d K=%d n_trees=%d buckets=%d..%d seed=0" % (args.workload, N, NQ, D, K, T, mn, mx))
    out.update({"recall_at_k": round(hits / float(nq * K), 4), "recall_queries": nq,
                "roofline": {"kernel": "per-tree query update (k_planes, k_route, scan, k_ann_fill, k_ann_leaf)", "bound": "hbm",
                             "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                             "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_ms": round(upd_s * 1e3, 4),
                             "launches_per_step": T},
                "cpu_baseline": cpu})
    print(json.dumps(out))


def bench_graph(args):
    """CSR export: a step = one full rsfk_symmetrize_device call on a graph built beforehand."""
    import torch
    from gpu_rsfk import capi
    if not torch.cuda.is_available() or capi.lib().rsfk_device_count() < 1:
        raise SystemExit("bench.py: no GPU visible")
    N, D, K, T = args.n, args.d, args.k, args.trees
    mn = K + 1 if args.min_children < 0 else args.min_children
    mx = 2 * mn if args.max_children < 0 else args.max_children
    X = make_points(N, D, args.workload)
    dX = torch.from_numpy(X).cuda()
    idx = torch.full((N, K), -1, dtype=torch.int32, device="cuda")
    idx[:, 0] = torch.arange(N, dtype=torch.int32, device="cuda")
    dist = torch.full((N, K), float("inf"), dtype=torch.float32, device="cuda")
    dist[:, 0] = 0.0
    capi.knn_forest_device(T, K, N, D, mn, mx, 5000, 0, 0, args.explore, dX.data_ptr(), idx.data_ptr(), dist.data_ptr())
    indptr = torch.empty(N + 1, dtype=torch.int32, device="cuda")
    nnz = capi.symmetrize_device(idx.data_ptr(), dist.data_ptr(), N, K, True, indptr.data_ptr(), 0, 0, 0)
    cols = torch.empty(nnz, dtype=torch.int32, device="cuda")
    vals = torch.empty(nnz, dtype=torch.float32, device="cuda")

    def step():
        capi.symmetrize_device(idx.data_ptr(), dist.data_ptr(), N, K, True, indptr.data_ptr(), cols.data_ptr(),
                               vals.data_ptr(), nnz)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / max(args.steps, 1)
    cpu = None
    if args.cpu_sample > 0:
        from oracle import rsfk_oracle as orc
        hi, hd = idx.cpu().numpy(), dist.cpu().numpy()
        c0 = time.perf_counter()
        op, oc, ov = orc.symmetrize(hi, hd, drop_self=True)
        cs = time.perf_counter() - c0
        same = bool(np.array_equal(op, indptr.cpu().numpy()) and np.array_equal(oc, cols.cpu().numpy()) and
                    np.array_equal(ov, vals.cpu().numpy()))
        cpu = {"value": round(len(oc) / cs, 1), "unit": "edges/s", "cores": 1, "kind": "port", "seconds": round(cs, 3),
               "sample": "the same graph, whole", "identical_to_gpu_result": same}
    alg_bytes = float(N) * K * 8 + float(nnz) * 8 + (N + 1) * 4.0
    out = _base("graph_export_edges_per_sec", nnz / sec, "edges/s", args, sec,
                "%s N=%d D=%d K=%d n_trees=%d exploration=%d: symmetrised CSR without self edges, %d entries" % (
                    args.workload, N, D, K, T, args.explore, nnz))
    out.update({"roofline": {"kernel": "whole export (k_sym_flags, scan, k_sym_fill, segmented sort)", "bound": "hbm",
                             "achieved": round(alg_bytes / sec / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(alg_bytes / sec / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                             "algorithmic_bytes_per_launch": alg_bytes},
                "cpu_baseline": cpu})
    print(json.dumps(out))


# The benchmark configurations: (workload, N, D, K, trees, min, max, exploration passes)
CONFIGS = {
    "c1": ("uniform", 10000, 32, 16, 4, 32, 128, 1),
    "c2": ("uniform", 1000000, 100, 32, 50, 33, 66, 1),
    "c3": ("gmm64", 1000000, 256, 32, 20, 33, 66, 1),
    "c4": ("sparse", 70000, 784, 90, 10, 91, 182, 1),
    "c5": ("normal", 10000000, 32, 32, 10, 64, 256, 1),
}
FP32_PEAK_TFLOPS = 157.3


def gather_probe(dX, N, D, reps=5):
    """Rate of rsfk_probe_gather_device (the benchmark's own helper library, gpu-rsfk_amd/bench/librsfk_probe.so)
    over all rows of dX in a random order (HIP events on the launching stream).
    Twice: back to back ("GB/s": the last-level cache still holds what the run before left of the matrix -- all of a
    small one), and each time after 600 MB of other data were written ("GB/s_after_other_writes": the caches hold
    modified lines of something else, as they do between two kernels of a build, whose K-NN rows, permutations and
    screening copies pass through them)."""
    import ctypes
    import torch
    probe = ctypes.CDLL(os.path.join(ROOT, "gpu-rsfk_amd", "bench", "librsfk_probe.so")).rsfk_probe_gather_device
    probe.restype = ctypes.c_int
    probe.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_longlong, ctypes.c_void_p,
                      ctypes.c_void_p]
    ids = torch.randperm(N, device=dX.device, dtype=torch.int64).to(torch.int32)
    sums = torch.empty(4096, dtype=torch.float32, device=dX.device)
    other = torch.empty(150 * 1024 * 1024, dtype=torch.float32, device=dX.device)
    stream = torch.cuda.current_stream()
    rates = []
    for spoil in (False, True):
        times = []
        for rep in range(reps + 1):
            if spoil:
                other.fill_(float(rep))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            if probe(dX.data_ptr(), N, D, ids.data_ptr(), N, sums.data_ptr(), stream.cuda_stream) != 0:
                raise RuntimeError("gather probe: launch failed")
            e1.record(stream)
            e1.synchronize()
            if rep > 0:
                times.append(e0.elapsed_time(e1) * 1e-3)
        rates.append(float(np.median(times)))
    del other
    return {"row_bytes": 4 * D, "rows": N, "seconds": round(rates[0], 7), "GB/s": round(4.0 * D * N / rates[0] / 1e9, 1),
            "seconds_after_other_writes": round(rates[1], 7),
            "GB/s_after_other_writes": round(4.0 * D * N / rates[1] / 1e9, 1),
            "note": "rows of the point matrix read once in a random order and nothing else; second figure: after 600 MB "
                    "of other data were written, so that the caches hold none of the matrix"}


PROFILE_FILES = {"c2": "knng_build_c2_uniform_1M_d100_k32.md", "c3": "knng_build_c3_gmm64_1M_d256_k32.md",
                 "c4": "knng_build_c4_sparse_70k_d784_k90.md", "c5": "knng_build_c5_normal_10M_d32_k32.md"}
FETCH_SCALE = 1.92          # FETCH_SIZE reads 0.52 of the bytes a copy kernel of known size loads; WRITE_SIZE matches


def bucket_sources_hash():
    """Hash of the sources of the bucket K-NN kernels: a tracked profile states the hash it was made with, and its
    counters are only taken for this run's line when the kernels are still the same."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "gpu-rsfk_amd", "csrc")
    for fn in sorted(os.listdir(src)):
        if fn.startswith("bucket_knn") or fn in ("bucket_small_body.hpp", "knn_list.hpp", "mfma_split.hpp", "wave64.hpp"):
            h.update(open(os.path.join(src, fn), "rb").read())
    return h.hexdigest()[:16]


def profiled_traffic(config, steps_profiled=2):
    """HBM bytes per tree of the bucket K-NN kernels from the tracked rocprofv3 summary of this workload
    (profiles/: FETCH_SIZE and WRITE_SIZE in KiB per launch, launches of two builds), or None -- also None when the
    summary was made with other sources of the bucket kernels than this run's (its line "bucket kernel sources:").
    The counters cannot be collected inside this run; the summary is of the same command (bench.py --config <c>)."""
    fn = PROFILE_FILES.get(config)
    path = os.path.join(ROOT, "profiles", fn) if fn else None
    if not path or not os.path.exists(path):
        return None
    text = open(path).read()
    if ("bucket kernel sources: " + bucket_sources_hash()) not in text:
        return None
    launches, kib = {}, {}
    for line in text.splitlines():
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) == 7 and cells[0].startswith("k_bucket_"):
            try:
                if "." in cells[2]:                       # trace table: launches, total ms, ...
                    launches[cells[0]] = int(cells[1])
                else:                                     # counter table: FETCH KiB, WRITE KiB per launch
                    kib[cells[0]] = (float(cells[1]), float(cells[2]))
            except ValueError:
                pass
    total = 0.0
    for k, n in launches.items():
        if k in kib:
            total += n * (kib[k][0] * FETCH_SCALE + kib[k][1]) * 1024.0
    return total / steps_profiled if total > 0 else None


def bucket_roofline(N, D, K, T, mn, mx, knn_s, leaf_counts, kernels):
    """Roofline object of the bucket K-NN step of one tree (one step of the forest loop = one tree's launches).

    Bytes: N (4D + 4 + 16K) per tree.  Flops: 3 D P with P = pairs of the tree's buckets, estimated from the number of
    buckets L the run reported as N (N / L - 1) / 2 (equal buckets: a lower bound of the true sum).  The bound is the
    one the workload's arithmetic intensity selects: fp32 when flops / bytes exceeds peak flops / peak bandwidth.
    kernels: what the library says it launched (runs of trees and kernel names, rsfk_last_build_report)."""
    alg_bytes = float(N) * (4 * D + 4 + 16 * K)
    mean_leaves = float(np.mean(leaf_counts)) if len(leaf_counts) else max(1.0, N / (0.75 * mx))
    pairs = 0.5 * N * (N / mean_leaves - 1.0)
    alg_flops = 3.0 * D * pairs
    balance = FP32_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
    kernel = "; ".join("trees %d..%d: %s" % (a, b, " + ".join(names)) for a, b, names in kernels) if kernels else "none"
    if alg_flops / alg_bytes > balance:
        ach = alg_flops / knn_s / 1e12 if knn_s > 0 else 0.0
        # "mfma" is the name the bench contract has for the compute roofline; the peak used is the fp32 one (vector
        # and matrix fp32 peaks are the same figure on this device) and "unit_used" names what the kernel ran on
        return {"kernel": kernel, "bound": "mfma", "unit_used": "fp32 vector ALUs (the chains of the direct-difference path)",
                "achieved": round(ach, 2), "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(ach / FP32_PEAK_TFLOPS, 4), "traffic": None, "algorithmic_flops_per_launch": alg_flops,
                "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_ms": round(knn_s * 1e3, 4), "launches_per_step": T,
                "note": "flops = 3 D P of the direct-difference path (fp32 peak 157.3 TFLOP/s); HBM traffic: see profiles/"}
    ach = alg_bytes / knn_s / 1e9 if knn_s > 0 else 0.0
    return {"kernel": kernel, "bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes_per_launch": alg_bytes,
            "algorithmic_flops_per_launch": alg_flops, "avg_launch_ms": round(knn_s * 1e3, 4), "launches_per_step": T,
            "note": "traffic (HBM bytes per launch from FETCH_SIZE / WRITE_SIZE) is not measured by this run: see profiles/"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", default=None, choices=sorted(CONFIGS), help="one of the benchmark configurations (sets the shape flags)")
    ap.add_argument("--n", type=int, default=1000000)
    ap.add_argument("--d", type=int, default=100)
    ap.add_argument("--k", type=int, default=32)
    ap.add_argument("--trees", type=int, default=50)
    ap.add_argument("--explore", type=int, default=1)
    ap.add_argument("--min-children", type=int, default=-1)
    ap.add_argument("--max-children", type=int, default=-1)
    ap.add_argument("--workload", default="uniform", choices=["uniform", "normal", "gmm64", "sparse"])
    ap.add_argument("--recall-queries", type=int, default=10000)
    ap.add_argument("--cpu-sample", type=int, default=-1,
                    help="rows of the workload the CPU baseline runs on (0 = skip; default: what about 30 s of CPU time cover, the whole workload if that suffices)")
    ap.add_argument("--cpu-full", action="store_true", help="CPU baseline on the whole workload (minutes at the large configurations)")
    ap.add_argument("--host-calls", type=int, default=2, help="timed calls of RSFK.find_nearest_neighbors (host buffers in and out)")
    ap.add_argument("--path", default="knng", choices=["knng", "ann", "graph"],
                    help="knng = K-NN-graph build (the headline metric); ann = query-set search; graph = CSR export")
    ap.add_argument("--queries", type=int, default=-1, help="query points of --path ann (default: as many as points)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on one GPU only (--gpus 1); nothing here uses a second GPU")
    if args.config:
        args.workload, args.n, args.d, args.k, args.trees, args.min_children, args.max_children, args.explore = CONFIGS[args.config]
    if args.path == "ann":
        if args.cpu_sample < 0:
            args.cpu_sample = 100000
        return bench_ann(args)
    if args.path == "graph":
        if args.cpu_sample < 0:
            args.cpu_sample = 1
        return bench_graph(args)

    import torch
    import gpu_rsfk
    from gpu_rsfk import capi
    from gpu_rsfk.RSFK import ForestLog

    if not torch.cuda.is_available() or capi.lib().rsfk_device_count() < 1:
        raise SystemExit("bench.py: no GPU visible")
    N, D, K, T = args.n, args.d, args.k, args.trees
    mn = K + 1 if args.min_children < 0 else args.min_children
    mx = 2 * mn if args.max_children < 0 else args.max_children
    X = make_points(N, D, args.workload)
    dX = torch.from_numpy(X).cuda()
    idx = torch.empty((N, K), dtype=torch.int32, device="cuda")
    dist = torch.empty((N, K), dtype=torch.float32, device="cuda")
    self_ids = torch.arange(N, dtype=torch.int32, device="cuda")

    def reset_lists():
        idx.fill_(-1)
        idx[:, 0] = self_ids
        dist.fill_(float("inf"))
        dist[:, 0] = 0.0

    logs = []

    def step(keep):
        reset_lists()
        log = np.zeros(16 * T + 2, np.float32)
        capi.knn_forest_device(T, K, N, D, mn, mx, 5000, 0, 0, args.explore,
                               dX.data_ptr(), idx.data_ptr(), dist.data_ptr(), log)
        if keep:
            logs.append(log)

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(True)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    sec_per_step = elapsed / max(args.steps, 1)
    report = capi.last_build_report()               # of the last timed step

    # recall against exact K-NN on a seeded sample of query rows
    nq = min(args.recall_queries, N)
    queries = torch.from_numpy(np.random.default_rng(1).choice(N, nq, replace=False)).cuda()
    truth = exact_knn_sample(torch, dX, queries, K)
    approx = idx[queries].long()
    hits = (approx[:, :, None] == truth[:, None, :]).any(2).sum().item()
    recall = hits / float(nq * K)

    # the call the reference times (python/gpu_rsfk/RSFK.py:329,368: host arrays in, host arrays out)
    host_s = None
    if args.host_calls > 0:
        r = gpu_rsfk.RSFK(random_state=0)
        ts = []
        for _ in range(args.host_calls):
            r.find_nearest_neighbors(X, K, n_trees=T, min_tree_children=mn, max_tree_children=mx,
                                     nn_exploring_factor=args.explore)
            ts.append(r._last_search_time)
        host_s = float(min(ts))

    fls = [ForestLog(l) for l in logs]
    knn_s = float(np.mean([np.mean(f.data["KNN Sets Updates"]) for f in fls])) if fls and T > 0 else 0.0
    tree_s = float(np.mean([np.mean(f.data["Total Tree Building Time"]) for f in fls])) if fls and T > 0 else 0.0
    expl_s = float(np.mean([f.exploration_time for f in fls])) if fls else 0.0
    leaves = fls[0].data["Total Leaves"] if fls and T > 0 else []
    roofline = bucket_roofline(N, D, K, T, mn, mx, knn_s, leaves, report.get("bucket_kernels", []))
    roofline_tree = roofline_explore = None
    if T > 0 and report.get("tree_points_tested", 0) > 0:
        R = report["tree_screen_row_bytes"]
        tb = (report["tree_points_tested"] * (R + 16.0) + report["tree_points_undecided"] * 4.0 * D) / T + 4.0 * N
        ach = tb / tree_s / 1e9 if tree_s > 0 else 0.0
        roofline_tree = {"kernel": "tree build of one tree (k_pm_sweep / k_side, k_scatter, k_tail; trees are built in batches, level by level)",
                         "bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes_per_launch": round(tb),
                         "avg_launch_ms": round(tree_s * 1e3, 4), "launches_per_step": T,
                         "point_levels_per_point": round(report["tree_points_tested"] / float(T) / N, 3),
                         "undecided_share": round(report["tree_points_undecided"] / float(report["tree_points_tested"]), 5),
                         "screen_row_bytes": R,
                         "note": "bytes = sum over levels of the points of split nodes x (screening row + 16 for the permutation entry "
                                 "read and written by side test and scatter) + undecided points x 4 D + 4 N; time = host time of a "
                                 "batch of trees / trees"}
    if args.explore > 0 and report.get("explore_passes", 0) > 0:
        per_pass = report["explore_exact_distances"] / float(report["explore_passes"])
        eb = per_pass * 4.0 * D + float(N) * (4.0 * K * K + 16.0 * K)
        es = expl_s / report["explore_passes"]
        ach = eb / es / 1e9 if es > 0 else 0.0
        roofline_explore = {"kernel": "one exploration pass (reversed graph, join on the matrix cores, merge)", "bound": "hbm",
                            "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                            "traffic": None, "algorithmic_bytes_per_launch": round(eb), "avg_launch_ms": round(es * 1e3, 4),
                            "launches_per_step": report["explore_passes"],
                            "exact_distances_per_point": round(per_pass / N, 2),
                            "note": "bytes = N (U 4 D + 4 K^2 + 16 K), U = exact distances per point counted by the merge kernels"}
    cfg_name = next((name for name, c in CONFIGS.items()
                     if (args.workload, N, D, K, T, mn, mx, args.explore) == c), None)
    per_build = profiled_traffic(cfg_name) if T > 0 and cfg_name else None
    if per_build:
        roofline["traffic"] = round(per_build / T)
        roofline["note"] = ("traffic: HBM bytes per tree of the bucket K-NN kernels from the tracked rocprofv3 summary of this "
                            "command, made with the same kernel sources (profiles/%s: FETCH_SIZE x %.2f + WRITE_SIZE, all "
                            "bucket kernels of a build / trees)" % (PROFILE_FILES[cfg_name], FETCH_SCALE))
    elif cfg_name in PROFILE_FILES:
        roofline["note"] = ("traffic: null -- the tracked rocprofv3 summary (profiles/%s) was made with other sources of the "
                            "bucket kernels than this run's" % PROFILE_FILES[cfg_name])
    # what the device delivers when scattered rows of 4 D bytes are only read: every row of the matrix once, in a random
    # order, by rsfk_probe_gather_device (one wavefront per row, nothing computed); the bucket kernels gather the same
    # rows in the order of a tree's permutation and cannot be faster than this on their N 4 D bytes
    try:
        roofline["gather_probe"] = gather_probe(dX, N, D)
        if roofline.get("bound") == "hbm" and roofline["gather_probe"]["GB/s"] > 0:
            # the same achieved rate against what scattered rows of this size reach on the device
            roofline["frac_of_gather_rate"] = round(roofline["achieved"] / roofline["gather_probe"]["GB/s"], 4)
            roofline["frac_of_gather_rate_after_other_writes"] = round(
                roofline["achieved"] / roofline["gather_probe"]["GB/s_after_other_writes"], 4)
    except Exception as e:           # the probe is an aid: the line is valid without it
        roofline["gather_probe"] = {"error": str(e)}

    # CPU baseline: the oracle (a port of the reference algorithm, OpenMP) on the same workload -- whole with
    # --cpu-full, else on its first rows, as many as about 30 s of CPU time cover (the rate per point of a smaller
    # input is higher: shallower trees, same work per bucket)
    cpu = None
    if args.cpu_sample != 0:
        from oracle import rsfk_oracle as orc
        if args.cpu_full:
            ns = N
        elif args.cpu_sample > 0:
            ns = min(args.cpu_sample, N)
        else:
            per_point = T * (D * (0.75 * mx) * 1.5 + 40.0 * D) + args.explore * K * K * D * 0.6      # rough flop count
            ns = int(min(N, max(20000, 35.0 * 1.2e9 * orc.num_threads() / per_point)))
        Xs = np.ascontiguousarray(X[:ns])
        oi, od = orc.init_lists(ns, K)
        c0 = time.perf_counter()
        orc.forest(Xs, K, T, mn, mx, 5000, 0, args.explore, knn_idx=oi, knn_dist=od)
        cs = time.perf_counter() - c0
        cpu = {"value": round(ns / cs, 1), "unit": "points/s", "cores": orc.num_threads(), "kind": "port",
               "seconds": round(cs, 3),
               "sample": ("the whole workload" if ns == N else "first %d rows of the workload" % ns) +
                         ", same D, K, %d trees, %d exploration pass(es), OpenMP with %d threads" % (T, args.explore, orc.num_threads())}

    out = {
        "metric": "knng_build_points_per_sec",
        "value": round(N / sec_per_step, 1),
        "unit": "points/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec_per_step * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "%s%s N=%d D=%d K=%d n_trees=%d buckets=%d..%d exploration=%d seed=0" % (
            (args.config + " = ") if args.config else "", args.workload, N, D, K, T, mn, mx, args.explore)},
        "timed_region": "device-resident build: points and K-NN rows in HBM before and after (rsfk_knn_forest_device); "
                        "host_call_seconds is the region the reference times (host arrays in and out)",
        "build_seconds": round(sec_per_step, 5),
        "host_call_seconds": None if host_s is None else round(host_s, 5),
        "host_call_points_per_sec": None if host_s is None else round(N / host_s, 1),
        "recall_at_k": round(recall, 4),
        "recall_queries": nq,
        "phase_seconds": {"tree_build_per_tree": round(tree_s, 6), "bucket_knn_per_tree": round(knn_s, 6),
                          "exploration": round(expl_s, 6)},
        "roofline": roofline,
        "roofline_tree": roofline_tree,
        "roofline_explore": roofline_explore,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
