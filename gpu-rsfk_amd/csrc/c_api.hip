// extern "C" boundary of librsfk.so (declarations: include/rsfk.h).
#include "../../include/rsfk.h"
#include "forest.hpp"
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <vector>
#include <algorithm>

using namespace rsfk;

namespace {

[[noreturn]] void die(const char* where)
{
    // same convention as the reference: message on stderr, exit(1) (src/rsfk.cu:40-50)
    std::fprintf(stderr, "%s: %s\n", where, last_error());
    std::exit(1);
}

struct DevMem {
    void* p = nullptr;
    ~DevMem() { ws_free(p); }
    int alloc(size_t bytes) { return ws_alloc(&p, bytes); }
};

}  // namespace

extern "C" {

#define RSFK_API __attribute__((visibility("default")))

RSFK_API void pymodule_rsfk_knn(int n_trees, int num_neighbors, int N, int D, int MIN_TREE_CHILD,
                                int MAX_TREE_CHILD, int MAX_DEPTH, int VERBOSE, int RANDOM_STATE,
                                int nn_exploring_factor, float* points, int* knn_indices,
                                float* knn_sqr_distances, float* log_forest)
{
    if (knn_forest_host(n_trees, num_neighbors, N, D, MIN_TREE_CHILD, MAX_TREE_CHILD, MAX_DEPTH, VERBOSE,
                        RANDOM_STATE, nn_exploring_factor, points, knn_indices, knn_sqr_distances, log_forest))
        die("pymodule_rsfk_knn");
}

RSFK_API void pymodule_rsfk_knn_ann(int n_trees, int num_neighbors, int N, int NQ, int D, int MIN_TREE_CHILD,
                                    int MAX_TREE_CHILD, int MAX_DEPTH, int VERBOSE, int RANDOM_STATE,
                                    int /*nn_exploring_factor: accepted and ignored, as in the reference*/,
                                    float* points, float* query_points, int* knn_indices, float* knn_sqr_distances,
                                    float* log_forest)
{
    if (knn_ann_forest_host(n_trees, num_neighbors, N, NQ, D, MIN_TREE_CHILD, MAX_TREE_CHILD, MAX_DEPTH, VERBOSE,
                            RANDOM_STATE, points, query_points, knn_indices, knn_sqr_distances, log_forest))
        die("pymodule_rsfk_knn_ann");
}

RSFK_API void pymodule_cluster_by_sample_tree(int N, int D, int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH,
                                              int VERBOSE, int RANDOM_STATE, float* points, int** nodes_buckets,
                                              int** bucket_sizes, int* total_leaves, int* max_child)
{
    const auto t0 = std::chrono::steady_clock::now();
    std::vector<int> perm, ls, lz;
    int stats[5] = {0, 0, 0, 0, 0};
    {
        DevMem dp;
        if (N < 1 || D < 1) { set_last_error("N and D must be positive"); die("pymodule_cluster_by_sample_tree"); }
        if (dp.alloc(sizeof(float) * (size_t)N * (size_t)D)) die("pymodule_cluster_by_sample_tree");
        if (hipMemcpy(dp.p, points, sizeof(float) * (size_t)N * (size_t)D, hipMemcpyHostToDevice) != hipSuccess) {
            set_last_error("hipMemcpy of the points failed");
            die("pymodule_cluster_by_sample_tree");
        }
        if (build_tree_host(static_cast<const float*>(dp.p), N, D, MIN_TREE_CHILD, MAX_TREE_CHILD, MAX_DEPTH,
                            RANDOM_STATE, perm, ls, lz, stats))
            die("pymodule_cluster_by_sample_tree");
    }
    const int nl = stats[0], mc = stats[2];
    int* nb = static_cast<int*>(std::malloc(sizeof(int) * std::max<size_t>((size_t)nl * (size_t)mc, 1)));
    int* bs = static_cast<int*>(std::malloc(sizeof(int) * std::max<size_t>((size_t)nl, 1)));
    if (!nb || !bs) { set_last_error("out of host memory"); die("pymodule_cluster_by_sample_tree"); }
    for (int b = 0; b < nl; ++b) {
        bs[b] = lz[b];
        int* row = nb + (size_t)b * mc;
        for (int i = 0; i < lz[b]; ++i) row[i] = perm[(size_t)ls[b] + i];
        for (int i = lz[b]; i < mc; ++i) row[i] = -1;
    }
    *nodes_buckets = nb;
    *bucket_sizes = bs;
    *total_leaves = nl;
    *max_child = mc;
    if (VERBOSE >= 1) {
        const double dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        std::printf("Creating cluster with one tree takes %lf seconds\n", dt);
        if (VERBOSE >= 2) {
            std::printf("Tree depth: %d\nMax child count: %d\nMin child count: %d\nTotal leaves: %d\n", stats[1],
                        stats[2], stats[3], stats[0]);
        }
    }
}

RSFK_API int rsfk_knn_forest_device(int n_trees, int num_neighbors, int N, int D, int MIN_TREE_CHILD,
                                    int MAX_TREE_CHILD, int MAX_DEPTH, int VERBOSE, int RANDOM_STATE,
                                    int nn_exploring_factor, const float* d_points, int* d_knn_indices,
                                    float* d_knn_sqr_distances, float* log_forest, void* stream)
{
    return knn_forest_device(n_trees, num_neighbors, N, D, MIN_TREE_CHILD, MAX_TREE_CHILD, MAX_DEPTH, VERBOSE,
                             RANDOM_STATE, nn_exploring_factor, d_points, d_knn_indices, d_knn_sqr_distances,
                             log_forest, static_cast<hipStream_t>(stream));
}

RSFK_API int rsfk_knn_ann_device(int n_trees, int num_neighbors, int N, int NQ, int D, int MIN_TREE_CHILD,
                                 int MAX_TREE_CHILD, int MAX_DEPTH, int VERBOSE, int RANDOM_STATE,
                                 const float* d_points, const float* d_query_points, int* d_knn_indices,
                                 float* d_knn_sqr_distances, float* log_forest, void* stream)
{
    return knn_ann_forest_device(n_trees, num_neighbors, N, NQ, D, MIN_TREE_CHILD, MAX_TREE_CHILD, MAX_DEPTH, VERBOSE,
                                 RANDOM_STATE, d_points, d_query_points, d_knn_indices, d_knn_sqr_distances, log_forest,
                                 static_cast<hipStream_t>(stream));
}

RSFK_API int rsfk_knn_forest_fresh_host(int n_trees, int num_neighbors, int N, int D, int MIN_TREE_CHILD, int MAX_TREE_CHILD,
                                        int MAX_DEPTH, int VERBOSE, int RANDOM_STATE, int nn_exploring_factor,
                                        int point_in_self_neigh, const float* points, int* knn_indices,
                                        float* knn_sqr_distances, float* log_forest)
{
    return knn_forest_host(n_trees, num_neighbors, N, D, MIN_TREE_CHILD, MAX_TREE_CHILD, MAX_DEPTH, VERBOSE, RANDOM_STATE,
                           nn_exploring_factor, points, knn_indices, knn_sqr_distances, log_forest,
                           point_in_self_neigh ? 2 : 1);
}

RSFK_API int rsfk_symmetrize_device(const int* d_knn_indices, const float* d_knn_sqr_distances, int N, int num_neighbors,
                                    int drop_self, int* d_indptr, int* d_indices, float* d_data, long long capacity,
                                    long long* nnz, void* stream)
{
    return symmetrize_device(d_knn_indices, d_knn_sqr_distances, N, num_neighbors, drop_self, d_indptr, d_indices, d_data,
                             capacity, nnz, static_cast<hipStream_t>(stream));
}

RSFK_API int rsfk_symmetrize_count_noalloc(const int* d_knn_indices, int N, int num_neighbors, int drop_self,
                                           int* d_indptr, long long* nnz, void* stream)
{
    return symmetrize_count_noalloc(d_knn_indices, N, num_neighbors, drop_self, d_indptr, nnz, static_cast<hipStream_t>(stream));
}

RSFK_API int rsfk_symmetrize_host(const int* knn_indices, const float* knn_sqr_distances, int N, int num_neighbors,
                                  int drop_self, int* indptr, int* indices, float* data, long long capacity, long long* nnz)
{
    return symmetrize_host(knn_indices, knn_sqr_distances, N, num_neighbors, drop_self, indptr, indices, data, capacity, nnz);
}

RSFK_API int rsfk_bucket_knn_device(const float* d_points, int N, int D, int num_neighbors, const int* d_ids,
                                    const int* d_starts, const int* d_sizes, int n_buckets, int stride,
                                    int* d_knn_indices, float* d_knn_sqr_distances, void* stream)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (launch_bucket_knn(d_points, N, D, num_neighbors, d_ids, d_starts, d_sizes, n_buckets, stride, -1,
                          d_knn_indices, d_knn_sqr_distances, s))
        return 1;
    RSFK_HIP(hipStreamSynchronize(s));
    return 0;
}

RSFK_API int rsfk_explore_device(const float* d_points, int N, int D, int num_neighbors, int* d_knn_indices,
                                 float* d_knn_sqr_distances, int* d_scratch, void* stream)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    Bf16Copy bf;
    int rc = bf16_copy_alloc(&bf, N, D);
    if (!rc) rc = bf16_copy_fill(bf, d_points, N, D, s);
    ExploreWorkspace* ws = nullptr;
    Bf16Copy bfc;            // centred copy for the join
    if (!rc && explore_join_enabled(N, num_neighbors)) {
        rc = explore_ws_alloc(&ws, N, num_neighbors, explore_join_keeps_bounds(N, D, num_neighbors));
        if (!rc) rc = bf16_copy_alloc(&bfc, N, D, true);
        if (!rc) rc = bf16_copy_fill(bfc, d_points, N, D, s);
    }
    if (!rc) rc = launch_explore(d_points, &bf, &bfc, N, D, num_neighbors, d_knn_indices, d_knn_sqr_distances, d_scratch, ws, s);
    if (!rc && hipStreamSynchronize(s) != hipSuccess) { set_last_error("hipStreamSynchronize failed"); rc = 1; }
    explore_ws_free(ws);
    bf16_copy_free(&bfc);
    bf16_copy_free(&bf);
    return rc;
}

RSFK_API int rsfk_build_tree_host(const float* points, int N, int D, int MIN_TREE_CHILD, int MAX_TREE_CHILD,
                                  int MAX_DEPTH, int RANDOM_STATE, int* perm, int* leaf_start, int* leaf_size,
                                  int leaf_cap, int* stats)
{
    if (N < 1 || D < 1) { set_last_error("N and D must be positive"); return -2; }
    DevMem dp;
    if (dp.alloc(sizeof(float) * (size_t)N * (size_t)D)) return -1;
    if (hipMemcpy(dp.p, points, sizeof(float) * (size_t)N * (size_t)D, hipMemcpyHostToDevice) != hipSuccess) {
        set_last_error("hipMemcpy of the points failed");
        return -1;
    }
    std::vector<int> pv, ls, lz;
    int st[5];
    if (build_tree_host(static_cast<const float*>(dp.p), N, D, MIN_TREE_CHILD, MAX_TREE_CHILD, MAX_DEPTH,
                        RANDOM_STATE, pv, ls, lz, st))
        return -1;
    if (st[0] > leaf_cap) { set_last_error("leaf_cap too small"); return -3; }
    std::memcpy(perm, pv.data(), sizeof(int) * (size_t)N);
    std::memcpy(leaf_start, ls.data(), sizeof(int) * ls.size());
    std::memcpy(leaf_size, lz.data(), sizeof(int) * lz.size());
    if (stats) std::memcpy(stats, st, sizeof(int) * 4);
    return st[0];
}

RSFK_API int rsfk_bucket_knn_host(const float* points, int N, int D, int num_neighbors, const int* ids, int n_ids,
                                  const int* starts, const int* sizes, int n_buckets, int stride, int* knn_indices,
                                  float* knn_sqr_distances)
{
    RSFK_CHECK(N >= 1 && D >= 1 && num_neighbors >= 1 && n_buckets >= 0 && n_ids >= 0, "bad sizes");
    // host-side validation: every bucket must lie inside ids[] and every id inside [0,N)
    int max_bucket = 0;
    for (int b = 0; b < n_buckets; ++b) {
        max_bucket = std::max(max_bucket, sizes[b]);
        const long long st = starts ? (long long)starts[b] : (long long)b * stride;
        RSFK_CHECK(sizes[b] >= 0 && st >= 0 && st + sizes[b] <= n_ids, "bucket outside the id array");
        for (int i = 0; i < sizes[b]; ++i)
            RSFK_CHECK(ids[st + i] >= 0 && ids[st + i] < N, "point id out of range");
    }
    DevMem dp, di, dst, dsz, dki, dkd;
    const size_t nk = (size_t)N * (size_t)num_neighbors;
    if (dp.alloc(sizeof(float) * (size_t)N * (size_t)D) || di.alloc(sizeof(int) * (size_t)n_ids) ||
        dsz.alloc(sizeof(int) * (size_t)n_buckets) || dki.alloc(sizeof(int) * nk) || dkd.alloc(sizeof(float) * nk))
        return 1;
    if (starts && dst.alloc(sizeof(int) * (size_t)n_buckets)) return 1;
    RSFK_HIP(hipMemcpy(dp.p, points, sizeof(float) * (size_t)N * (size_t)D, hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(di.p, ids, sizeof(int) * (size_t)n_ids, hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(dsz.p, sizes, sizeof(int) * (size_t)n_buckets, hipMemcpyHostToDevice));
    if (starts) RSFK_HIP(hipMemcpy(dst.p, starts, sizeof(int) * (size_t)n_buckets, hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(dki.p, knn_indices, sizeof(int) * nk, hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(dkd.p, knn_sqr_distances, sizeof(float) * nk, hipMemcpyHostToDevice));
    if (launch_bucket_knn(static_cast<const float*>(dp.p), N, D, num_neighbors, static_cast<const int*>(di.p),
                          starts ? static_cast<const int*>(dst.p) : nullptr, static_cast<const int*>(dsz.p),
                          n_buckets, stride, max_bucket, static_cast<int*>(dki.p), static_cast<float*>(dkd.p), nullptr))
        return 1;
    RSFK_HIP(hipDeviceSynchronize());
    RSFK_HIP(hipMemcpy(knn_indices, dki.p, sizeof(int) * nk, hipMemcpyDeviceToHost));
    RSFK_HIP(hipMemcpy(knn_sqr_distances, dkd.p, sizeof(float) * nk, hipMemcpyDeviceToHost));
    return 0;
}

RSFK_API int rsfk_explore_host(const float* points, int N, int D, int num_neighbors, int* knn_indices,
                               float* knn_sqr_distances, int passes)
{
    RSFK_CHECK(N >= 1 && D >= 1 && num_neighbors >= 1 && passes >= 0, "bad sizes");
    DevMem dp, dki, dkd, dold;
    const size_t nk = (size_t)N * (size_t)num_neighbors;
    if (dp.alloc(sizeof(float) * (size_t)N * (size_t)D) || dki.alloc(sizeof(int) * nk) ||
        dkd.alloc(sizeof(float) * nk) || dold.alloc(sizeof(int) * nk))
        return 1;
    RSFK_HIP(hipMemcpy(dp.p, points, sizeof(float) * (size_t)N * (size_t)D, hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(dki.p, knn_indices, sizeof(int) * nk, hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(dkd.p, knn_sqr_distances, sizeof(float) * nk, hipMemcpyHostToDevice));
    Bf16Copy bf;
    int rc = bf16_copy_alloc(&bf, N, D);
    if (!rc) rc = bf16_copy_fill(bf, static_cast<const float*>(dp.p), N, D, nullptr);
    ExploreWorkspace* ws = nullptr;
    Bf16Copy bfc;            // centred copy for the join
    if (!rc && explore_join_enabled(N, num_neighbors)) {
        rc = explore_ws_alloc(&ws, N, num_neighbors, explore_join_keeps_bounds(N, D, num_neighbors));
        if (!rc) rc = bf16_copy_alloc(&bfc, N, D, true);
        if (!rc) rc = bf16_copy_fill(bfc, static_cast<const float*>(dp.p), N, D, nullptr);
    }
    for (int it = 0; it < passes && !rc; ++it)
        rc = launch_explore(static_cast<const float*>(dp.p), &bf, &bfc, N, D, num_neighbors, static_cast<int*>(dki.p),
                            static_cast<float*>(dkd.p), static_cast<int*>(dold.p), ws, nullptr);
    if (!rc && hipDeviceSynchronize() != hipSuccess) { set_last_error("hipDeviceSynchronize failed"); rc = 1; }
    explore_ws_free(ws);
    bf16_copy_free(&bfc);
    bf16_copy_free(&bf);
    if (rc) return rc;
    RSFK_HIP(hipDeviceSynchronize());
    RSFK_HIP(hipMemcpy(knn_indices, dki.p, sizeof(int) * nk, hipMemcpyDeviceToHost));
    RSFK_HIP(hipMemcpy(knn_sqr_distances, dkd.p, sizeof(float) * nk, hipMemcpyDeviceToHost));
    return 0;
}

RSFK_API const char* rsfk_last_error(void) { return last_error(); }

RSFK_API int rsfk_last_build_report(char* buf, int capacity) { return build_report_json(buf, capacity); }

RSFK_API void rsfk_release_workspace(void)
{
    ws_release_all();
    release_copy_buffers();
}

RSFK_API int rsfk_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

}  // extern "C"
