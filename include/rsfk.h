/*
 * rsfk.h -- C ABI of librsfk.so, the gfx950 (MI355X) implementation of RSFK
 * K-NN-graph construction.
 *
 * The first three functions are the entry points the gpu_rsfk Python package
 * binds with ctypes (python/gpu_rsfk/RSFK.py:112-168 of the reference); their
 * names, argument order and meaning are those of the reference's
 * src/python/pymodule_ext.cu:44-92.  The remaining functions expose the same
 * path with device-resident buffers and stage by stage; they return 0 on
 * success and a non-zero code otherwise (rsfk_last_error() has the text).
 *
 * Conventions: points are float32, row-major N x D.  K-NN state is int32 N x K
 * indices and float32 N x K squared distances, same slot <-> same neighbour,
 * rows unordered, empty slot = (-1, +inf or FLT_MAX).  The library merges into
 * whatever the K-NN arrays hold on entry; it never resets them.
 * All calls use the current HIP device and block until their results are
 * complete.  K is limited to 1024.
 */
#ifndef RSFK_H
#define RSFK_H

#ifdef __cplusplus
extern "C" {
#endif

/* ---- entry points of the reference's shared library -------------------- */

/* K-NN graph of `points` with a forest of n_trees random-sample trees followed
 * by nn_exploring_factor exploration passes.  Host buffers.
 * Replaces pymodule_rsfk_knn (src/python/pymodule_ext.cu:124-147 ->
 * RSFK::knn_gpu_rsfk_forest, src/rsfk.cu:2033-2183).  Tree t uses seed
 * RANDOM_STATE + t (src/rsfk.cu:2087).  log_forest: 16*n_trees+2 floats,
 * series-major (src/rsfk.cu:2148-2173).  On a device error the message goes to
 * stderr and the process exits with status 1 (src/rsfk.cu:40-50). */
void pymodule_rsfk_knn(int n_trees, int num_neighbors, int N, int D,
                       int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH,
                       int VERBOSE, int RANDOM_STATE, int nn_exploring_factor,
                       float* points, int* knn_indices, float* knn_sqr_distances,
                       float* log_forest);

/* Query-set search.  Replaces pymodule_rsfk_knn_ann (src/python/pymodule_ext.cu:149-181 ->
 * RSFK::knn_gpu_rsfk_forest_ann, src/rsfk.cu:98-498): n_trees trees are built on `points`
 * (tree t with seed RANDOM_STATE + t); per tree every query point is routed to a leaf and
 * the points of that leaf are merged into the query's row.  knn_indices / knn_sqr_distances
 * are NQ x num_neighbors, in/out (merged into, -1 / +inf = empty), indices refer to
 * `points`.  nn_exploring_factor is accepted and ignored, as in the reference.
 * log_forest: 16*n_trees+2 floats (series of pymodule_rsfk_knn; entry 16*n_trees = total
 * seconds).  Errors: message on stderr, exit(1). */
void pymodule_rsfk_knn_ann(int n_trees, int num_neighbors, int N, int NQ, int D,
                           int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH,
                           int VERBOSE, int RANDOM_STATE, int nn_exploring_factor,
                           float* points, float* query_points,
                           int* knn_indices, float* knn_sqr_distances, float* log_forest);

/* Partition of the points by one random-sample tree.
 * Replaces pymodule_cluster_by_sample_tree (src/python/pymodule_ext.cu:183-212 ->
 * RSFK::cluster_by_sample_tree, src/rsfk.cu:2185-2228).
 * *nodes_buckets = malloc'ed int[total_leaves*max_child], row b = the ids of
 * bucket b padded with -1; *bucket_sizes = malloc'ed int[total_leaves].  The
 * caller owns both (free()).  Buckets are ordered by their position in the
 * tree (left to right), ids inside a bucket ascend. */
void pymodule_cluster_by_sample_tree(int N, int D,
                                     int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH,
                                     int VERBOSE, int RANDOM_STATE,
                                     float* points,
                                     int** nodes_buckets, int** bucket_sizes,
                                     int* total_leaves, int* max_child);

/* ---- the same path, device-resident ------------------------------------ */

/* As pymodule_rsfk_knn but points / knn_indices / knn_sqr_distances are device
 * pointers (log_forest stays a host pointer, may be NULL) and `stream` is a
 * hipStream_t (NULL = default stream).  Replaces the body of
 * RSFK::knn_gpu_rsfk_forest between its host-to-device and device-to-host
 * copies (src/rsfk.cu:2073-2135). */
int rsfk_knn_forest_device(int n_trees, int num_neighbors, int N, int D,
                           int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH,
                           int VERBOSE, int RANDOM_STATE, int nn_exploring_factor,
                           const float* d_points, int* d_knn_indices, float* d_knn_sqr_distances,
                           float* log_forest, void* stream);

/* pymodule_rsfk_knn_ann with device-resident buffers (points N x D, queries NQ x D, rows
 * NQ x num_neighbors); log_forest is host memory or NULL.  Replaces the body of
 * RSFK::knn_gpu_rsfk_forest_ann between its copies (src/rsfk.cu:117-128).  Returns 0, or
 * nonzero with the reason in rsfk_last_error(). */
int rsfk_knn_ann_device(int n_trees, int num_neighbors, int N, int NQ, int D,
                        int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH,
                        int VERBOSE, int RANDOM_STATE,
                        const float* d_points, const float* d_query_points,
                        int* d_knn_indices, float* d_knn_sqr_distances,
                        float* log_forest, void* stream);

/* Bucket K-NN over a given partition, device pointers.  Bucket b holds
 * d_ids[start_b .. start_b + d_sizes[b]) with start_b = d_starts ? d_starts[b]
 * : b*stride (stride = max_child of the padded bucket matrix).  Replaces
 * RSFK::update_knn_indice_with_buckets and the kernel it launches
 * (src/rsfk.cu:1967-2030, src/kernels/compute_knn_from_buckets.cu:998-1378). */
int rsfk_bucket_knn_device(const float* d_points, int N, int D, int num_neighbors,
                           const int* d_ids, const int* d_starts, const int* d_sizes,
                           int n_buckets, int stride,
                           int* d_knn_indices, float* d_knn_sqr_distances, void* stream);

/* One exploration pass, device pointers; d_scratch holds N*K ints (it receives
 * the snapshot of the indices).  Replaces one iteration of the loop at
 * src/rsfk.cu:2117-2131 (nearest_neighbors_exploring,
 * src/kernels/nearest_neighbors_exploring.cu:41-146). */
int rsfk_explore_device(const float* d_points, int N, int D, int num_neighbors,
                        int* d_knn_indices, float* d_knn_sqr_distances, int* d_scratch, void* stream);

/* Symmetrised K-NN graph in compressed-row (CSR) form, device pointers: row p holds every neighbour stored for p and
 * every point that stores p, each once, with the squared distance of the pair; columns ascend inside a row.
 * d_indptr: N + 1 ints.  d_indices / d_data: room for `capacity` entries (2 * N * num_neighbors always suffices), or both
 * NULL to obtain d_indptr and *nnz only.  Slots that are negative or >= N are no edges; drop_self != 0 removes p from
 * its own row; d_knn_sqr_distances may be NULL (data is then zero).  A row must not hold a point twice.  Replaces the
 * kernels the reference keeps commented out beside its spectral experiment (symmetric_knn_graph_edge_count,
 * symmetric_knn_graph_offset, symmetric_knn_graph_add_edges, src/rsfk.cu:1229-1299). */
int rsfk_symmetrize_device(const int* d_knn_indices, const float* d_knn_sqr_distances, int N, int num_neighbors,
                           int drop_self, int* d_indptr, int* d_indices, float* d_data, long long capacity,
                           long long* nnz, void* stream);

/* The count-only form of rsfk_symmetrize_device (d_indices = d_data = NULL there): fills d_indptr (N + 1 ints) and *nnz
 * with the row offsets and the number of entries of the symmetrised graph.  It has no counterpart in the reference.
 * It is for callers that cannot allocate device memory -- tight serving loops, harnesses that forbid hipMalloc, code
 * that records a HIP graph: it calls no hipMalloc, hipFree or other allocating routine.  With nnz != NULL it ends with
 * a copy of the count to the host and a synchronisation of the stream (not allowed on a stream under capture); with
 * nnz == NULL it only enqueues kernels and the count is d_indptr[N] on the device.  Its working memory
 * (edge flags, per-point counters, the temporary storage of the prefix sum) is a fixed array of 45 MiB that every GPU
 * the library runs on holds until the process ends.  Limits: N <= 2^20 and N * num_neighbors <= 2^25; larger inputs
 * are refused with an error.  All calls on one GPU share the array, so calls that overlap on one GPU (other
 * streams, other threads) race; calls on one stream, or serialised by the caller, are safe. */
int rsfk_symmetrize_count_noalloc(const int* d_knn_indices, int N, int num_neighbors, int drop_self,
                                  int* d_indptr, long long* nnz, void* stream);

/* ---- stage-level calls with host buffers (copies in and out) ------------ */

/* One tree (RSFK::create_bucket_from_sample_tree, src/rsfk.cu:500-1207).
 * perm[N] receives the ids grouped by bucket; leaf_start/leaf_size (capacity
 * leaf_cap) the buckets in ascending start order; stats[4] = {number of
 * buckets, number of levels, largest bucket, smallest bucket}.  Returns the
 * number of buckets or a negative value on error. */
int rsfk_build_tree_host(const float* points, int N, int D,
                         int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH, int RANDOM_STATE,
                         int* perm, int* leaf_start, int* leaf_size, int leaf_cap, int* stats);

/* rsfk_bucket_knn_device with host buffers; n_ids = length of ids. */
int rsfk_bucket_knn_host(const float* points, int N, int D, int num_neighbors,
                         const int* ids, int n_ids, const int* starts, const int* sizes,
                         int n_buckets, int stride,
                         int* knn_indices, float* knn_sqr_distances);

/* pymodule_rsfk_knn for rows that start empty (point_in_self_neigh = 0) or with the point itself at distance 0 in
 * slot 0 (!= 0), which is how RSFK.find_nearest_neighbors prepares them (python/gpu_rsfk/RSFK.py:330-335): the rows
 * are made on the device, knn_indices / knn_sqr_distances are only written, and a third of the bytes of the call
 * stay off the PCIe bus.  Returns 0, or nonzero with the reason in rsfk_last_error(). */
int rsfk_knn_forest_fresh_host(int n_trees, int num_neighbors, int N, int D,
                               int MIN_TREE_CHILD, int MAX_TREE_CHILD, int MAX_DEPTH,
                               int VERBOSE, int RANDOM_STATE, int nn_exploring_factor, int point_in_self_neigh,
                               const float* points, int* knn_indices, float* knn_sqr_distances, float* log_forest);

/* rsfk_symmetrize_device with host buffers. */
int rsfk_symmetrize_host(const int* knn_indices, const float* knn_sqr_distances, int N, int num_neighbors,
                         int drop_self, int* indptr, int* indices, float* data, long long capacity, long long* nnz);

/* `passes` exploration passes with host buffers. */
int rsfk_explore_host(const float* points, int N, int D, int num_neighbors,
                      int* knn_indices, float* knn_sqr_distances, int passes);

/* ---- misc --------------------------------------------------------------- */

/* text of the last error of a call that returned non-zero */
const char* rsfk_last_error(void);

/* What the last K-NN-graph build of this process did (pymodule_rsfk_knn, rsfk_knn_forest_device, ...), as one line
 * of JSON written to buf (at most capacity - 1 characters and a final zero); returns the length of the whole text.
 * Keys: "bucket_kernels" (runs of trees [first, last, [kernel names]] -- which kernels the buckets of those trees
 * went to), "tree_points_tested" (sum over all trees and levels of the members of the nodes that were split),
 * "tree_points_undecided" (those the low-precision screen left to the exact fp32 test), "tree_screen_row_bytes",
 * "explore_exact_distances" (exact distances of all exploration passes), and the seconds of the three steps.  The
 * reference prints its phase times (src/rsfk.cu:1164-1176) and has no counterpart for the counts; bench.py computes
 * the algorithmic bytes of the tree build and of the exploration from them. */
int rsfk_last_build_report(char* buf, int capacity);

/* The library keeps the device buffers of a call (permutations, screening copies, exploration workspace) for the
 * next call instead of returning them to the driver; this returns all idle ones.  No counterpart in the
 * reference, which allocates and frees inside every tree level (src/rsfk.cu:640-1180). */
void rsfk_release_workspace(void);

/* number of HIP devices visible to the library (0 when there is none) */
int rsfk_device_count(void);

#ifdef __cplusplus
}
#endif
#endif /* RSFK_H */
