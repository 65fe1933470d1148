// Internal interfaces between the translation units of the library.
#pragma once
#include "rsfk_common.hpp"
#include "bf16.hpp"
#include <vector>

namespace rsfk {

struct TreeBatchWorkspace;

// tree_build.hip
size_t tree_ws_bytes(int N, int D, int MIN, int B);
int tree_ws_alloc(TreeBatchWorkspace** out, int N, int D, int MIN, int B);
void tree_ws_free(TreeBatchWorkspace* w);
int tree_ws_enable_index(TreeBatchWorkspace* w, int MIN, int MAX_DEPTH);
const TreeRec* tree_ws_recs(const TreeBatchWorkspace* w, int t);
int tree_ws_leaf_cap(const TreeBatchWorkspace* w);
const int* tree_ws_perm(const TreeBatchWorkspace* w, int t);
const int* tree_ws_leaf_start(const TreeBatchWorkspace* w, int t);
const int* tree_ws_leaf_size(const TreeBatchWorkspace* w, int t);
int tree_small_threshold(int D, int N, int B);
const float* tree_ws_phase_seconds(const TreeBatchWorkspace* w);
const unsigned long long* tree_ws_counts(const TreeBatchWorkspace* w);
int tree_screen_row_bytes(int D, bool q8);
int build_tree_batch(TreeBatchWorkspace* w, const float* points, const uint16_t* pb16, const uint8_t* q8, int N, int D,
                     int MIN, int MAX,
                     int MAX_DEPTH, int seed0, int nb, int* host_stats, hipStream_t stream);

// bucket_knn.hip
int launch_bucket_knn(const float* points, int N, int D, int K, const int* ids, const int* starts,
                      const int* sizes, int n_buckets, int stride, int max_bucket, int* knn_idx, float* knn_dist,
                      hipStream_t stream);

// bucket_knn_gram.hip
int launch_bucket_knn_gram(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                           int n_buckets, int stride, int min_size, int max_size, int* knn_idx, float* knn_dist,
                           hipStream_t stream);
// trees from this index on take the kernel that screens the pair matrix on the matrix cores (RSFK_GRAM_FROM)
int bucket_gram_from();

// Kernels a tree's buckets can go to (bits of *launched of launch_bucket_knn_tree, and of the report of a build)
enum : int {
    kBucketKernelSmall = 1,      // k_bucket_knn_small<64>: two wavefronts per bucket of up to 64 points, every pair exact
    kBucketKernelScreen = 2,     // k_bucket_knn_screen: the same with the pair matrix bounded on the matrix cores first
    kBucketKernelAuto = 128,     // k_bucket_knn_auto: one of the two, chosen on the device from the previous tree's pairs
    kBucketKernelMedium = 4,     // k_bucket_knn_small<72>: three wavefronts, buckets of 65..72 points
    kBucketKernelRows = 8,       // k_bucket_knn_rows: a bucket's points resident in LDS
    kBucketKernelTiled = 16,     // k_bucket_knn<SL, false>: 64 x 64 tiles, a workgroup per bucket
    kBucketKernelStrip = 32,     // k_bucket_knn<SL, true>: 64 x 64 tiles, a workgroup per 64 members of a bucket
    kBucketKernelGram = 64,      // k_bucket_knn_gram: any bucket size, pair matrix bounded on the matrix cores
    kBucketKernelPairs = 256,    // k_bucket_pairs + k_bucket_merge_pairs: 64 x 64 tiles, every pair once, distances through memory
};
// Working memory of k_bucket_pairs / k_bucket_merge_pairs: the pair matrices of as many buckets as fit are in it at a
// time.  One per stream of launches; p == null: the forms of the general kernel that need none are taken.
struct PairScratch {
    float* p = nullptr;
    size_t floats = 0;
};
// Floats of working memory the buckets of a launch would like (0: none of them reaches the general kernel, or the
// form is switched off); at most pair_scratch_max() (512 MB; RSFK_BUCKET_PAIRS_MB overrides), the launch then goes in
// several parts.
size_t pair_scratch_max();
size_t bucket_pairs_scratch_floats(int D, int K, int n_buckets, int max_bucket);
int launch_bucket_knn_tree(const float* points, const unsigned long long* prev_stats, unsigned long long* stats,
                           bool rows_sorted, bool gram, int D, int K, const int* ids, const int* starts, const int* sizes,
                           int leaf_cap, int n_small, int n_big, int max_bucket, int* knn_idx, float* knn_dist,
                           hipStream_t stream, int part = 0, bool young_rows = true, int* launched = nullptr,
                           const PairScratch* pairs = nullptr);

// What the last K-NN-graph build of this process did, as a line of JSON (rsfk_last_build_report): which bucket
// kernels every tree went to, the counts the algorithmic bytes of the tree build and of the exploration are made of,
// and the time of each of the three steps.  Returns the length of the text (without the final zero), which is
// truncated to cap - 1 characters.
int build_report_json(char* buf, int cap);

// bucket_knn_screen.hip
int launch_sort_rows(int* knn_idx, float* knn_dist, int N, int K, hipStream_t stream);
int launch_bucket_knn_screen(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                             int n_buckets, int stride, int* knn_idx, float* knn_dist, hipStream_t stream);
// Buckets of up to 64 points of one tree of a forest, the form of the kernel (every pair exact, or bounded on the matrix
// cores first) chosen on the device from the numbers of pairs the tree before left in prev (8 words; null: first tree);
// stats: 8 zeroed words for this tree's numbers.
int launch_bucket_knn_auto(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                           int n_buckets, int* knn_idx, float* knn_dist, const unsigned long long* prev,
                           unsigned long long* stats, hipStream_t stream);
// share of the pairs (in 1 / 65536) below which the screened form is taken (RSFK_BUCKET_SCREEN); kScreenAlways: always
constexpr unsigned int kScreenAlways = 0xffffffffu;
unsigned int bucket_screen_share_q16();

// bucket_knn_rows.hip
int bucket_rows_cap(int D, int K);
int launch_bucket_knn_rows(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes, int n_buckets,
                           int stride, int min_size, int max_size, bool rows_sorted, bool young_rows, int* knn_idx,
                           float* knn_dist, hipStream_t stream);

// bucket_knn_small.hip
int small_bucket_cap();
int medium_bucket_cap();
int launch_bucket_knn_medium(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                             int n_buckets, int stride, bool rows_sorted, int* knn_idx, float* knn_dist, hipStream_t stream);
int launch_bucket_knn_small(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                            int n_buckets, int stride, bool rows_sorted, int* knn_idx, float* knn_dist, hipStream_t stream);

// host_copy.hip: pageable host memory <-> device memory through pinned buffers, on several threads
int copy_to_device(void* dev_ptr, const void* host_ptr, size_t bytes);
int copy_to_host(void* host_ptr, const void* dev_ptr, size_t bytes);
void release_copy_buffers();

// explore_join.hip
struct ExploreWorkspace;
bool explore_join_enabled(int N, int K);
bool explore_merge_fits(int D, int K);
size_t explore_ws_bytes(int N, int K);
int explore_ws_alloc(ExploreWorkspace** out, int N, int K, bool with_bounds = false);
void explore_ws_free(ExploreWorkspace* w);
const uint32_t* explore_ws_pass(const ExploreWorkspace* w);
const uint16_t* explore_ws_bounds(const ExploreWorkspace* w);
int* explore_ws_todo(ExploreWorkspace* w, int which);
int* explore_ws_host_count(ExploreWorkspace* w);
// order: null, or a permutation of the points that keeps nearby points together (the buckets of a tree): the points
// are then worked on in that order, a contiguous eighth of it per die (die_local_place)
int launch_explore_join(ExploreWorkspace* w, const Bf16Copy& bf, int N, int D, int K, const int* old_idx,
                        const float* knn_dist, hipStream_t stream, const int* order = nullptr);

// explore.hip
// true when rows of K neighbours of D-dimensional points get the merge kernel that takes a point's candidates in the
// order of their lower bounds (the workspace should then be allocated with room for the bounds)
bool explore_merge_uses_bounds(int D, int K);
bool explore_join_keeps_bounds(int N, int D, int K);
int launch_explore(const float* points, const Bf16Copy* bf, const Bf16Copy* bf_join, int N, int D, int K, int* knn_idx,
                   float* knn_dist, int* old_idx, ExploreWorkspace* ws, hipStream_t stream, bool rows_sorted = false,
                   unsigned long long* stat = nullptr,       // stat: kExploreStatWords words, or null (count_exact)
                   const int* order = nullptr);              // order: see launch_explore_join
constexpr int kExploreStatWords = 32 * 256;

// graph_export.hip
int symmetrize_device(const int* d_idx, const float* d_dist, int N, int K, int drop_self, int* d_indptr, int* d_cols,
                      float* d_vals, long long cap, long long* nnz, hipStream_t stream);
// Count-only form of symmetrize_device (d_indptr and *nnz) whose working memory is a fixed device array of the
// library: no allocation of any kind.  At most 2^20 points and 2^25 slots.
int symmetrize_count_noalloc(const int* d_idx, int N, int K, int drop_self, int* d_indptr, long long* nnz, hipStream_t stream);
int symmetrize_host(const int* idx, const float* dist, int N, int K, int drop_self, int* indptr, int* cols, float* vals,
                    long long cap, long long* nnz);

// ann.hip
size_t ann_ws_ints(int NQ, int rec_cap);
int ann_plane_pitch(int D);
int launch_ann_ws_init(int* ws, int NQ, int rec_cap, hipStream_t stream);
int launch_ann_tree(const float* points, const float* queries, int NQ, int D, int K, const int* perm, const TreeRec* recs,
                    const int* n_rec_dev, int rec_cap, int n_leaves, int* ws, float* planes, int* q_idx, float* q_dist,
                    hipStream_t stream);
int knn_ann_forest_device(int n_trees, int K, int N, int NQ, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                          const float* d_points, const float* d_queries, int* d_qidx, float* d_qdist, float* log_forest,
                          hipStream_t stream);
int knn_ann_forest_host(int n_trees, int K, int N, int NQ, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                        const float* points, const float* queries, int* q_idx, float* q_dist, float* log_forest);
int tree_ws_rec_cap(const TreeBatchWorkspace* w);
const int* tree_ws_n_rec(const TreeBatchWorkspace* w, int t);     // device address of the number of records of tree t
int knn_forest_device(int n_trees, int K, int N, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                      int nnef, const float* d_points, int* d_idx, float* d_dist, float* log_forest,
                      hipStream_t stream);
int knn_forest_host(int n_trees, int K, int N, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                    int nnef, const float* points, int* knn_idx, float* knn_dist, float* log_forest, int fresh_rows = 0);
int build_tree_host(const float* d_points, int N, int D, int MIN, int MAX, int MAX_DEPTH, int seed,
                    std::vector<int>& perm, std::vector<int>& leaf_start, std::vector<int>& leaf_size, int stats[5]);

}  // namespace rsfk
