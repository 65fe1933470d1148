// Host orchestration: the forest loop (trees -> bucket K-NN), the exploration
// passes, the per-tree log and the single-tree clustering call.  Replaces
// RSFK::knn_gpu_rsfk_forest (src/rsfk.cu:2033-2183), RSFK::cluster_by_sample_tree
// (src/rsfk.cu:2185-2228) and RSFK::update_knn_indice_with_buckets
// (src/rsfk.cu:1967-2030).
//
// Differences in schedule: trees are built in batches (all trees of a batch
// advance one level per launch), device memory is allocated once per call, and
// the host synchronises once per tree level of a batch instead of after every
// kernel.
#include "forest.hpp"
#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

namespace rsfk {

namespace {
std::mutex g_err_mutex;
std::string g_last_error;
}  // namespace

void set_last_error(const std::string& msg)
{
    std::lock_guard<std::mutex> lock(g_err_mutex);
    g_last_error = msg;
}
const char* last_error()
{
    std::lock_guard<std::mutex> lock(g_err_mutex);
    return g_last_error.c_str();
}

namespace {

// the last build of this process (knn_forest_device), for build_report_json
struct BuildReport {
    int N = 0, D = 0, K = 0, n_trees = 0, passes = 0, row_bytes = 0;
    std::vector<int> kernels;                          // per tree: kBucketKernel... bits
    std::vector<unsigned long long> pairs;             // per tree: pairs of its small buckets << 32 | those evaluated exactly
    unsigned int screen_share_q16 = 0;
    unsigned long long tested = 0, undecided = 0;      // tree build: point-levels, and those left to the exact test
    unsigned long long exact = 0;                      // exploration: exact distances over all passes
    double tree_s = 0.0, bucket_s = 0.0, explore_s = 0.0;
};
std::mutex g_report_mutex;
BuildReport g_report;

double now_s()
{
    return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// how many trees to build per batch: as many as fit in a quarter of the free memory
int choose_batch(int n_trees, int N, int D, int MIN)
{
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) free_b = (size_t)8 << 30;
    const size_t budget = free_b / 4;
    int B = std::min(n_trees, 64);
    if (const char* e = std::getenv("RSFK_TREE_BATCH")) B = std::min(B, std::max(1, std::atoi(e)));     // for tests
    while (B > 1 && tree_ws_bytes(N, D, MIN, B) > budget) --B;
    return std::max(B, 1);
}

struct WsGuard {
    TreeBatchWorkspace* w = nullptr;
    ~WsGuard() { tree_ws_free(w); }
};
struct DevBuf {
    void* p = nullptr;
    ~DevBuf() { ws_free(p); }
};
// second stream (default priority) and the event that tells the caller's stream when its work is done
struct SideStream {
    hipStream_t side = nullptr;
    hipEvent_t big = nullptr;
    int open()
    {
        RSFK_HIP(hipStreamCreateWithFlags(&side, hipStreamNonBlocking));
        RSFK_HIP(hipEventCreateWithFlags(&big, hipEventDisableTiming));
        return 0;
    }
    ~SideStream()
    {
        if (side) { (void)hipStreamSynchronize(side); (void)hipStreamDestroy(side); }
        if (big) (void)hipEventDestroy(big);
    }
};
struct Bf16Guard {
    Bf16Copy c;
    ~Bf16Guard() { bf16_copy_free(&c); }
};
struct ExploreWsGuard {
    ExploreWorkspace* w = nullptr;
    ~ExploreWsGuard() { explore_ws_free(w); }
};
struct Q8Guard {
    Q8Copy c;
    ~Q8Guard() { q8_copy_free(&c); }
};
// An event with a time stamp; released when the owner goes out of scope, on every path.
struct TimedEvent {
    hipEvent_t e = nullptr;
    TimedEvent() = default;
    TimedEvent(const TimedEvent&) = delete;
    TimedEvent& operator=(const TimedEvent&) = delete;
    TimedEvent(TimedEvent&& o) noexcept : e(o.e) { o.e = nullptr; }
    int create()
    {
        RSFK_HIP(hipEventCreate(&e));
        return 0;
    }
    ~TimedEvent()
    {
        if (e) (void)hipEventDestroy(e);
    }
};

// Side tests of the trees are screened on the 8-bit copy when its quantisation error is within a small factor
// of the bfloat16 rounding error on these points (half the bytes per row), else on the bfloat16 copy.
// RSFK_TREE_SCREEN=q8 / bf16 forces one of them.  *rows = the 8-bit rows, or null for the bfloat16 screen.
int make_tree_screen(Q8Guard& q8, const float* d_points, int N, int D, int verbose, hipStream_t stream, const uint8_t** rows)
{
    *rows = nullptr;
    const char* env_tree = std::getenv("RSFK_TREE_SCREEN");
    const bool force_bf16 = env_tree && env_tree[0] == 'b';
    const bool force_q8 = env_tree && env_tree[0] == 'q';
    if (force_bf16) return 0;
    if (q8_copy_alloc(&q8.c, N, D) || q8_copy_fill(q8.c, d_points, N, D, stream)) return 1;
    float rho = 0.0f;
    if (q8_copy_mean_rho(q8.c, N, &rho, stream)) return 1;
    if (force_q8 || rho <= 6.0f) *rows = q8.c.rows;
    if (verbose >= 2)
        std::printf("8-bit copy: quantisation error %.2f x bfloat16 rounding error -> %s screen\n", rho,
                    *rows ? "8-bit" : "bfloat16");
    return 0;
}

}  // namespace

int build_report_json(char* buf, int cap)
{
    BuildReport r;
    {
        std::lock_guard<std::mutex> lock(g_report_mutex);
        r = g_report;
    }
    static const struct { int bit; const char* name; } names[] = {
        {kBucketKernelSmall, "k_bucket_knn_small<64>"}, {kBucketKernelScreen, "k_bucket_knn_screen"},
        {kBucketKernelMedium, "k_bucket_knn_small<72>"}, {kBucketKernelRows, "k_bucket_knn_rows"},
        {kBucketKernelTiled, "k_bucket_knn<per bucket>"}, {kBucketKernelStrip, "k_bucket_knn<per 64 members>"},
        {kBucketKernelGram, "k_bucket_knn_gram"}, {kBucketKernelAuto, "k_bucket_knn_auto"},
        {kBucketKernelPairs, "k_bucket_pairs + k_bucket_merge_pairs"}};
    std::string s = "{";
    auto num = [&](const char* key, double v, bool last = false) {
        char t[96];
        std::snprintf(t, sizeof t, "\"%s\": %.9g%s", key, v, last ? "" : ", ");
        s += t;
    };
    num("N", r.N); num("D", r.D); num("K", r.K); num("n_trees", r.n_trees);
    // runs of trees that went to the same kernels: [first tree, last tree, [names]]
    s += "\"bucket_kernels\": [";
    for (size_t a = 0; a < r.kernels.size();) {
        size_t b = a;
        while (b + 1 < r.kernels.size() && r.kernels[b + 1] == r.kernels[a]) ++b;
        if (a) s += ", ";
        s += "[" + std::to_string(a) + ", " + std::to_string(b) + ", [";
        bool first = true;
        for (const auto& nm : names)
            if (r.kernels[a] & nm.bit) { s += std::string(first ? "\"" : ", \"") + nm.name + "\""; first = false; }
        s += "]]";
        a = b + 1;
    }
    s += "], ";
    // k_bucket_knn_auto: share of the pairs of a tree's small buckets that had to be evaluated exactly, and the form of
    // the kernel that share selected for the next tree (the first tree takes the direct form)
    s += "\"bucket_pair_share\": [";
    for (size_t t = 0; t < r.pairs.size(); ++t) {
        const double total = (double)(r.pairs[t] >> 32), listed = (double)(r.pairs[t] & 0xffffffffull);
        char tmp[32];
        std::snprintf(tmp, sizeof tmp, "%s%.4f", t ? ", " : "", total > 0 ? listed / total : 0.0);
        s += tmp;
    }
    s += "], \"bucket_screened\": [";
    for (size_t t = 0; t < r.pairs.size(); ++t) {
        bool scr = r.screen_share_q16 == kScreenAlways;
        if (t > 0 && !scr) {
            const unsigned long long total = r.pairs[t - 1] >> 32, listed = r.pairs[t - 1] & 0xffffffffull;
            scr = total > 0 && (listed << 16) < total * r.screen_share_q16;
        }
        s += std::string(t ? ", " : "") + ((r.kernels[t] & kBucketKernelAuto) && scr ? "1" : "0");
    }
    s += "], ";
    num("bucket_screen_share", r.screen_share_q16 == kScreenAlways ? 2.0 : r.screen_share_q16 / 65536.0);
    num("tree_points_tested", (double)r.tested); num("tree_points_undecided", (double)r.undecided);
    num("tree_screen_row_bytes", r.row_bytes); num("tree_seconds", r.tree_s); num("bucket_seconds", r.bucket_s);
    num("explore_passes", r.passes); num("explore_exact_distances", (double)r.exact);
    num("explore_seconds", r.explore_s, true);
    s += "}";
    if (buf && cap > 0) {
        const size_t n = std::min(s.size(), (size_t)cap - 1);
        std::memcpy(buf, s.data(), n);
        buf[n] = 0;
    }
    return (int)s.size();
}

int knn_forest_device(int n_trees, int K, int N, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                      int nnef, const float* d_points, int* d_idx, float* d_dist, float* log_forest,
                      hipStream_t stream)
{
    RSFK_CHECK(N >= 1 && D >= 1 && K >= 1, "forest: N, D and K must be positive");
    RSFK_CHECK(n_trees >= 0, "forest: n_trees must not be negative");
    RSFK_CHECK(K <= kMaxK, "forest: K above 1024 is not supported");
    if (log_forest) std::memset(log_forest, 0, sizeof(float) * ((size_t)16 * n_trees + 2));
    if (n_trees == 0 && nnef <= 0) return 0;          // nothing to do: no copies are made, nothing is queued
    const double t_forest0 = now_s();
    BuildReport rep;
    rep.N = N; rep.D = D; rep.K = K; rep.n_trees = n_trees; rep.passes = std::max(nnef, 0);
    rep.kernels.assign((size_t)n_trees, 0);

    Q8Guard q8;
    const uint8_t* q8_rows = nullptr;
    if (n_trees > 0 && make_tree_screen(q8, d_points, N, D, verbose, stream, &q8_rows)) return 1;
    // The permutation of the last tree (points grouped by bucket) is kept for the exploration: points of a bucket are
    // close to each other and share neighbours, so working on them one after the other on the same die finds the rows
    // of those neighbours in its L2.
    // (RSFK_EXPLORE_ORDER=0: the points in their own order)
    DevBuf order;
    const char* order_env = std::getenv("RSFK_EXPLORE_ORDER");
    const bool in_bucket_order = !(order_env && order_env[0] == '0');
    if (n_trees > 0 && nnef > 0 && in_bucket_order && ws_alloc(&order.p, sizeof(int) * (size_t)N)) return 1;
    // The uncentred bfloat16 copy screens the side tests when the 8-bit copy does not, and the general exploration
    // kernel; with the 8-bit screen and the join nobody needs it (the few points the merge kernels may hand back to
    // the general kernel are then worked on without a screen).
    const bool join_explores = nnef > 0 && explore_join_enabled(N, K) && explore_merge_fits(D, K);
    const bool plain_copy = (n_trees > 0 && q8_rows == nullptr) || (nnef > 0 && !join_explores);
    Bf16Guard bf;
    if (plain_copy && (bf16_copy_alloc(&bf.c, N, D) || bf16_copy_fill(bf.c, d_points, N, D, stream))) return 1;

    rep.row_bytes = tree_screen_row_bytes(D, q8_rows != nullptr);
    if (n_trees > 0) {
        // the bucket kernels read a row's maximum from its last slot: rows the caller passed in unsorted are put
        // in order once
        if (launch_sort_rows(d_idx, d_dist, N, K, stream)) return 1;
        const int B = choose_batch(n_trees, N, D, MIN);
        WsGuard ws;
        if (tree_ws_alloc(&ws.w, N, D, MIN, B)) return 1;
        std::vector<int> stats((size_t)5 * B);
        // ev[j] is recorded where the K-NN update of tree j of a batch begins (both parts of tree j - 1 are done), ev[nb]
        // where the last one ends: one event per tree between the launches, not two
        std::vector<TimedEvent> ev((size_t)B + 1);
        for (auto& e : ev)
            if (e.create()) return 1;
        // numbers of pairs of every tree's small buckets (8 words per tree, added up on the host for the report): the
        // kernel of tree t reads those of tree t - 1 to choose its form
        DevBuf pair_stats;
        const size_t stat_words = (size_t)8 * (size_t)n_trees;
        if (ws_alloc(&pair_stats.p, sizeof(unsigned long long) * stat_words)) return 1;
        RSFK_HIP(hipMemsetAsync(pair_stats.p, 0, sizeof(unsigned long long) * stat_words, stream));
        unsigned long long* d_pairs = static_cast<unsigned long long*>(pair_stats.p);
        rep.screen_share_q16 = bucket_screen_share_q16();
        const int gram_from = bucket_gram_from();
        constexpr int kYoungTrees = 2;          // trees of a build whose bucket step still finds rows that are far from done
        SideStream sync;
        if (std::getenv("RSFK_KNN_ONE_STREAM") == nullptr && sync.open()) return 1;
        // working memory of the bucket kernels that pass the distances of a bucket's pairs through memory (only
        // buckets the specialised kernels do not take): one block per stream, grown when a tree asks for more
        DevBuf pair_buf[2];
        PairScratch pair_mem[2];
        auto pair_room = [&](int which, size_t want) -> int {
            if (want <= pair_mem[which].floats) return 0;
            RSFK_HIP(hipStreamSynchronize(stream));
            if (sync.side) RSFK_HIP(hipStreamSynchronize(sync.side));
            if (pair_buf[which].p) { ws_free(pair_buf[which].p); pair_buf[which].p = nullptr; }
            pair_mem[which] = PairScratch();
            want = std::min(pair_scratch_max(), want + want / 4);
            if (ws_try_alloc(&pair_buf[which].p, want * sizeof(float)) == 0) {
                pair_mem[which].p = static_cast<float*>(pair_buf[which].p);
                pair_mem[which].floats = want;
            }
            return 0;
        };
        int rc = 0;
        for (int t0 = 0; t0 < n_trees && rc == 0; t0 += B) {
            const int nb = std::min(B, n_trees - t0);
            const double tb0 = now_s();
            rc = build_tree_batch(ws.w, d_points, bf.c.rows, q8_rows, N, D, MIN, MAX, MAX_DEPTH, seed + t0, nb, stats.data(), stream);
            if (rc) break;
            const double tb = now_s() - tb0;
            rep.tree_s += tb;
            rep.tested += tree_ws_counts(ws.w)[0];
            rep.undecided += tree_ws_counts(ws.w)[1];
            // The larger buckets of a tree (a few per cent of the points at the default sizes: a grid too small to fill
            // the device) run on a second stream beside the small ones: different buckets of one tree touch different
            // rows.  Both parts of tree j wait for both parts of tree j - 1.
            bool big_pending = false;                    // sync.big holds the larger buckets of the previous tree
            for (int j = 0; j < nb && rc == 0; ++j) {
                const int n_big = stats[5 * j + 4], n_small = stats[5 * j] - n_big;
                const bool split = sync.side != nullptr && n_big > 0 && n_small > 0;
                if (big_pending) (void)hipStreamWaitEvent(stream, sync.big, 0);
                (void)hipEventRecord(ev[j].e, stream);                         // both parts of the previous tree are done
                if (split) (void)hipStreamWaitEvent(sync.side, ev[j].e, 0);      // everything before this tree
                const bool gram = t0 + j >= gram_from;
                const int t = t0 + j;
                {
                    const size_t want_small = K > 64 ? bucket_pairs_scratch_floats(D, K, n_small, kBucketSplit) : 0;
                    const size_t want_big = bucket_pairs_scratch_floats(D, K, n_big, stats[5 * j + 2]);
                    if (pair_room(0, split ? want_small : std::max(want_small, want_big))) return 1;
                    if (split && pair_room(1, want_big)) return 1;
                }
                rc = launch_bucket_knn_tree(d_points, t > 0 ? d_pairs + (size_t)8 * (t - 1) : nullptr, d_pairs + (size_t)8 * t, true,
                                            gram, D, K, tree_ws_perm(ws.w, j), tree_ws_leaf_start(ws.w, j),
                                            tree_ws_leaf_size(ws.w, j), tree_ws_leaf_cap(ws.w), n_small, n_big, stats[5 * j + 2],
                                            d_idx, d_dist, stream, split ? 1 : 0, t0 + j < kYoungTrees, &rep.kernels[(size_t)(t0 + j)],
                                            &pair_mem[0]);
                if (!rc && split) {
                    rc = launch_bucket_knn_tree(d_points, nullptr, nullptr, true, gram, D, K, tree_ws_perm(ws.w, j), tree_ws_leaf_start(ws.w, j),
                                                tree_ws_leaf_size(ws.w, j), tree_ws_leaf_cap(ws.w), n_small, n_big,
                                                stats[5 * j + 2], d_idx, d_dist, sync.side, 2, t0 + j < kYoungTrees,
                                                &rep.kernels[(size_t)(t0 + j)], &pair_mem[1]);
                    (void)hipEventRecord(sync.big, sync.side);
                }
                big_pending = split;
            }
            if (big_pending) (void)hipStreamWaitEvent(stream, sync.big, 0);
            (void)hipEventRecord(ev[nb].e, stream);
            if (rc) break;
            RSFK_HIP(hipStreamSynchronize(stream));
            for (int j = 0; j < nb; ++j) {
                float ms = 0.0f;
                (void)hipEventElapsedTime(&ms, ev[j].e, ev[j + 1].e);
                rep.bucket_s += ms * 1e-3;
                const int t = t0 + j;
                if (log_forest) {
                    log_forest[(size_t)0 * n_trees + t] = (float)stats[5 * j + 1];   // Tree Depth
                    log_forest[(size_t)1 * n_trees + t] = (float)stats[5 * j + 2];   // Max Leaf Size
                    log_forest[(size_t)2 * n_trees + t] = (float)stats[5 * j + 3];   // Min Leaf Size
                    log_forest[(size_t)3 * n_trees + t] = (float)stats[5 * j + 0];   // Total Leaves
                    log_forest[(size_t)5 * n_trees + t] = (float)(tb / nb);          // Total Tree Building Time
                    // the trees of a batch are built together, level by level: a tree's share of the batch's kernels
                    const float* ph = tree_ws_phase_seconds(ws.w);
                    log_forest[(size_t)7 * n_trees + t] = ph[0] / nb;                // Check Points Side Time (k_side)
                    log_forest[(size_t)11 * n_trees + t] = ph[1] / nb;               // Create Nodes Time (k_level_planes)
                    log_forest[(size_t)12 * n_trees + t] = ph[2] / nb;               // Update Nodes Time (k_scatter)
                    log_forest[(size_t)13 * n_trees + t] = ph[3] / nb;               // Bucket Creation Time (k_tail)
                    log_forest[(size_t)15 * n_trees + t] = ms * 1e-3f;               // KNN Sets Updates
                }
                if (verbose >= 2)
                    std::printf("tree %d: depth %d, leaves %d, leaf size %d..%d, K-NN update %.6f s\n", t,
                                stats[5 * j + 1], stats[5 * j + 0], stats[5 * j + 3], stats[5 * j + 2], ms * 1e-3);
            }
        }
        if (rc) return rc;
        if (order.p) {
            // (finished before the tree workspace goes back to the pool)
            RSFK_HIP(hipMemcpyAsync(order.p, tree_ws_perm(ws.w, (n_trees - 1) % B), sizeof(int) * (size_t)N, hipMemcpyDeviceToDevice, stream));
            RSFK_HIP(hipStreamSynchronize(stream));
        }
        std::vector<unsigned long long> h_pairs(stat_words);
        RSFK_HIP(hipMemcpy(h_pairs.data(), d_pairs, sizeof(unsigned long long) * stat_words, hipMemcpyDeviceToHost));
        rep.pairs.assign((size_t)n_trees, 0);
        for (size_t i = 0; i < stat_words; ++i) rep.pairs[i / 8] += h_pairs[i];
    }
    const double t_forest = now_s() - t_forest0;
    if (verbose >= 1) std::printf("Creating RSFK forest takes %lf seconds\n", t_forest);

    const double t_exp0 = now_s();
    if (nnef > 0) {
        DevBuf old;
        if (ws_alloc(&old.p, sizeof(int) * (size_t)N * (size_t)K)) return 1;
        ExploreWsGuard ews;      // without a workspace every point enumerates its own candidates
        Bf16Guard bfc;           // centred copy for the join
        DevBuf stat;             // count of the exact distances (for the report)
        if (ws_alloc(&stat.p, sizeof(unsigned long long) * kExploreStatWords)) return 1;
        RSFK_HIP(hipMemsetAsync(stat.p, 0, sizeof(unsigned long long) * kExploreStatWords, stream));
        if (explore_join_enabled(N, K)) {
            if (explore_ws_alloc(&ews.w, N, K, explore_join_keeps_bounds(N, D, K))) return 1;
            if (bf16_copy_alloc(&bfc.c, N, D, true) || bf16_copy_fill(bfc.c, d_points, N, D, stream)) return 1;
        }
        for (int it = 0; it < nnef; ++it) {
            // (the bucket step of the forest, and every exploration pass, leave all rows in order)
            if (launch_explore(d_points, plain_copy ? &bf.c : nullptr, &bfc.c, N, D, K, d_idx, d_dist, static_cast<int*>(old.p), ews.w, stream,
                               n_trees > 0 || it > 0, static_cast<unsigned long long*>(stat.p), static_cast<const int*>(order.p)))
                return 1;
        }
        std::vector<unsigned long long> h_stat((size_t)kExploreStatWords);
        RSFK_HIP(hipMemcpyAsync(h_stat.data(), stat.p, sizeof(unsigned long long) * kExploreStatWords, hipMemcpyDeviceToHost, stream));
        RSFK_HIP(hipStreamSynchronize(stream));
        for (int i = 0; i < kExploreStatWords; i += 32) rep.exact += h_stat[(size_t)i];
    }
    const double t_exp = now_s() - t_exp0;
    if (verbose >= 1) std::printf("Nearest Neighbors Exploring computation Kernel takes %lf seconds\n", t_exp);
    if (log_forest) {
        log_forest[(size_t)16 * n_trees] = (float)t_forest;
        log_forest[(size_t)16 * n_trees + 1] = (float)t_exp;
    }
    rep.explore_s = t_exp;
    {
        std::lock_guard<std::mutex> lock(g_report_mutex);
        g_report = std::move(rep);
    }
    return 0;
}

// Query-set search (RSFK::knn_gpu_rsfk_forest_ann, src/rsfk.cu:98-155): n_trees trees on the base points (seed + tree
// index, as in the forest above); per tree the queries are routed to a leaf and the base points of that leaf are
// offered to the query's row.  Rows are merged into, indices refer to the base points.  The log receives the
// per-tree series of the forest (tree statistics, tree time, update time) and the total time.
int knn_ann_forest_device(int n_trees, int K, int N, int NQ, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                          const float* d_points, const float* d_queries, int* d_qidx, float* d_qdist, float* log_forest,
                          hipStream_t stream)
{
    RSFK_CHECK(N >= 1 && D >= 1 && K >= 1 && NQ >= 0, "query-set search: N, D and K must be positive");
    RSFK_CHECK(n_trees >= 0, "query-set search: n_trees must not be negative");
    RSFK_CHECK(K <= kMaxK, "query-set search: K above 1024 is not supported");
    if (log_forest) std::memset(log_forest, 0, sizeof(float) * ((size_t)16 * n_trees + 2));
    const double t0 = now_s();
    if (n_trees > 0 && NQ > 0) {
        Bf16Guard bf;
        if (bf16_copy_alloc(&bf.c, N, D)) return 1;
        if (bf16_copy_fill(bf.c, d_points, N, D, stream)) return 1;
        Q8Guard q8;
        const uint8_t* q8_rows = nullptr;
        if (make_tree_screen(q8, d_points, N, D, verbose, stream, &q8_rows)) return 1;
        const int B = choose_batch(n_trees, N, D, MIN);
        WsGuard ws;
        if (tree_ws_alloc(&ws.w, N, D, MIN, B)) return 1;
        if (tree_ws_enable_index(ws.w, MIN, MAX_DEPTH)) return 1;
        const int rec_cap = tree_ws_rec_cap(ws.w);
        DevBuf aws;
        if (ws_alloc(&aws.p, sizeof(int) * ann_ws_ints(NQ, rec_cap))) return 1;
        if (launch_ann_ws_init(static_cast<int*>(aws.p), NQ, rec_cap, stream)) return 1;
        DevBuf planes;
        if (ws_alloc(&planes.p, sizeof(float) * (size_t)rec_cap * (size_t)ann_plane_pitch(D))) return 1;
        std::vector<int> stats((size_t)5 * B);
        std::vector<TimedEvent> ev((size_t)B + 1);          // ev[j]: the search in tree j of a batch begins, ev[nb]: the last ends
        for (auto& e : ev)
            if (e.create()) return 1;
        int rc = 0;
        for (int tb0 = 0; tb0 < n_trees && rc == 0; tb0 += B) {
            const int nb = std::min(B, n_trees - tb0);
            const double tt0 = now_s();
            rc = build_tree_batch(ws.w, d_points, bf.c.rows, q8_rows, N, D, MIN, MAX, MAX_DEPTH, seed + tb0, nb, stats.data(),
                                  stream);
            if (rc) break;
            const double tt = now_s() - tt0;
            for (int j = 0; j < nb && rc == 0; ++j) {
                (void)hipEventRecord(ev[j].e, stream);
                rc = launch_ann_tree(d_points, d_queries, NQ, D, K, tree_ws_perm(ws.w, j), tree_ws_recs(ws.w, j),
                                     tree_ws_n_rec(ws.w, j), rec_cap, stats[5 * j + 0], static_cast<int*>(aws.p),
                                     static_cast<float*>(planes.p), d_qidx, d_qdist, stream);
            }
            (void)hipEventRecord(ev[nb].e, stream);
            if (rc) break;
            RSFK_HIP(hipStreamSynchronize(stream));
            for (int j = 0; j < nb; ++j) {
                float ms = 0.0f;
                (void)hipEventElapsedTime(&ms, ev[j].e, ev[j + 1].e);
                const int t = tb0 + j;
                if (log_forest) {
                    log_forest[(size_t)0 * n_trees + t] = (float)stats[5 * j + 1];   // Tree Depth
                    log_forest[(size_t)1 * n_trees + t] = (float)stats[5 * j + 2];   // Max Leaf Size
                    log_forest[(size_t)2 * n_trees + t] = (float)stats[5 * j + 3];   // Min Leaf Size
                    log_forest[(size_t)3 * n_trees + t] = (float)stats[5 * j + 0];   // Total Leaves
                    log_forest[(size_t)5 * n_trees + t] = (float)(tt / nb);          // Total Tree Building Time
                    log_forest[(size_t)15 * n_trees + t] = ms * 1e-3f;               // KNN Sets Updates
                }
                if (verbose >= 2)
                    std::printf("tree %d: depth %d, leaves %d, leaf size %d..%d, query update %.6f s\n", t, stats[5 * j + 1],
                                stats[5 * j + 0], stats[5 * j + 3], stats[5 * j + 2], ms * 1e-3);
            }
        }
        if (rc) return rc;
    }
    const double t_total = now_s() - t0;
    if (verbose >= 1) std::printf("Query-set search over %d trees takes %lf seconds\n", n_trees, t_total);
    if (log_forest) log_forest[(size_t)16 * n_trees] = (float)t_total;
    return 0;
}

int knn_ann_forest_host(int n_trees, int K, int N, int NQ, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                        const float* points, const float* queries, int* q_idx, float* q_dist, float* log_forest)
{
    RSFK_CHECK(N >= 1 && D >= 1 && K >= 1 && NQ >= 0, "query-set search: N, D and K must be positive");
    if (NQ == 0) return 0;
    DevBuf dp, dq, di, dd;
    const size_t nd = (size_t)N * (size_t)D, qd = (size_t)NQ * (size_t)D, nk = (size_t)NQ * (size_t)K;
    if (ws_alloc(&dp.p, nd * sizeof(float)) || ws_alloc(&dq.p, qd * sizeof(float)) || ws_alloc(&di.p, nk * sizeof(int)) ||
        ws_alloc(&dd.p, nk * sizeof(float)))
        return 1;
    RSFK_HIP(hipMemcpy(dp.p, points, nd * sizeof(float), hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(dq.p, queries, qd * sizeof(float), hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(di.p, q_idx, nk * sizeof(int), hipMemcpyHostToDevice));
    RSFK_HIP(hipMemcpy(dd.p, q_dist, nk * sizeof(float), hipMemcpyHostToDevice));
    const int rc = knn_ann_forest_device(n_trees, K, N, NQ, D, MIN, MAX, MAX_DEPTH, verbose, seed,
                                         static_cast<const float*>(dp.p), static_cast<const float*>(dq.p),
                                         static_cast<int*>(di.p), static_cast<float*>(dd.p), log_forest, nullptr);
    if (rc) return rc;
    RSFK_HIP(hipMemcpy(q_idx, di.p, nk * sizeof(int), hipMemcpyDeviceToHost));
    RSFK_HIP(hipMemcpy(q_dist, dd.p, nk * sizeof(float), hipMemcpyDeviceToHost));
    return 0;
}

namespace {
// rows as the Python layer prepares them (RSFK.py:330-335 of the reference): empty, or the point itself in slot 0
__global__ __launch_bounds__(256) void k_fresh_rows(int* __restrict__ idx, float* __restrict__ dist, size_t total, int K,
                                                    int self_in)
{
    for (size_t e = blockIdx.x * (size_t)256 + threadIdx.x; e < total; e += (size_t)gridDim.x * 256) {
        const bool first = self_in && e % (size_t)K == 0;
        idx[e] = first ? (int)(e / (size_t)K) : -1;
        dist[e] = first ? 0.0f : INFINITY;
    }
}
}  // namespace

// fresh_rows: 0 = the rows are in/out (copied to the device first), 1 = they start empty, 2 = they start with the
// point itself (distance 0) in slot 0; with 1 or 2 the host arrays are only written.
int knn_forest_host(int n_trees, int K, int N, int D, int MIN, int MAX, int MAX_DEPTH, int verbose, int seed,
                    int nnef, const float* points, int* knn_idx, float* knn_dist, float* log_forest, int fresh_rows)
{
    RSFK_CHECK(N >= 1 && D >= 1 && K >= 1, "forest: N, D and K must be positive");
    DevBuf dp, di, dd;
    const size_t nd = (size_t)N * (size_t)D, nk = (size_t)N * (size_t)K;
    if (ws_alloc(&dp.p, nd * sizeof(float))) return 1;
    if (ws_alloc(&di.p, nk * sizeof(int))) return 1;
    if (ws_alloc(&dd.p, nk * sizeof(float))) return 1;
    if (copy_to_device(dp.p, points, nd * sizeof(float))) return 1;
    if (fresh_rows) {
        const unsigned grid = (unsigned)std::min<size_t>((nk + 255) / 256, 65536);
        hipLaunchKernelGGL(k_fresh_rows, dim3(grid), dim3(256), 0, nullptr, static_cast<int*>(di.p), static_cast<float*>(dd.p),
                           nk, K, fresh_rows == 2 ? 1 : 0);
        RSFK_HIP(hipGetLastError());
    } else {
        if (copy_to_device(di.p, knn_idx, nk * sizeof(int))) return 1;
        if (copy_to_device(dd.p, knn_dist, nk * sizeof(float))) return 1;
    }
    const int rc = knn_forest_device(n_trees, K, N, D, MIN, MAX, MAX_DEPTH, verbose, seed, nnef,
                                     static_cast<const float*>(dp.p), static_cast<int*>(di.p),
                                     static_cast<float*>(dd.p), log_forest, nullptr);
    if (rc) return rc;
    if (copy_to_host(knn_idx, di.p, nk * sizeof(int))) return 1;
    if (copy_to_host(knn_dist, dd.p, nk * sizeof(float))) return 1;
    return 0;
}

// One tree; results on the host.  perm: N ints; leaves sorted by start.
int build_tree_host(const float* d_points, int N, int D, int MIN, int MAX, int MAX_DEPTH, int seed,
                    std::vector<int>& perm, std::vector<int>& leaf_start, std::vector<int>& leaf_size, int stats[5])
{
    WsGuard ws;
    if (tree_ws_alloc(&ws.w, N, D, MIN, 1)) return 1;
    Bf16Guard bf;
    if (bf16_copy_alloc(&bf.c, N, D)) return 1;
    if (bf16_copy_fill(bf.c, d_points, N, D, nullptr)) return 1;
    Q8Guard q8;
    const uint8_t* q8_rows = nullptr;
    if (make_tree_screen(q8, d_points, N, D, 0, nullptr, &q8_rows)) return 1;
    if (build_tree_batch(ws.w, d_points, bf.c.rows, q8_rows, N, D, MIN, MAX, MAX_DEPTH, seed, 1, stats, nullptr)) return 1;
    const int nl = stats[0], n_big = stats[4], n_small = nl - n_big, cap = tree_ws_leaf_cap(ws.w);
    perm.resize((size_t)N);
    std::vector<int> ls((size_t)nl), lz((size_t)nl);
    RSFK_HIP(hipMemcpy(perm.data(), tree_ws_perm(ws.w, 0), sizeof(int) * (size_t)N, hipMemcpyDeviceToHost));
    if (n_small > 0) {
        RSFK_HIP(hipMemcpy(ls.data(), tree_ws_leaf_start(ws.w, 0), sizeof(int) * (size_t)n_small, hipMemcpyDeviceToHost));
        RSFK_HIP(hipMemcpy(lz.data(), tree_ws_leaf_size(ws.w, 0), sizeof(int) * (size_t)n_small, hipMemcpyDeviceToHost));
    }
    if (n_big > 0) {
        RSFK_HIP(hipMemcpy(ls.data() + n_small, tree_ws_leaf_start(ws.w, 0) + (cap - n_big), sizeof(int) * (size_t)n_big, hipMemcpyDeviceToHost));
        RSFK_HIP(hipMemcpy(lz.data() + n_small, tree_ws_leaf_size(ws.w, 0) + (cap - n_big), sizeof(int) * (size_t)n_big, hipMemcpyDeviceToHost));
    }
    std::vector<int> order((size_t)nl);
    for (int i = 0; i < nl; ++i) order[i] = i;
    std::sort(order.begin(), order.end(), [&](int a, int b) { return ls[a] < ls[b]; });
    leaf_start.resize((size_t)nl);
    leaf_size.resize((size_t)nl);
    for (int i = 0; i < nl; ++i) { leaf_start[i] = ls[order[i]]; leaf_size[i] = lz[order[i]]; }
    return 0;
}

}  // namespace rsfk
