/*
 * rsfk_oracle.c -- CPU restatement of the RSFK K-NN-graph algorithm.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the GPU library is
 * compared against (tests, the smoke check, the CPU-baseline leg of the
 * benchmark).  Nothing in the shipped GPU path includes, links or calls it.
 *
 * What it restates (paths relative to the reference repository):
 *   - hyperplane of a node from a random point pair   src/kernels/create_node.cu:101-137
 *   - side test  n.x < b  (right side)                src/kernels/build_tree_check_points_side.cu:123-149
 *   - split / min-size merge / leaf rules             src/kernels/build_tree_update_parents.cu:64-75,106-134
 *   - pair draw per (node, side)                      src/kernels/build_tree_create_nodes.cu:86-104
 *   - squared distance, direct differences            src/kernels/compute_knn_from_buckets.cu:40-54
 *   - bucket K-NN update, diagonal schedule           src/kernels/compute_knn_from_buckets.cu:998-1378
 *   - neighbours-of-neighbours exploration            src/kernels/nearest_neighbors_exploring.cu:41-146
 *   - forest loop, seed increment, exploration loop   src/rsfk.cu:2033-2183
 *   - query-set search: routing and bucket update     src/rsfk.cu:98-498,
 *                                                     src/kernels/build_tree_update_parents_ann.cu:77-517
 *   - symmetrised graph in compressed-row form        src/rsfk.cu:1229-1299 (commented out there)
 *
 * Deliberate differences from the reference (none of them is pinned by any
 * fixture in the reference, see the parity notes at the end of this header):
 *   - random numbers: the reference uses cuRAND XORWOW seeded from the launch
 *     geometry (build_tree_create_nodes.cu:64-68); here a counter-based
 *     generator keyed by the node's path is used so that a tree is a pure
 *     function of (points, MIN, MAX, MAX_DEPTH, seed).
 *   - order of the members of a node: the reference orders them by the
 *     arrival order of atomics; here a node's members are kept in the order
 *     produced by stable partitions of 0..N-1.
 *   - reference defects that are not reproduced: empty leaf slots for empty
 *     sides, the unordered is_leaf write, points stranded when MAX_DEPTH is
 *     hit (they become a leaf here), out-of-range reads for -1 neighbours in
 *     the exploration pass, self-insertion in the exploration pass, NaN
 *     distances entering a row in the bucket step (they never enter here).
 *
 * Arithmetic is fp32 with explicitly fused multiply-adds where the CUDA
 * compiler would contract them; compile with -ffp-contract=off so nothing
 * else is fused.
 *
 * Parity pinning status:
 *   sqdist / dot / hyperplane : pinned by closed forms and by fp64 evaluation
 *                               (tests/test_oracle_math.py)
 *   bucket K-NN               : pinned by brute force (one bucket holding all
 *                               points == exact K-NN) and set invariants
 *   exploration               : pinned by a pure-Python restatement on tiny
 *                               graphs and by invariants
 *   tree build rules          : pinned by invariants, hand-traceable cases and
 *                               a pure-Python restatement of the same rules
 *   query-set search          : routing pinned by a pure-Python restatement and by
 *                               "a base point used as a query lands in its own leaf";
 *                               the update by brute force inside the reached leaves
 *   symmetrised graph         : pinned by scipy.sparse (A.maximum(A.T) of the directed graph) and by a
 *                               hand-written 5-point case (tests/test_oracle_graph.py)
 *   random draw sequence      : parity unpinned (cuRAND is not available and
 *                               no reference fixture holds a partition)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <float.h>
#include <stdio.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define RSFK_OR_EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* counter-based random numbers                                        */
/* ------------------------------------------------------------------ */

static inline uint64_t mix64(uint64_t z)
{
    z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ULL;
    z ^= z >> 27; z *= 0x94D049BB133111EBULL;
    z ^= z >> 31;
    return z;
}

RSFK_OR_EXPORT uint64_t rsfk_or_root_key(int seed)
{
    return mix64((uint64_t)(int64_t)seed ^ 0x5253464B524F4F54ULL);
}

RSFK_OR_EXPORT uint64_t rsfk_or_child_key(uint64_t key, int side)
{
    return mix64(key + 0x9E3779B97F4A7C15ULL * (uint64_t)(side + 1));
}

RSFK_OR_EXPORT uint32_t rsfk_or_draw(uint64_t key, uint32_t i)
{
    return (uint32_t)(mix64(key ^ (0xD6E8FEB86659FD93ULL * (uint64_t)(i + 1))) >> 32);
}

/* Two member ranks in [0, count): the second is redrawn while it equals the
 * first (build_tree_create_nodes.cu:96-100), at most 64 times. */
RSFK_OR_EXPORT void rsfk_or_pick_pair(uint64_t key, int count, int* r1, int* r2)
{
    uint32_t c = (uint32_t)count;
    uint32_t a = rsfk_or_draw(key, 0) % c;
    uint32_t b = rsfk_or_draw(key, 1) % c;
    if (count >= 2) {
        uint32_t i = 2;
        while (b == a && i < 66) { b = rsfk_or_draw(key, i) % c; ++i; }
        if (b == a) b = (a + 1) % c;
    }
    *r1 = (int)a; *r2 = (int)b;
}

/* ------------------------------------------------------------------ */
/* arithmetic kernels                                                  */
/* ------------------------------------------------------------------ */

/* sum_i (a_i-b_i)^2, sequential, one fused multiply-add per dimension
 * (compute_knn_from_buckets.cu:40-54 as nvcc contracts it). */
RSFK_OR_EXPORT float rsfk_or_sqdist(const float* a, const float* b, int D)
{
    float acc = 0.0f;
    for (int i = 0; i < D; ++i) {
        float diff = a[i] - b[i];
        acc = fmaf(diff, diff, acc);
    }
    return acc;
}

RSFK_OR_EXPORT double rsfk_or_sqdist_f64(const float* a, const float* b, int D)
{
    double acc = 0.0;
    for (int i = 0; i < D; ++i) {
        double diff = (double)a[i] - (double)b[i];
        acc += diff * diff;
    }
    return acc;
}

static inline float butterfly32(float* p)
{
    /* xor butterfly 1,2,4,8,16 over 32 partial sums
     * (build_tree_check_points_side.cu:139-143) */
    float q[32];
    for (int m = 1; m < 32; m <<= 1) {
        for (int l = 0; l < 32; ++l) q[l] = p[l] + p[l ^ m];
        memcpy(p, q, sizeof(q));
    }
    return p[0];
}

/* n.x with 32 lane-strided partial sums (fused multiply-add), then the
 * butterfly (build_tree_check_points_side.cu:131-143). */
RSFK_OR_EXPORT float rsfk_or_dot32(const float* n, const float* x, int D)
{
    float p[32];
    for (int l = 0; l < 32; ++l) p[l] = 0.0f;
    for (int d = 0; d < D; ++d) p[d & 31] = fmaf(n[d], x[d], p[d & 31]);
    return butterfly32(p);
}

/* n = x1 - x2 ; b = sum n_i*(x1_i+x2_i)/2, same lane-strided order
 * (create_node.cu:122-135). */
RSFK_OR_EXPORT float rsfk_or_hyperplane(const float* x1, const float* x2, int D, float* n)
{
    float p[32];
    for (int l = 0; l < 32; ++l) p[l] = 0.0f;
    for (int d = 0; d < D; ++d) {
        float t1 = x1[d], t2 = x2[d];
        float nd = t1 - t2;
        n[d] = nd;
        float prod = nd * (t1 + t2);
        p[d & 31] = p[d & 31] + prod * 0.5f;
    }
    return butterfly32(p);
}

/* ------------------------------------------------------------------ */
/* one random-sample tree                                              */
/* ------------------------------------------------------------------ */

typedef struct {
    int start, count;      /* members = perm[start .. start+count)              */
    int dstart, dcount;    /* the pair is drawn from perm[dstart .. +dcount)     */
    int depth;             /* level of the node, root = 0                        */
    int leaf;
    uint64_t key;
    int qstart, qcount;    /* query points that reached the node = qperm[qstart .. +qcount) */
} or_node;

/*
 * Builds one tree.  perm (N ints) receives the point ids grouped by leaf;
 * leaf_start/leaf_size (capacity leaf_cap) receive the leaves in ascending
 * start order.  Returns the number of leaves, or -1 if leaf_cap is too small.
 * stats[0] = number of levels, stats[1] = max leaf size, stats[2] = min leaf size.
 */
/*
 * The same with NQ query points routed down the tree while it is built (the routing of
 * RSFK::knn_gpu_rsfk_forest_ann_tree, src/rsfk.cu:262-356: the side test of
 * build_tree_check_points_side.cu on the query, then the child on that side, or the only child where the
 * node has one -- src/kernels/build_tree_update_parents_ann.cu:141-151).  q_leaf_start/q_leaf_size
 * (NQ ints each) receive the leaf each query ends in, as a segment of perm.  queries may be NULL.
 */
static int build_tree_ex(const float* points, int N, int D,
                         int MIN, int MAX, int MAX_DEPTH, int seed,
                         int* perm, int* leaf_start, int* leaf_size,
                         int leaf_cap, int* stats,
                         const float* queries, int NQ, int* q_leaf_start, int* q_leaf_size)
{
    if (N <= 0) { if (stats) { stats[0] = 0; stats[1] = 0; stats[2] = 0; } return 0; }
    if (!queries) NQ = 0;
    int* qperm = (int*)malloc(sizeof(int) * (size_t)(NQ > 0 ? NQ : 1));
    int* qtmp = (int*)malloc(sizeof(int) * (size_t)(NQ > 0 ? NQ : 1));
    for (int i = 0; i < NQ; ++i) qperm[i] = i;
    int* tmp = (int*)malloc(sizeof(int) * (size_t)N);
    unsigned char* side = (unsigned char*)malloc((size_t)N);
    float* nvec = (float*)malloc(sizeof(float) * (size_t)(D > 0 ? D : 1));
    size_t cap = 64, top = 0;
    or_node* stack = (or_node*)malloc(sizeof(or_node) * cap);
    for (int i = 0; i < N; ++i) perm[i] = i;

    int n_leaves = 0, levels = 1, maxleaf = 0, minleaf = 0x7fffffff, overflow = 0;
    or_node root = {0, N, 0, N, 0, 0, rsfk_or_root_key(seed), 0, NQ};   /* never a leaf: build_tree_init.cu:79 */
    stack[top++] = root;

    while (top > 0) {
        or_node nd = stack[--top];
        if (nd.depth + 1 > levels) levels = nd.depth + 1;
        if (nd.leaf || nd.depth >= MAX_DEPTH - 1) {
            if (leaf_start) {
                if (n_leaves < leaf_cap) { leaf_start[n_leaves] = nd.start; leaf_size[n_leaves] = nd.count; }
                else overflow = 1;
            }
            for (int i = 0; i < nd.qcount; ++i) {
                q_leaf_start[qperm[nd.qstart + i]] = nd.start;
                q_leaf_size[qperm[nd.qstart + i]] = nd.count;
            }
            ++n_leaves;
            if (nd.count > maxleaf) maxleaf = nd.count;
            if (nd.count < minleaf) minleaf = nd.count;
            continue;
        }
        int r1, r2;
        rsfk_or_pick_pair(nd.key, nd.dcount, &r1, &r2);
        const float* x1 = points + (size_t)perm[nd.dstart + r1] * D;
        const float* x2 = points + (size_t)perm[nd.dstart + r2] * D;
        float b = rsfk_or_hyperplane(x1, x2, D, nvec);

        int a = 0;
        for (int i = 0; i < nd.count; ++i) {
            const float* x = points + (size_t)perm[nd.start + i] * D;
            int right = rsfk_or_dot32(nvec, x, D) < b;      /* build_tree_check_points_side.cu:149 */
            side[i] = (unsigned char)right;
            a += !right;
        }
        int r = nd.count - a;
        /* stable partition: left members first */
        {
            int il = 0, ir = a;
            for (int i = 0; i < nd.count; ++i) {
                int id = perm[nd.start + i];
                if (side[i]) tmp[ir++] = id; else tmp[il++] = id;
            }
            memcpy(perm + nd.start, tmp, sizeof(int) * (size_t)nd.count);
        }
        /* the queries in the node take the same test; where the node gets one child they all follow it */
        int qa = nd.qcount;
        if (a != 0 && r != 0 && (a < r ? a : r) >= MIN) {
            int il = 0, ir = 0;
            for (int i = 0; i < nd.qcount; ++i) {
                int q = qperm[nd.qstart + i];
                int right = rsfk_or_dot32(nvec, queries + (size_t)q * D, D) < b;
                if (right) qtmp[nd.qcount - 1 - ir++] = q; else qperm[nd.qstart + il++] = q;
            }
            qa = il;
            for (int i = 0; i < ir; ++i) qperm[nd.qstart + il + i] = qtmp[nd.qcount - 1 - i];
        }
        uint64_t kl = rsfk_or_child_key(nd.key, 0), kr = rsfk_or_child_key(nd.key, 1);
        or_node c0, c1; int nchild;
        if (a == 0 || r == 0) {
            /* only one child exists (build_tree_create_nodes.cu:90); it gets the
             * plain leaf test of build_tree_update_parents.cu:71-73 */
            c0.start = nd.start; c0.count = nd.count; c0.dstart = nd.start; c0.dcount = nd.count;
            c0.depth = nd.depth + 1; c0.key = a ? kl : kr; c0.leaf = nd.count <= MAX - 2;
            nchild = 1;
        } else if ((a < r ? a : r) < MIN) {
            /* min-size rule: the small side moves into the sibling
             * (build_tree_update_parents.cu:106-134) */
            int left_big = a >= r;
            c0.start = nd.start; c0.count = nd.count;
            c0.dstart = left_big ? nd.start : nd.start + a;
            c0.dcount = left_big ? a : r;
            c0.depth = nd.depth + 1; c0.key = left_big ? kl : kr; c0.leaf = nd.count <= MAX;
            nchild = 1;
        } else {
            c0.start = nd.start; c0.count = a; c0.dstart = nd.start; c0.dcount = a;
            c0.depth = nd.depth + 1; c0.key = kl; c0.leaf = a <= MAX - 2;
            c1.start = nd.start + a; c1.count = r; c1.dstart = nd.start + a; c1.dcount = r;
            c1.depth = nd.depth + 1; c1.key = kr; c1.leaf = r <= MAX - 2;
            nchild = 2;
        }
        c0.qstart = nd.qstart; c0.qcount = nchild == 2 ? qa : nd.qcount;
        c1.qstart = nd.qstart + qa; c1.qcount = nd.qcount - qa;
        if (top + 2 > cap) { cap *= 2; stack = (or_node*)realloc(stack, sizeof(or_node) * cap); }
        /* push right first so that leaves come out in ascending start order */
        if (nchild == 2) stack[top++] = c1;
        stack[top++] = c0;
    }
    free(tmp); free(side); free(nvec); free(stack); free(qperm); free(qtmp);
    if (stats) { stats[0] = levels; stats[1] = maxleaf; stats[2] = n_leaves ? minleaf : 0; }
    return overflow ? -1 : n_leaves;
}

RSFK_OR_EXPORT int rsfk_or_build_tree(const float* points, int N, int D,
                                      int MIN, int MAX, int MAX_DEPTH, int seed,
                                      int* perm, int* leaf_start, int* leaf_size,
                                      int leaf_cap, int* stats)
{
    return build_tree_ex(points, N, D, MIN, MAX, MAX_DEPTH, seed, perm, leaf_start, leaf_size, leaf_cap, stats,
                         NULL, 0, NULL, NULL);
}

/* One tree on the points, the queries routed to their leaves: see build_tree_ex.  Returns the number of leaves. */
RSFK_OR_EXPORT int rsfk_or_route_queries(const float* points, int N, int D,
                                         int MIN, int MAX, int MAX_DEPTH, int seed,
                                         const float* queries, int NQ,
                                         int* perm, int* q_leaf_start, int* q_leaf_size)
{
    return build_tree_ex(points, N, D, MIN, MAX, MAX_DEPTH, seed, perm, NULL, NULL, 0, NULL,
                         queries, NQ, q_leaf_start, q_leaf_size);
}

/* ------------------------------------------------------------------ */
/* K-NN list update rule                                               */
/* ------------------------------------------------------------------ */

/*
 * The rows are ordered by (distance, index): entry (d1, c1) is above (d2, c2) iff d1 > d2, or d1 == d2 and
 * c1 > c2.  An empty slot (-1, +inf or FLT_MAX) is above every candidate that can enter.
 */
static inline int pair_above(float d1, int c1, float d2, int c2)
{
    return d1 > d2 || (d1 == d2 && c1 > c2);
}

/* position of the largest (distance, index) of the row */
static inline int row_max(const int* idx, const float* dist, int K)
{
    int m = 0;
    for (int j = 1; j < K; ++j) if (pair_above(dist[j], idx[j], dist[m], idx[m])) m = j;
    return m;
}

/*
 * Candidate c at distance d against one row; returns 1 if inserted.  The reference lets a candidate enter iff it
 * is strictly closer than the row's maximum and not in the row, and it then replaces the (first) maximum
 * (compute_knn_from_buckets.cu:1215-1230, nearest_neighbors_exploring.cu:124-141); among points at exactly the
 * K-th distance the row then keeps whichever arrived first.  Here a candidate enters iff its (distance, index) is
 * below the row's largest (distance, index), which it replaces: the row ends with the K smallest (distance, index)
 * pairs of everything it was offered, whatever the order of arrival.  The two rules differ only among points tied
 * at a row's K-th distance.  A candidate at +inf or NaN never enters (the reference's bucket kernel would store
 * a NaN, its exploration kernel would not).
 */
static inline int try_insert(int* idx, float* dist, int K, int* maxpos, int c, float d)
{
    const int m = *maxpos;
    if (!(d < INFINITY)) return 0;
    if (!(d < dist[m] || (d == dist[m] && c < idx[m]))) return 0;
    for (int k = 0; k < K; ++k) if (idx[k] == c) return 0;
    idx[m] = c; dist[m] = d;
    *maxpos = row_max(idx, dist, K);
    return 1;
}

/*
 * Bucket K-NN.  Bucket b holds ids[start_b .. start_b+sizes[b]) where
 * start_b = starts ? starts[b] : b*stride.  Pairs are visited in the order of
 * the reference's diagonal schedule: for each super-diagonal off = 1..s-1 first
 * every (i <- i+off) update, then every (i+off <- i) update.
 */
RSFK_OR_EXPORT void rsfk_or_bucket_knn(const float* points, int N, int D, int K,
                                       const int* ids, const int* starts, const int* sizes,
                                       int n_buckets, int stride,
                                       int* knn_idx, float* knn_dist)
{
    (void)N;
#pragma omp parallel
    {
        float* cand = NULL; int* maxpos = NULL; int capc = 0;
#pragma omp for schedule(dynamic, 16)
        for (int b = 0; b < n_buckets; ++b) {
            int s = sizes[b];
            const int* bid = ids + (starts ? (size_t)starts[b] : (size_t)b * (size_t)stride);
            if (s > capc) {
                capc = s;
                cand = (float*)realloc(cand, sizeof(float) * (size_t)capc);
                maxpos = (int*)realloc(maxpos, sizeof(int) * (size_t)capc);
            }
            for (int i = 0; i < s; ++i) maxpos[i] = row_max(knn_idx + (size_t)bid[i] * K, knn_dist + (size_t)bid[i] * K, K);
            for (int off = 1; off < s; ++off) {
                for (int i = 0; i + off < s; ++i)
                    cand[i] = rsfk_or_sqdist(points + (size_t)bid[i] * D, points + (size_t)bid[i + off] * D, D);
                for (int i = 0; i + off < s; ++i) {
                    int p1 = bid[i], p2 = bid[i + off];
                    try_insert(knn_idx + (size_t)p1 * K, knn_dist + (size_t)p1 * K, K, &maxpos[i], p2, cand[i]);
                }
                for (int i = 0; i + off < s; ++i) {
                    int p1 = bid[i], p2 = bid[i + off];
                    try_insert(knn_idx + (size_t)p2 * K, knn_dist + (size_t)p2 * K, K, &maxpos[i + off], p1, cand[i]);
                }
            }
        }
        free(cand); free(maxpos);
    }
}

/* One Jacobi exploration pass (nearest_neighbors_exploring.cu:70-141):
 * candidates come from a snapshot of the index array, the row being updated
 * is the live one. */
RSFK_OR_EXPORT void rsfk_or_explore(const float* points, int N, int D, int K,
                                    int* knn_idx, float* knn_dist)
{
    size_t tot = (size_t)N * (size_t)K;
    int* old = (int*)malloc(sizeof(int) * (tot ? tot : 1));
    memcpy(old, knn_idx, sizeof(int) * tot);
#pragma omp parallel for schedule(dynamic, 64)
    for (int p = 0; p < N; ++p) {
        int* idx = knn_idx + (size_t)p * K;
        float* dist = knn_dist + (size_t)p * K;
        const float* xp = points + (size_t)p * D;
        int maxpos = row_max(idx, dist, K);
        for (int i = 0; i < K; ++i) {
            int q = old[(size_t)p * K + i];
            if (q < 0 || q >= N) continue;
            for (int k = 0; k < K; ++k) {
                int c = old[(size_t)q * K + k];
                if (c < 0 || c >= N || c == p) continue;
                int dup = 0;
                for (int j = 0; j < K; ++j) if (idx[j] == c) { dup = 1; break; }
                if (dup) continue;
                float d = rsfk_or_sqdist(points + (size_t)c * D, xp, D);
                try_insert(idx, dist, K, &maxpos, c, d);
            }
        }
    }
    free(old);
}

/* ------------------------------------------------------------------ */
/* forest = the C-ABI call of the reference (rsfk.cu:2033-2183)        */
/* ------------------------------------------------------------------ */

/*
 * log_forest (may be NULL): float[16*n_trees+2], series-major, same layout as
 * the reference (rsfk.cu:2148-2173).  Only the four integer series, the total
 * tree time, the K-NN time and the two tail scalars are filled.
 */
RSFK_OR_EXPORT int rsfk_or_forest(int n_trees, int K, int N, int D,
                                  int MIN, int MAX, int MAX_DEPTH, int seed, int nnef,
                                  const float* points, int* knn_idx, float* knn_dist,
                                  float* log_forest)
{
    if (N <= 0 || n_trees < 0) return 0;
    int leaf_cap = N / (MIN > 0 ? MIN : 1) + 2;
    int nthreads = 1;
#ifdef _OPENMP
    nthreads = omp_get_max_threads();
#endif
    int batch = nthreads < n_trees ? nthreads : n_trees;
    if (batch < 1) batch = 1;
    /* keep the per-batch partitions below ~2 GiB */
    while (batch > 1 && (size_t)batch * (size_t)N * 4u > ((size_t)1 << 31)) --batch;
    int* perm = (int*)malloc(sizeof(int) * (size_t)N * batch);
    int* lstart = (int*)malloc(sizeof(int) * (size_t)leaf_cap * batch);
    int* lsize = (int*)malloc(sizeof(int) * (size_t)leaf_cap * batch);
    int* nl = (int*)malloc(sizeof(int) * batch);
    int* st = (int*)malloc(sizeof(int) * 3 * batch);
    double* tt = (double*)malloc(sizeof(double) * batch);
    if (log_forest) memset(log_forest, 0, sizeof(float) * ((size_t)16 * n_trees + 2));
    double t_forest0 = 0.0, t_expl = 0.0;
#ifdef _OPENMP
    t_forest0 = omp_get_wtime();
#endif
    int rc = 0;
    for (int t0 = 0; t0 < n_trees; t0 += batch) {
        int nb = n_trees - t0 < batch ? n_trees - t0 : batch;
#pragma omp parallel for schedule(dynamic, 1)
        for (int j = 0; j < nb; ++j) {
            double a = 0.0;
#ifdef _OPENMP
            a = omp_get_wtime();
#endif
            nl[j] = rsfk_or_build_tree(points, N, D, MIN, MAX, MAX_DEPTH, seed + t0 + j,
                                       perm + (size_t)j * N, lstart + (size_t)j * leaf_cap,
                                       lsize + (size_t)j * leaf_cap, leaf_cap, st + 3 * j);
#ifdef _OPENMP
            tt[j] = omp_get_wtime() - a;
#else
            tt[j] = a;
#endif
        }
        for (int j = 0; j < nb; ++j) {
            if (nl[j] < 0) { rc = -1; continue; }
            double a = 0.0, e = 0.0;
#ifdef _OPENMP
            a = omp_get_wtime();
#endif
            rsfk_or_bucket_knn(points, N, D, K, perm + (size_t)j * N, lstart + (size_t)j * leaf_cap,
                               lsize + (size_t)j * leaf_cap, nl[j], 0, knn_idx, knn_dist);
#ifdef _OPENMP
            e = omp_get_wtime() - a;
#endif
            if (log_forest) {
                int t = t0 + j;
                log_forest[0 * n_trees + t] = (float)st[3 * j + 0];
                log_forest[1 * n_trees + t] = (float)st[3 * j + 1];
                log_forest[2 * n_trees + t] = (float)st[3 * j + 2];
                log_forest[3 * n_trees + t] = (float)nl[j];
                log_forest[5 * n_trees + t] = (float)tt[j];
                log_forest[15 * n_trees + t] = (float)e;
            }
        }
    }
#ifdef _OPENMP
    t_forest0 = omp_get_wtime() - t_forest0;
    t_expl = omp_get_wtime();
#endif
    for (int it = 0; it < nnef; ++it) rsfk_or_explore(points, N, D, K, knn_idx, knn_dist);
#ifdef _OPENMP
    t_expl = omp_get_wtime() - t_expl;
#endif
    if (log_forest) {
        log_forest[(size_t)16 * n_trees] = (float)t_forest0;
        log_forest[(size_t)16 * n_trees + 1] = (float)t_expl;
    }
    free(perm); free(lstart); free(lsize); free(nl); free(st); free(tt);
    return rc;
}

/* ------------------------------------------------------------------ */
/* exact K-NN by brute force (ground truth for recall)                 */
/* ------------------------------------------------------------------ */

/* For each query row id in queries[0..nq): the K nearest points (the query
 * itself included), fp64 distances, ties broken by smaller index; sorted. */
/*
 * Query-set search (RSFK::knn_gpu_rsfk_forest_ann, src/rsfk.cu:98-155): for every tree (seed + tree index, as in
 * the forest above) the queries are routed to a leaf and every point of that leaf is offered to the query's
 * row (compute_knn_from_buckets_perwarp_coalesced_ann, src/kernels/build_tree_update_parents_ann.cu:239-517,
 * update rule as everywhere).  Indices in q_idx refer to `points`.  No exploration pass (the reference accepts
 * the parameter and ignores it).  Distances use the sequential chain of rsfk_or_sqdist like every other
 * stage here; the reference's kernel uses its 32-lane form for this one.
 */
RSFK_OR_EXPORT int rsfk_or_ann_forest(int n_trees, int K, int N, int NQ, int D,
                                      int MIN, int MAX, int MAX_DEPTH, int seed,
                                      const float* points, const float* queries,
                                      int* q_idx, float* q_dist)
{
    int* perm = (int*)malloc(sizeof(int) * (size_t)(N > 0 ? N : 1));
    int* qs = (int*)malloc(sizeof(int) * (size_t)(NQ > 0 ? NQ : 1));
    int* qz = (int*)malloc(sizeof(int) * (size_t)(NQ > 0 ? NQ : 1));
    for (int t = 0; t < n_trees; ++t) {
        rsfk_or_route_queries(points, N, D, MIN, MAX, MAX_DEPTH, seed + t, queries, NQ, perm, qs, qz);
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 64)
#endif
        for (int q = 0; q < NQ; ++q) {
            int* idx = q_idx + (size_t)q * K;
            float* dist = q_dist + (size_t)q * K;
            int maxpos = row_max(idx, dist, K);
            for (int i = 0; i < qz[q]; ++i) {
                int c = perm[qs[q] + i];
                float d = rsfk_or_sqdist(queries + (size_t)q * D, points + (size_t)c * D, D);
                try_insert(idx, dist, K, &maxpos, c, d);
            }
        }
    }
    free(perm); free(qs); free(qz);
    return 0;
}

/*
 * Symmetrised K-NN graph in compressed-row form (the commented-out kernels symmetric_knn_graph_edge_count /
 * _offset / _add_edges, src/rsfk.cu:1229-1299): every stored edge p -> c goes into row p; if row c does not store p
 * the reverse edge goes into row c (line 1243-1249 / 1287-1296: "force the bidirectional edge if it doesn't exist").
 * Differences: slots that are negative or >= N are skipped (the reference would read out of range), drop_self
 * removes p from its own row, and the columns of a row are sorted ascending (the reference leaves the arrival order
 * of atomics).  indptr: N + 1; cols / vals: capacity cap or NULL (count only).  Returns the number of entries, or
 * -1 when cap is too small.
 */
typedef struct { int col; float val; } or_edge;
static int or_edge_cmp(const void* a, const void* b)
{
    int ca = ((const or_edge*)a)->col, cb = ((const or_edge*)b)->col;
    return (ca > cb) - (ca < cb);
}

RSFK_OR_EXPORT long long rsfk_or_symmetrize(const int* idx, const float* dist, int N, int K, int drop_self,
                                            int* indptr, int* cols, float* vals, long long cap)
{
    long long* len = (long long*)calloc((size_t)N + 1, sizeof(long long));
    for (int pass = 0; pass < 2; ++pass) {
        if (pass == 1) {
            long long run = 0;
            for (int p = 0; p <= N; ++p) { long long l = len[p]; indptr[p] = (int)run; len[p] = run; run += l; }
            if (!cols) { free(len); return run; }
            if (run > cap) { free(len); return -1; }
        }
        for (int p = 0; p < N; ++p) {
            for (int k = 0; k < K; ++k) {
                int c = idx[(size_t)p * K + k];
                if (c < 0 || c >= N || (drop_self && c == p)) continue;
                float d = dist ? dist[(size_t)p * K + k] : 0.0f;
                int mutual = 0;
                for (int j = 0; j < K; ++j) mutual |= idx[(size_t)c * K + j] == p;
                if (pass == 0) {
                    len[p]++;
                    if (!mutual) len[c]++;
                } else {
                    cols[len[p]] = c; vals[len[p]] = d; len[p]++;
                    if (!mutual) { cols[len[c]] = p; vals[len[c]] = d; len[c]++; }
                }
            }
        }
    }
    long long total = indptr[N];
    or_edge* tmp = (or_edge*)malloc(sizeof(or_edge) * (size_t)(2 * K + 1));
    size_t tmp_cap = (size_t)(2 * K + 1);
    for (int p = 0; p < N; ++p) {
        size_t n = (size_t)(indptr[p + 1] - indptr[p]);
        if (n > tmp_cap) { tmp_cap = n; tmp = (or_edge*)realloc(tmp, sizeof(or_edge) * tmp_cap); }
        for (size_t i = 0; i < n; ++i) { tmp[i].col = cols[indptr[p] + i]; tmp[i].val = vals[indptr[p] + i]; }
        qsort(tmp, n, sizeof(or_edge), or_edge_cmp);
        for (size_t i = 0; i < n; ++i) { cols[indptr[p] + i] = tmp[i].col; vals[indptr[p] + i] = tmp[i].val; }
    }
    free(tmp); free(len);
    return total;
}

RSFK_OR_EXPORT void rsfk_or_bruteforce(const float* points, int N, int D, int K,
                                       const int* queries, int nq,
                                       int* out_idx, double* out_dist)
{
#pragma omp parallel for schedule(dynamic, 8)
    for (int qi = 0; qi < nq; ++qi) {
        int q = queries ? queries[qi] : qi;
        int* oi = out_idx + (size_t)qi * K;
        double* od = out_dist + (size_t)qi * K;
        int cnt = 0;
        for (int j = 0; j < N; ++j) {
            double d = rsfk_or_sqdist_f64(points + (size_t)q * D, points + (size_t)j * D, D);
            if (cnt == K && !(d < od[K - 1])) continue;
            int pos = cnt < K ? cnt : K - 1;
            while (pos > 0 && od[pos - 1] > d) { od[pos] = od[pos - 1]; oi[pos] = oi[pos - 1]; --pos; }
            od[pos] = d; oi[pos] = j;
            if (cnt < K) ++cnt;
        }
        for (int k = cnt; k < K; ++k) { oi[k] = -1; od[k] = INFINITY; }
    }
}

RSFK_OR_EXPORT int rsfk_or_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

RSFK_OR_EXPORT void rsfk_or_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
