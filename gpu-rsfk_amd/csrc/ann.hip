// Query-set search: query points are routed through a tree built on the base points and every base point
// of the leaf a query reaches is offered to the query's K-NN row.  Replaces the per-tree part of
// RSFK::knn_gpu_rsfk_forest_ann_tree (src/rsfk.cu:262-441): the level loop that moves the queries down
// (build_tree_check_active_points / build_tree_check_points_side / build_tree_update_parents_ann, one launch and
// one device synchronisation each per level) and compute_knn_from_buckets_perwarp_coalesced_ann
// (src/kernels/build_tree_update_parents_ann.cu:239-517).
//
// The tree builder records an index of each tree on request (TreeRec: the drawn pair and the children of every
// node, the segment of every bucket), so a query descends the whole tree in one kernel: a half wavefront per
// query recomputes the hyperplane of a node from its pair and takes the side test with the arithmetic of the
// builder (32 lane-strided partial sums + xor butterfly: build_tree_check_points_side.cu:131-149,
// create_node.cu:122-135); a node with one child (empty side, or the min-size merge) needs no test and is not in
// the index.
#include "forest.hpp"
#include "exact_batch.hpp"
#include <algorithm>

namespace rsfk {

namespace {

__global__ __launch_bounds__(256) void k_route(const float* __restrict__ points, const float* __restrict__ queries, int NQ,
                                               int D, const TreeRec* __restrict__ recs, int max_steps,
                                               int* __restrict__ q_start, int* __restrict__ q_size)
{
    const int hl = threadIdx.x & 31;
    const int q = (int)((blockIdx.x * (size_t)blockDim.x + threadIdx.x) >> 5);
    const bool valid = q < NQ;
    const float* x = queries + (size_t)(valid ? q : 0) * (size_t)D;
    int cur = 0;
    bool done = !valid;
    for (int step = 0; step <= max_steps; ++step) {      // a path is never longer than the number of records
        const TreeRec r = recs[done ? 0 : cur];
        if (!done && r.c0 < 0) {
            if (hl == 0) { q_start[q] = r.a; q_size[q] = r.b; }
            done = true;
        }
        if (ballot64(!done) == 0) break;
        const bool test = !done && r.c0 != r.c1;
        float sb = 0.0f, sd = 0.0f;
        if (test) {
            const float* x1 = points + (size_t)r.a * (size_t)D;
            const float* x2 = points + (size_t)r.b * (size_t)D;
            for (int d0 = hl; d0 < D; d0 += 256) {            // loads of eight steps of the chains together
                float a1[8], a2[8], xv[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int d = d0 + 32 * k;
                    a1[k] = d < D ? x1[d] : 0.0f;
                    a2[k] = d < D ? x2[d] : 0.0f;
                    xv[k] = d < D ? x[d] : 0.0f;
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    if (d0 + 32 * k < D) {
                        const float nd = a1[k] - a2[k];
                        const float prod = nd * (a1[k] + a2[k]);
                        sb = sb + prod * 0.5f;
                        sd = __builtin_fmaf(nd, xv[k], sd);
                    }
                }
            }
        }
        sb = half_butterfly_sum(sb);
        sd = half_butterfly_sum(sd);
        if (!done) cur = (test && sd < sb) ? r.c1 : r.c0;
    }
}

// One wavefront per query.  Per-wavefront LDS (ints): tile[64 * 20] | xrow[dpad].
constexpr int kAnnChunk = 16;
constexpr int kAnnTile = 64 * (kAnnChunk + 4);

template <int SL, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void k_ann_knn(const float* __restrict__ points, const float* __restrict__ queries,
                                                         int NQ, int D, int K, const int* __restrict__ perm,
                                                         const int* __restrict__ q_start, const int* __restrict__ q_size,
                                                         int* __restrict__ q_idx, float* __restrict__ q_dist, int dpad,
                                                         int wave_lds_ints)
{
    extern __shared__ __align__(16) int lds_a[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int q = blockIdx.x * WAVES + wave;
    if (q >= NQ) return;                                  // whole wavefront leaves together
    int* base = lds_a + (size_t)wave * (size_t)wave_lds_ints;
    ExploreLds L;
    L.tile = reinterpret_cast<float*>(base);
    L.xrow = reinterpret_cast<float*>(base + kAnnTile);
    L.queue2 = nullptr;
    L.table = nullptr;
    L.srow = nullptr;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int start = q_start[q], size = q_size[q];
    if (size <= 0) return;
    KnnRow<SL> row;
    row.load(q_idx + (size_t)q * K, q_dist + (size_t)q * K, K);
    const float* xq = queries + (size_t)q * D;
    for (int d = lane; d < dpad; d += 64) L.xrow[d] = d < D ? xq[d] : 0.0f;
    for (int off = 0; off < size; off += 64) {
        wave_lds_sync();
        exact_batch<SL, kAnnChunk>(L, perm + start + off, min(64, size - off), points, D, vec_ok, row);
    }
    if (row.changed) row.store(q_idx + (size_t)q * K, q_dist + (size_t)q * K);
}

}  // namespace

// Leaf of every query in the tree with the index recs (n_rec records): its segment of the tree's permutation.
int launch_route_queries(const float* points, const float* queries, int NQ, int D, const TreeRec* recs, int n_rec,
                         int* q_start, int* q_size, hipStream_t stream)
{
    if (NQ <= 0) return 0;
    RSFK_CHECK(recs != nullptr && n_rec >= 1, "query routing: the tree has no index");
    const unsigned grid = (unsigned)(((size_t)NQ * 32 + 255) / 256);
    hipLaunchKernelGGL(k_route, dim3(grid), dim3(256), 0, stream, points, queries, NQ, D, recs, n_rec, q_start, q_size);
    RSFK_HIP(hipGetLastError());
    return 0;
}

// Offers the base points perm[q_start[q] .. + q_size[q]) to the row of every query q.
int launch_ann_knn(const float* points, const float* queries, int NQ, int D, int K, const int* perm, const int* q_start,
                   const int* q_size, int* q_idx, float* q_dist, hipStream_t stream)
{
    if (NQ <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 256, "query-set search: K must be in 1..256");
    constexpr int kWaves = 4;
    const int dpad = (D + 7) & ~7;
    const int wave_ints = (kAnnTile + dpad + 3) & ~3;
    const size_t lds = (size_t)kWaves * (size_t)wave_ints * sizeof(int);
    RSFK_CHECK(lds <= 150 * 1024, "query-set search: D too large for the LDS budget");
    const dim3 grid((unsigned)((NQ + kWaves - 1) / kWaves)), block(64 * kWaves);
#define RSFK_ANN_CASE(SLV)                                                                                              \
    {                                                                                                                   \
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_ann_knn<SLV, kWaves>),                             \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                            \
        hipLaunchKernelGGL((k_ann_knn<SLV, kWaves>), grid, block, lds, stream, points, queries, NQ, D, K, perm, q_start, \
                           q_size, q_idx, q_dist, dpad, wave_ints);                                                     \
    }
    if (K <= 64) RSFK_ANN_CASE(1)
    else if (K <= 128) RSFK_ANN_CASE(2)
    else RSFK_ANN_CASE(4)
#undef RSFK_ANN_CASE
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
