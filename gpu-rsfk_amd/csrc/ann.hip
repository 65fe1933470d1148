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
//
// The queries are then grouped by the bucket they reached (a count per bucket taken while routing, a scan, a fill)
// and a workgroup works on one bucket and up to 16 of its queries: the rows of the bucket pass through LDS once per
// workgroup instead of once per query, every lane runs the sequential chain of "its" bucket member against four
// queries whose coordinates are wavefront-uniform, and the candidates are merged into the queries' rows.
#include "forest.hpp"
#include "exact_batch.hpp"
#include <algorithm>

namespace rsfk {

namespace {

constexpr int kQB = 16;               // queries per workgroup
constexpr int kQW = 4;                // queries a wavefront works on together
constexpr int kCG = 128;              // bucket members per pass: two per lane
constexpr int kCH = 32;               // dimensions per staging step
constexpr int kTP = kCH + 4;          // tile pitch: odd number of 16-byte units
constexpr int kPieces = kCH / 4;      // 16-byte pieces of a row per staging step = lanes per row
constexpr int kRowsPer = 256 / kPieces;   // rows per load instruction of the workgroup
constexpr int kLoads = kCG / kRowsPer;    // load instructions per staging step

__global__ __launch_bounds__(256) void k_zero_ints(int* __restrict__ p, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Hyperplane of every two-child node of the index, one wavefront per record: row r of `planes` (pitch floats) is
// [offset, 0, 0, 0 | normal, zero padded to a multiple of 4].  Normal and offset are the values the builder works with
// (create_node.cu:122-135: n = x1 - x2, offset = sum n_d (x1_d + x2_d) / 2 as 32 lane-strided partial sums + xor butterfly).
__global__ __launch_bounds__(256) void k_planes(const float* __restrict__ points, int D, const TreeRec* __restrict__ recs,
                                                const int* __restrict__ n_rec_p, int rec_cap, float* __restrict__ planes,
                                                int pitch)
{
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= min(*n_rec_p, rec_cap)) return;
    const TreeRec rec = recs[r];
    if (rec.c0 < 0) return;
    const float* x1 = points + (size_t)rec.a * (size_t)D;
    const float* x2 = points + (size_t)rec.b * (size_t)D;
    float* row = planes + (size_t)r * (size_t)pitch;
    float s = 0.0f;
    if (lane < 32) {
        for (int d = lane; d < D; d += 32) {
            const float t1 = x1[d], t2 = x2[d];
            const float nd = t1 - t2;
            const float prod = nd * (t1 + t2);
            s = s + prod * 0.5f;
        }
    }
    s = half_butterfly_sum(s);
    if (lane < 4) row[lane] = lane == 0 ? s : 0.0f;
    for (int d = lane; d < pitch - 4; d += 64) row[4 + d] = d < D ? x1[d] - x2[d] : 0.0f;
}

// Eight lanes per query.  A lane owns four of the 32 partial sums of the side test (sums 4s..4s+3 of
// build_tree_check_points_side.cu:131-149: sum j takes the dimensions j, j+32, ... in turn) and adds them in the order
// of the xor butterfly; the other three steps of the butterfly run over the eight lanes.  The first 128 dimensions of
// the query stay in registers.  q_rec[q] = record of the bucket reached, q_rank[q] = arrival number of q among the
// queries of that bucket (cnt counts them).
constexpr int kXR = 4;
template <bool VEC>
__global__ __launch_bounds__(256) void k_route(const float* __restrict__ planes, int pitch, const float* __restrict__ queries,
                                               int NQ, int D, const TreeRec* __restrict__ recs, int max_steps,
                                               int* __restrict__ q_rec, int* __restrict__ q_rank, int* __restrict__ cnt)
{
    const int sub = threadIdx.x & 7;
    const int q = (int)((blockIdx.x * (size_t)blockDim.x + threadIdx.x) >> 3);
    const bool valid = q < NQ;
    const float* x = queries + (size_t)(valid ? q : 0) * (size_t)D;
    const int Dp = pitch - 4;
    float4 xr[kXR];
#pragma unroll
    for (int k = 0; k < kXR; ++k) xr[k] = load_piece(x, 32 * k + 4 * sub, D, VEC);
    int cur = 0;
    bool done = !valid;
    for (int step = 0; step <= max_steps; ++step) {          // a path is never longer than the number of records
        const int at = done ? 0 : cur;
        const TreeRec r = recs[at];
        const float* pl = planes + (size_t)at * (size_t)pitch;   // requested together with the record; unused for a bucket
        const float b = pl[0];
        float4 n4[kXR];
#pragma unroll
        for (int k = 0; k < kXR; ++k) {
            const int d = 32 * k + 4 * sub;
            n4[k] = d < Dp ? *reinterpret_cast<const float4*>(pl + 4 + d) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll
        for (int k = 0; k < kXR; ++k) {
            s0 = __builtin_fmaf(n4[k].x, xr[k].x, s0);
            s1 = __builtin_fmaf(n4[k].y, xr[k].y, s1);
            s2 = __builtin_fmaf(n4[k].z, xr[k].z, s2);
            s3 = __builtin_fmaf(n4[k].w, xr[k].w, s3);
        }
        for (int d0 = 32 * kXR; d0 < D; d0 += 64) {            // two steps of the chains per trip
            const int da = d0 + 4 * sub, db = da + 32;
            const float4 na = da < Dp ? *reinterpret_cast<const float4*>(pl + 4 + da) : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 nb = db < Dp ? *reinterpret_cast<const float4*>(pl + 4 + db) : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 xa = load_piece(x, da, D, VEC), xb = load_piece(x, db, D, VEC);
            s0 = __builtin_fmaf(na.x, xa.x, s0); s1 = __builtin_fmaf(na.y, xa.y, s1);
            s2 = __builtin_fmaf(na.z, xa.z, s2); s3 = __builtin_fmaf(na.w, xa.w, s3);
            s0 = __builtin_fmaf(nb.x, xb.x, s0); s1 = __builtin_fmaf(nb.y, xb.y, s1);
            s2 = __builtin_fmaf(nb.z, xb.z, s2); s3 = __builtin_fmaf(nb.w, xb.w, s3);
        }
        float t = (s0 + s1) + (s2 + s3);
        t += dpp_f<kDppXor1>(t);
        t += dpp_f<kDppXor2>(t);
        t += dpp_f<kDppHalfMirror>(t);
        if (!done) {
            if (r.c0 < 0) {
                if (sub == 0) { q_rec[q] = cur; q_rank[q] = atomicAdd(&cnt[cur], 1); }
                done = true;
            } else {
                cur = t < b ? r.c1 : r.c0;
            }
        }
        if (ballot64(!done) == 0) break;
    }
}

// Scan over the records of the tree in tiles of 1024 (a workgroup each): qoff = exclusive scan of the query counts,
// boff = exclusive scan of the numbers of workgroups (16 queries each) the buckets need; both get a closing entry at
// index n_rec.  The two sums travel as the halves of one 64-bit value.
typedef unsigned long long u64;
constexpr int kScanTile = 1024;

__device__ __forceinline__ u64 pack_count(int c) { return (u64)(unsigned)c | ((u64)(unsigned)((c + kQB - 1) / kQB) << 32); }

// exclusive scan of 256 values, one per thread; *total = their sum
__device__ __forceinline__ u64 block_scan_256(u64 v, u64* total, u64* lds4)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    u64 incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const u64 t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
    }
    if (lane == 63) lds4[wave] = incl;
    __syncthreads();
    u64 woff = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) { const u64 x = lds4[w]; if (w < wave) woff += x; tot += x; }
    __syncthreads();
    *total = tot;
    return woff + incl - v;
}

__global__ __launch_bounds__(256) void k_ann_tile_sums(const int* __restrict__ cnt, const int* __restrict__ n_rec_p, int rec_cap,
                                                       u64* __restrict__ tile_sum)
{
    __shared__ u64 lds4[4];
    const int n = min(*n_rec_p, rec_cap);
    const int i0 = blockIdx.x * kScanTile + threadIdx.x * 4;
    u64 mine = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) mine += i0 + j < n ? pack_count(cnt[i0 + j]) : 0ull;
    u64 tot;
    (void)block_scan_256(mine, &tot, lds4);
    if (threadIdx.x == 0) tile_sum[blockIdx.x] = tot;
}

// Second step; also sets the counts back to zero for the next tree.
__global__ __launch_bounds__(256) void k_ann_scan(int* __restrict__ cnt, const int* __restrict__ n_rec_p, int rec_cap,
                                                  const u64* __restrict__ tile_sum, int* __restrict__ qoff,
                                                  int* __restrict__ boff, int* __restrict__ n_blocks)
{
    __shared__ u64 lds4[4];
    const int n = min(*n_rec_p, rec_cap);
    if (blockIdx.x * kScanTile > n) return;                  // index n itself still gets the closing entries
    u64 before = 0;
    for (int t = threadIdx.x; t < (int)blockIdx.x; t += 256) before += tile_sum[t];
    u64 base;
    (void)block_scan_256(before, &base, lds4);
    const int i0 = blockIdx.x * kScanTile + threadIdx.x * 4;
    u64 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = i0 + j < n ? pack_count(cnt[i0 + j]) : 0ull;
    u64 tot;
    u64 run = base + block_scan_256(v[0] + v[1] + v[2] + v[3], &tot, lds4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = i0 + j;
        if (i <= n) {
            qoff[i] = (int)(unsigned)(run & 0xffffffffull);
            boff[i] = (int)(unsigned)(run >> 32);
            if (i == n) *n_blocks = (int)(unsigned)(run >> 32);
            else cnt[i] = 0;
        }
        run += v[j];
    }
}

// Thread i < NQ puts query i into the list of its bucket; thread i < n_rec writes the descriptors of the workgroups of
// bucket i: {start and size of the bucket in the tree's permutation, first query in qlist, number of queries}.
__global__ __launch_bounds__(256) void k_ann_fill(int NQ, const int* __restrict__ q_rec, const int* __restrict__ q_rank,
                                                  const int* __restrict__ n_rec_p, int rec_cap, const TreeRec* __restrict__ recs,
                                                  const int* __restrict__ qoff, const int* __restrict__ boff,
                                                  int* __restrict__ qlist, int4* __restrict__ blk_desc)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < NQ) qlist[qoff[q_rec[i]] + q_rank[i]] = i;
    if (i < min(*n_rec_p, rec_cap)) {
        const int b0 = boff[i], b1 = boff[i + 1];
        if (b1 > b0) {
            const TreeRec rec = recs[i];
            const int q0 = qoff[i], q1 = qoff[i + 1];
            for (int b = b0; b < b1; ++b) {
                const int first = q0 + (b - b0) * kQB;
                blk_desc[b] = make_int4(rec.a, rec.b, first, min(kQB, q1 - first));
            }
        }
    }
}

__device__ __forceinline__ void chain4(float& acc, const float4& a, const float4& x)
{
    float df;
    df = a.x - x.x; acc = __builtin_fmaf(df, df, acc);
    df = a.y - x.y; acc = __builtin_fmaf(df, df, acc);
    df = a.z - x.z; acc = __builtin_fmaf(df, df, acc);
    df = a.w - x.w; acc = __builtin_fmaf(df, df, acc);
}

// Workgroup b works on the bucket and the (up to 16) queries of blk_desc[b].  Per staging step 32 dimensions of up to
// 128 bucket rows and of the 16 query rows pass through LDS; a lane reads "its" bucket rows (two: lane, lane + 64)
// with 16-byte reads and the queries' coordinates as broadcasts.  VEC: D is a multiple of 4 and both matrices are
// 16-byte aligned.
template <int SL, bool VEC>
__global__ __launch_bounds__(256) void k_ann_leaf(const float* __restrict__ points, const float* __restrict__ queries, int D,
                                                  int K, const int* __restrict__ perm, const int4* __restrict__ blk_desc,
                                                  const int* __restrict__ n_blocks, const int* __restrict__ qlist,
                                                  int* __restrict__ q_idx, float* __restrict__ q_dist)
{
    __shared__ __align__(16) float tile[kCG * kTP];
    __shared__ __align__(16) float xs[kQB * kCH];
    __shared__ int cand[kCG];
    __shared__ int qid_s[kQB];
    const int b = blockIdx.x;
    if (b >= *n_blocks) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int4 desc = blk_desc[b];
    const int start = desc.x, S = desc.y, q0 = desc.z, nq = desc.w;
    if (tid < kQB) qid_s[tid] = qlist[q0 + (tid < nq ? tid : 0)];      // slots beyond nq repeat the first query (ignored later)
    __syncthreads();

    int qid[kQW];
    bool qv[kQW];
    KnnRow<SL> row[kQW];
#pragma unroll
    for (int i = 0; i < kQW; ++i) {
        const int slot = i * 4 + wave;                        // queries are dealt out to the four wavefronts in turn
        qv[i] = slot < nq;
        qid[i] = __builtin_amdgcn_readfirstlane(qid_s[slot]);
        row[i].load(q_idx + (size_t)qid[i] * K, q_dist + (size_t)qid[i] * K, K);
    }
    const int nqw = (nq - wave + 3) >> 2;                     // queries of this wavefront (0..4), the first nqw slots

    const int piece = tid % kPieces, prow = tid / kPieces;    // staging: kPieces lanes per row
    const bool stage_x = tid < kQB * kPieces;
    const float* xp = queries + (size_t)qid_s[stage_x ? prow : 0] * (size_t)D;
    for (int c0 = 0; c0 < S; c0 += kCG) {
        const int nc = min(kCG, S - c0);
        __syncthreads();                                      // the previous pass is done with cand
        if (tid < kCG) cand[tid] = tid < nc ? perm[start + c0 + tid] : -1;
        __syncthreads();
        const float* rp[kLoads];
        float4 pre[kLoads];
        float4 prex = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int rr = prow + kRowsPer * i;
            rp[i] = points + (size_t)cand[rr < nc ? rr : 0] * (size_t)D;       // rows beyond nc repeat row 0 (ignored later)
            pre[i] = load_piece(rp[i], piece * 4, D, VEC);
        }
        if (stage_x) prex = load_piece(xp, piece * 4, D, VEC);
        float acc0[kQW], acc1[kQW];
#pragma unroll
        for (int i = 0; i < kQW; ++i) { acc0[i] = 0.0f; acc1[i] = 0.0f; }
        const bool two = nc > 64;
        for (int d0 = 0; d0 < D; d0 += kCH) {
            __syncthreads();                                  // tile reads of the previous step are done
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                *reinterpret_cast<float4*>(&tile[(prow + kRowsPer * i) * kTP + piece * 4]) = pre[i];
            if (stage_x) *reinterpret_cast<float4*>(&xs[prow * kCH + piece * 4]) = prex;
            if (d0 + kCH < D) {
#pragma unroll
                for (int i = 0; i < kLoads; ++i) pre[i] = load_piece(rp[i], d0 + kCH + piece * 4, D, VEC);
                if (stage_x) prex = load_piece(xp, d0 + kCH + piece * 4, D, VEC);
            }
            __syncthreads();
            const int pieces = min(kPieces, (D - d0 + 3) >> 2);
            const float* m0 = &tile[lane * kTP];
            const float* m1 = &tile[(lane + 64) * kTP];
            const float* x0 = &xs[wave * kCH];                // slot i * 4 + wave: stride 4 rows
            if (nqw > 2) {
                for (int p = 0; p < pieces; ++p) {
                    float4 xv[kQW];
#pragma unroll
                    for (int i = 0; i < kQW; ++i) xv[i] = *reinterpret_cast<const float4*>(x0 + i * 4 * kCH + 4 * p);
                    const float4 a0 = *reinterpret_cast<const float4*>(m0 + 4 * p);
#pragma unroll
                    for (int i = 0; i < kQW; ++i) chain4(acc0[i], a0, xv[i]);
                    if (two) {
                        const float4 a1 = *reinterpret_cast<const float4*>(m1 + 4 * p);
#pragma unroll
                        for (int i = 0; i < kQW; ++i) chain4(acc1[i], a1, xv[i]);
                    }
                }
            } else if (nqw > 0) {
                for (int p = 0; p < pieces; ++p) {
                    float4 xv[2];
#pragma unroll
                    for (int i = 0; i < 2; ++i) xv[i] = *reinterpret_cast<const float4*>(x0 + i * 4 * kCH + 4 * p);
                    const float4 a0 = *reinterpret_cast<const float4*>(m0 + 4 * p);
#pragma unroll
                    for (int i = 0; i < 2; ++i) chain4(acc0[i], a0, xv[i]);
                    if (two) {
                        const float4 a1 = *reinterpret_cast<const float4*>(m1 + 4 * p);
#pragma unroll
                        for (int i = 0; i < 2; ++i) chain4(acc1[i], a1, xv[i]);
                    }
                }
            }
        }
        const int c_lo = cand[lane], c_hi = cand[lane + 64];
#pragma unroll
        for (int i = 0; i < kQW; ++i) {
            if (qv[i]) {
                const bool okv[2] = {lane < nc, two && lane + 64 < nc};
                const int cv[2] = {c_lo, c_hi};
                const float dv[2] = {acc0[i], acc1[i]};
                row[i].template merge<2>(okv, cv, dv);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kQW; ++i)
        if (qv[i] && row[i].changed) row[i].store(q_idx + (size_t)qid[i] * K, q_dist + (size_t)qid[i] * K);
}

}  // namespace

// floats per row of the table of hyperplanes: offset (4 floats) + normal padded to a multiple of 4
int ann_plane_pitch(int D) { return 4 + ((D + 3) & ~3); }

size_t ann_ws_ints(int NQ, int rec_cap)
{
    // q_rec | q_rank | qlist (NQ each) | cnt (rec_cap) | qoff | boff (rec_cap + 1 each) | descriptors of the workgroups
    // (4 ints each, 16-byte aligned) | n_blocks (4) | tile sums
    return (size_t)3 * NQ + (size_t)rec_cap + 2 * ((size_t)rec_cap + 1) + 4 + 4 * ((size_t)NQ / kQB + rec_cap + 1) + 4 +
           2 * ((size_t)rec_cap / kScanTile + 2);
}

// First use of a workspace: the bucket counters start at zero (every tree leaves them so).
int launch_ann_ws_init(int* ws, int NQ, int rec_cap, hipStream_t stream)
{
    int* cnt = ws + (size_t)3 * NQ;
    hipLaunchKernelGGL(k_zero_ints, dim3((unsigned)((rec_cap + 255) / 256)), dim3(256), 0, stream, cnt, rec_cap);
    RSFK_HIP(hipGetLastError());
    return 0;
}

// One tree of the query-set search: routes the queries through the index recs (*n_rec_dev records, at most rec_cap;
// the tree has n_leaves buckets), groups them by bucket and offers the base points perm[..] of the bucket a query
// reached to the query's row.  ws: ann_ws_ints(NQ, rec_cap) ints, prepared by launch_ann_ws_init; planes: rec_cap rows of
// ann_plane_pitch(D) floats.
int launch_ann_tree(const float* points, const float* queries, int NQ, int D, int K, const int* perm, const TreeRec* recs,
                    const int* n_rec_dev, int rec_cap, int n_leaves, int* ws, float* planes, int* q_idx, float* q_dist,
                    hipStream_t stream)
{
    if (NQ <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= kMaxK, "query-set search: K must be in 1..1024");
    RSFK_CHECK(recs != nullptr && rec_cap >= 1, "query-set search: the tree has no index");
    int* q_rec = ws;
    int* q_rank = q_rec + NQ;
    int* qlist = q_rank + NQ;
    int* cnt = qlist + NQ;
    int* qoff = cnt + rec_cap;
    int* boff = qoff + rec_cap + 1;
    int4* blk_desc = reinterpret_cast<int4*>(ws + (((boff + rec_cap + 1) - ws + 3) & ~(ptrdiff_t)3));
    int* n_blocks = reinterpret_cast<int*>(blk_desc + ((size_t)NQ / kQB + rec_cap + 1));
    u64* tile_sum = reinterpret_cast<u64*>(ws + ((ann_ws_ints(NQ, rec_cap) - 2 * ((size_t)rec_cap / kScanTile + 2)) & ~(size_t)1));
    const int pitch = ann_plane_pitch(D);
    hipLaunchKernelGGL(k_planes, dim3((unsigned)((rec_cap + 3) / 4)), dim3(256), 0, stream, points, D, recs, n_rec_dev, rec_cap,
                       planes, pitch);
    const unsigned g_route = (unsigned)(((size_t)NQ * 8 + 255) / 256);
    const bool vec_q = (D & 3) == 0 && (reinterpret_cast<uintptr_t>(queries) & 15) == 0;
    if (vec_q)
        hipLaunchKernelGGL(k_route<true>, dim3(g_route), dim3(256), 0, stream, planes, pitch, queries, NQ, D, recs, rec_cap, q_rec,
                           q_rank, cnt);
    else
        hipLaunchKernelGGL(k_route<false>, dim3(g_route), dim3(256), 0, stream, planes, pitch, queries, NQ, D, recs, rec_cap, q_rec,
                           q_rank, cnt);
    const unsigned g_scan = (unsigned)(rec_cap / kScanTile + 1);
    hipLaunchKernelGGL(k_ann_tile_sums, dim3(g_scan), dim3(256), 0, stream, cnt, n_rec_dev, rec_cap, tile_sum);
    hipLaunchKernelGGL(k_ann_scan, dim3(g_scan), dim3(256), 0, stream, cnt, n_rec_dev, rec_cap, tile_sum, qoff, boff, n_blocks);
    const unsigned g_fill = (unsigned)((std::max(NQ, rec_cap) + 255) / 256);
    hipLaunchKernelGGL(k_ann_fill, dim3(g_fill), dim3(256), 0, stream, NQ, q_rec, q_rank, n_rec_dev, rec_cap, recs, qoff, boff, qlist,
                       blk_desc);
    // a bucket with c queries takes ceil(c / 16) workgroups: at most NQ / 16 + (buckets with queries) in all
    const unsigned g_leaf = (unsigned)(NQ / kQB + std::min(n_leaves, NQ) + 1);
    const bool vec = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) | reinterpret_cast<uintptr_t>(queries)) & 15) == 0;
#define RSFK_ANN_CASE(SLV)                                                                                                   \
    {                                                                                                                        \
        if (vec)                                                                                                             \
            hipLaunchKernelGGL((k_ann_leaf<SLV, true>), dim3(g_leaf), dim3(256), 0, stream, points, queries, D, K, perm,       \
                               blk_desc, n_blocks, qlist, q_idx, q_dist);                                        \
        else                                                                                                                 \
            hipLaunchKernelGGL((k_ann_leaf<SLV, false>), dim3(g_leaf), dim3(256), 0, stream, points, queries, D, K, perm,       \
                               blk_desc, n_blocks, qlist, q_idx, q_dist);                                        \
    }
    if (K <= 64) RSFK_ANN_CASE(1)
    else if (K <= 128) RSFK_ANN_CASE(2)
    else if (K <= 256) RSFK_ANN_CASE(4)
    else if (K <= 512) RSFK_ANN_CASE(8)
    else RSFK_ANN_CASE(16)
#undef RSFK_ANN_CASE
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
