// Random-sample tree building for a batch of trees, level-synchronous.
//
// Replaces the reference's per-level kernel chain of
// RSFK::create_bucket_from_sample_tree (src/rsfk.cu:500-1207):
// build_tree_init, build_tree_check_active_points, build_tree_check_points_side,
// build_tree_count_new_nodes, build_tree_accumulate_child_count,
// build_tree_organize_sample_candidates, build_tree_create_nodes,
// build_tree_update_parents, build_tree_post_update_parents, build_tree_utils,
// build_tree_fix, build_tree_max_leaf_size, build_tree_set_leaves_idx and
// build_tree_bucket_points (src/kernels/build_tree_*.cu, create_node.cu).
//
// Representation: every tree keeps a permutation of 0..N-1 in which each node
// is a contiguous segment; splitting a node is a stable partition of its
// segment (left members first).  There are no per-point parent/depth arrays
// and no per-point atomics.
//
//   wide phase : nodes larger than `small` points.  Each level is three
//                launches over all trees of the batch: (1) hyperplane + side
//                test + per-chunk left counts, (2) stable scatter with
//                wave64 ballot / mbcnt ranks, child creation by the chunk-0
//                workgroup of each node, (3) chunk bookkeeping for the next
//                level.
//   tail phase : one workgroup finishes the whole subtree of a node with at
//                most `small` points inside LDS (all the re-draw levels that
//                the min/max rule causes touch only such nodes).
//
// Arithmetic follows the reference bit for bit: the hyperplane offset and the
// side test are sums of 32 lane-strided partials combined by the xor butterfly
// (create_node.cu:122-135, build_tree_check_points_side.cu:131-149); a half
// wavefront plays the role of the 32-lane warp.
#include "rsfk_common.hpp"
#include "wave64.hpp"
#include "bf16.hpp"
#include "tree_sweep.hpp"
#include <vector>
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <chrono>

namespace rsfk {

namespace {

constexpr int kBlock = 256;


struct LevelCounters {
    int n_next;        // nodes appended for the next wide level
    int n_tail;        // tail tasks appended so far
    int n_chunks;      // chunks of the current level (written by the scan kernel)
    int overflow;      // set when a queue capacity is exceeded
    // time spent in the three steps of the wide levels (hyperplanes, side tests, scatter), in ticks of the device's
    // constant-rate clock: the first thread of a kernel that opens a step closes the one before it
    long long last_tick;
    long long phase_ticks[3];
};

// Counts for the report of a build (how many points the side tests of all levels looked at, and how many of them
// the screen left to the exact test): kStatSlots slots a cache line apart, so that the workgroups' additions do not
// all go to one address; slot s holds [points, undecided points] at stat[kStatPitch * s + 0 / 1].
constexpr int kStatSlots = 64, kStatPitch = 32;
__device__ __forceinline__ void stat_add(unsigned long long* stat, int slot, int which, int v)
{
    if (stat && v) atomicAdd(&stat[kStatPitch * (slot & (kStatSlots - 1)) + which], (unsigned long long)v);
}

// ended: the step that ends where the calling kernel begins (-1: none, the clock is only started)
__device__ __forceinline__ void phase_tick(LevelCounters* ctr, int ended)
{
    const long long now = (long long)wall_clock64();
    if (ended >= 0 && ctr->last_tick != 0) ctr->phase_ticks[ended] += now - ctr->last_tick;
    ctr->last_tick = now;
}

// ---------------------------------------------------------------------------
// helpers
// ---------------------------------------------------------------------------

// Length of a normal in LDS: zero padded to whole 16-byte pieces of either screening copy.
__host__ __device__ inline int nvec_len(int D) { return (D + 15) & ~15; }

// Hyperplane of (x1,x2) by one wavefront (all 64 lanes call): normal into LDS nvec[0..nvec_len(D)), and
// hp[0] = offset (order of create_node.cu:122-135: 32 lane-strided partial sums + xor butterfly),
// hp[1] = an upper bound of the 1-norm of the normal, hp[2] = the sum of its components (any order: only the
// 8-bit screen uses them, with a margin).
__device__ __forceinline__ void make_hyperplane_wave(const float* __restrict__ x1, const float* __restrict__ x2,
                                                     int D, float* nvec, float* hp)
{
    const int lane = lane_id();
    const int Dn = nvec_len(D);
    const int hl = lane & 31;
    const bool lowh = lane < 32;
    // Both halves of the wavefront walk the dimensions hl, hl + 32, ... (the loads of eight steps are requested
    // together): the lower half forms the offset with the arithmetic of create_node.cu:122-135 and writes the normal,
    // the upper half the 1-norm and the sum of the components.
    float s = 0.0f, s2 = 0.0f;
    for (int d0 = hl; d0 < D; d0 += 256) {
        float t1[8], t2[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int d = d0 + 32 * k;
            t1[k] = d < D ? x1[d] : 0.0f;
            t2[k] = d < D ? x2[d] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int d = d0 + 32 * k;
            if (d < D) {
                const float nd = t1[k] - t2[k];
                if (lowh) {
                    nvec[d] = nd;
                    const float prod = nd * (t1[k] + t2[k]);
                    s = s + prod * 0.5f;
                } else {
                    s += fabsf(nd);
                    s2 += nd;
                }
            }
        }
    }
    for (int d = D + lane; d < Dn; d += 64) nvec[d] = 0.0f;
    s = half_butterfly_sum(s);
    s2 = half_butterfly_sum(s2);
    if (lane == 0) hp[0] = s;
    if (lane == 32) { hp[1] = s * 1.001f; hp[2] = s2; }
}

// Screen of the side test for eight points per wavefront (right = n.x < b): lanes 8g..8g+7 work on
// the point of group g; all lanes of a group return its answer.  (With the 8-bit copy and short rows a group may
// be LPP = 4 or 2 lanes: 16 or 32 points per wavefront.)
//
// The decision is always the one of the exact fp32 test (resolve_exact below: 32 lane-strided fused
// multiply-add chains + xor butterfly, build_tree_check_points_side.cu:131-149), but most points never
// touch their fp32 row: a bfloat16 copy of the row (half the bytes) gives an approximate n.x together
// with S~ = sum |n_d||x~_d|.  bfloat16 keeps 8 significant bits: rounding x to x~ (round to nearest)
// changes n.x by at most 2^-8 sum |n_d||x_d| <= 2^-8 (1+2^-7) S~, and the fp32 summations of the two
// paths are off by at most (D/8 + D/32 + 16) 2^-24 S~ together, so whenever |approx - b| exceeds
// `band` * S~ (band = 1.01 (2^-8 (1+2^-7) + (D/8 + D/32 + 16) 2^-24), computed by the caller) the sign of
// (n.x - b) is the same for the exact evaluation: right[u] is final.  Otherwise (a few per cent of the
// points; also NaN or infinite values, and every point when there is no bfloat16 copy) redo[u] is set and
// the caller hands the point to resolve_exact.
//
// NB points per group are handled per call, so that NB row gathers per lane are in flight before the
// first is needed (the loop over points is bound by the latency of these gathers otherwise).
//
// With the 8-bit copy (bf16.hpp) the row is 16 header bytes + one byte per coordinate: approx = lo sum_d n_d +
// scale sum_d n_d q_d, undecided band e1 ||n||_1 (hp1 = bound of the 1-norm, hp2 = sum of the components of the
// normal of the point's node).  Only lane 0 of a group holds the header, so only its right / redo are meaningful
// (with either copy the callers use lane 0 only).
template <int NB, bool Q8, int LPP = 8>
__device__ __forceinline__ void side_screen8(const float* nvec0, int nstride, const int (&j)[NB], const float (&b)[NB],
                                             const float (&hp1)[NB], const float (&hp2)[NB],
                                             const uint16_t* __restrict__ pb16, const uint8_t* __restrict__ q8,
                                             const int (&id)[NB], int D, float band,
                                             const bool (&valid)[NB], bool (&right)[NB], bool (&redo)[NB])
{
    if (Q8) {
        static_assert(LPP == 8 || LPP == 4 || LPP == 2, "lanes per point");
        const int sub = lane_id() & (LPP - 1);
#pragma unroll
        for (int u = 0; u < NB; ++u) { right[u] = false; redo[u] = valid[u]; }
        const size_t pitch = (size_t)q8_pitch(D);
        const int pieces = q8_padded(D) >> 4;
        float da[NB];
        uint4 head[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            da[u] = 0.0f;
            head[u] = make_uint4(0u, 0u, 0u, 0u);
            if (valid[u] && sub == 0) head[u] = *reinterpret_cast<const uint4*>(q8 + (size_t)id[u] * pitch);
        }
        for (int k = sub; k < pieces; k += LPP) {
            uint4 w[NB];
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                w[u] = make_uint4(0u, 0u, 0u, 0u);
                if (valid[u]) w[u] = *reinterpret_cast<const uint4*>(q8 + (size_t)id[u] * pitch + 16 + 16 * k);
            }
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const float* nvec = nvec0 + (size_t)j[u] * nstride + 16 * k;
                const uint32_t ww[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 nq = *reinterpret_cast<const float4*>(&nvec[4 * q]);
                    da[u] = __builtin_fmaf(nq.x, (float)((ww[q] >> 0) & 0xffu), da[u]);
                    da[u] = __builtin_fmaf(nq.y, (float)((ww[q] >> 8) & 0xffu), da[u]);
                    da[u] = __builtin_fmaf(nq.z, (float)((ww[q] >> 16) & 0xffu), da[u]);
                    da[u] = __builtin_fmaf(nq.w, (float)((ww[q] >> 24) & 0xffu), da[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            float d = da[u];
            d += dpp_f<kDppXor1>(d);
            if (LPP >= 4) d += dpp_f<kDppXor2>(d);
            if (LPP >= 8) d += dpp_f<kDppHalfMirror>(d);
            const float lo = __uint_as_float(head[u].y), scale = __uint_as_float(head[u].z), e1 = __uint_as_float(head[u].w);
            const float approx = __builtin_fmaf(scale, d, lo * hp2[u]);
            const bool certain = fabsf(approx - b[u]) > e1 * hp1[u];       // false if anything is NaN
            right[u] = approx < b[u];
            redo[u] = valid[u] && !certain;
        }
        return;
    }
    // hyperplane of point u of this group: normal nvec0 + j[u] * nstride, offset b[u] (groups may differ)
    const int lane = lane_id();
    const int sub = lane & 7;
#pragma unroll
    for (int u = 0; u < NB; ++u) { right[u] = false; redo[u] = valid[u]; }
    (void)hp1;
    (void)hp2;
    if (pb16 != nullptr) {
        const int Dv = bf16_valid(D);
        const size_t pitch = (size_t)bf16_pitch(D);
        float da[NB], sa[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) { da[u] = 0.0f; sa[u] = 0.0f; }
        for (int e = sub * 8; e < Dv; e += 64) {
            uint4 w[NB];
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                w[u] = make_uint4(0u, 0u, 0u, 0u);
                if (valid[u]) w[u] = *reinterpret_cast<const uint4*>(pb16 + (size_t)id[u] * pitch + e);
            }
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const float* nvec = nvec0 + (size_t)j[u] * nstride;
                const float4 n0 = *reinterpret_cast<const float4*>(&nvec[e]);
                const float4 n1 = *reinterpret_cast<const float4*>(&nvec[e + 4]);
                const uint32_t ww[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
                const float nn[8] = {n0.x, n0.y, n0.z, n0.w, n1.x, n1.y, n1.z, n1.w};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float x0 = __uint_as_float(ww[q] << 16);
                    const float x1 = __uint_as_float(ww[q] & 0xffff0000u);
                    da[u] = __builtin_fmaf(nn[2 * q], x0, da[u]);
                    da[u] = __builtin_fmaf(nn[2 * q + 1], x1, da[u]);
                    sa[u] = __builtin_fmaf(fabsf(nn[2 * q]), fabsf(x0), sa[u]);
                    sa[u] = __builtin_fmaf(fabsf(nn[2 * q + 1]), fabsf(x1), sa[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            // sum over the 8 lanes of the group (any order will do for the screen)
            float d = da[u], a = sa[u];
            d += dpp_f<kDppXor1>(d); d += dpp_f<kDppXor2>(d); d += dpp_f<kDppHalfMirror>(d);
            a += dpp_f<kDppXor1>(a); a += dpp_f<kDppXor2>(a); a += dpp_f<kDppHalfMirror>(a);
            const bool certain = fabsf(d - b[u]) > a * band + 1e-30f;
            right[u] = d < b[u];
            redo[u] = valid[u] && !certain;
        }
    }
}

// Exact side tests for the points the screen could not decide: n.x by one half wavefront (32 lanes, lane hl
// runs the chain over d = hl, hl + 32, ...; the loads of a chain are issued eight at a time), then the xor butterfly.  list[i] = position of the
// point (local to the caller) | slot of its node << 16.  One half wavefront per point, two points per half
// wavefront at a time so that their row loads overlap; all threads of the workgroup call.  id_at(pos) gives the
// point, apply(pos, right) receives the answer in lane 0 of the half wavefront.
template <typename IdAt, typename Apply>
__device__ __forceinline__ void resolve_exact(const int* list, int n, const float* nvec0, int nstride, const float* b_of,
                                              const float* __restrict__ points, int D, IdAt id_at, Apply apply)
{
    const int halves = blockDim.x >> 5;
    const int h = threadIdx.x >> 5, hl = threadIdx.x & 31;
    for (int base = 0; base < n; base += 2 * halves) {
        const int ia = base + h, ib = base + halves + h;
        const bool va = ia < n, vb = ib < n;
        const int ea = va ? list[ia] : 0, eb = vb ? list[ib] : 0;
        const float* xa = points + (size_t)id_at(ea & 0xffff) * D;
        const float* xb = points + (size_t)id_at(eb & 0xffff) * D;
        const float* na = nvec0 + (size_t)(ea >> 16) * nstride;
        const float* nb = nvec0 + (size_t)(eb >> 16) * nstride;
        float sa = 0.0f, sb = 0.0f;
        for (int d0 = hl; d0 < D; d0 += 256) {
            float xv[8], yv[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                xv[k] = (va && d0 + 32 * k < D) ? xa[d0 + 32 * k] : 0.0f;
                yv[k] = (vb && d0 + 32 * k < D) ? xb[d0 + 32 * k] : 0.0f;
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if (d0 + 32 * k < D) {
                    sa = __builtin_fmaf(na[d0 + 32 * k], xv[k], sa);
                    sb = __builtin_fmaf(nb[d0 + 32 * k], yv[k], sb);
                }
            }
        }
        sa = half_butterfly_sum(sa);
        sb = half_butterfly_sum(sb);
        if (hl == 0) {
            if (va) apply(ea & 0xffff, sa < b_of[ea >> 16]);
            if (vb) apply(eb & 0xffff, sb < b_of[eb >> 16]);
        }
    }
}

constexpr int kSideBatch = 4;        // points per group and call of the screen in the wide phase
constexpr int kTailBatch = 2;        // ... in the tail kernel

// Append a child node either to the next wide level or to the tail queue.  Returns its place in the queue of the next
// wide level, or -1.
__device__ __forceinline__ int emit_node(const TreeNode& c, const TreeParams& P, TreeNode* next, int next_cap,
                                         TreeNode* tail, int tail_cap, LevelCounters* ctr)
{
    const bool forced = c.depth >= P.MAX_DEPTH - 1;
    if (!c.leaf && !forced && c.count > P.small) {
        const int at = atomicAdd(&ctr->n_next, 1);
        if (at < next_cap) { next[at] = c; return at; }
        ctr->overflow = 1;
        return -1;
    }
    TreeNode t = c;
    if (forced) t.leaf = 1;
    const int at = atomicAdd(&ctr->n_tail, 1);
    if (at < tail_cap) tail[at] = t; else ctr->overflow = 1;
    return -1;
}

// The split / min-size-merge / leaf rules for a node whose left side has `a`
// members (src/kernels/build_tree_update_parents.cu:64-75,106-134).  Returns the
// number of children written to c0, c1.
__device__ __forceinline__ int split_rules(const TreeNode& nd, int a, int MIN, int MAX, int child_buf,
                                           TreeNode& c0, TreeNode& c1)
{
    const int r = nd.count - a;
    const uint64_t kl = child_key(nd.key, 0), kr = child_key(nd.key, 1);
    c0.tree = c1.tree = nd.tree;
    c0.depth = c1.depth = nd.depth + 1;
    c0.buf = c1.buf = child_buf;
    c0.rec = c1.rec = 0;
    c0.pad_ = c1.pad_ = 0;
    if (a == 0 || r == 0) {
        c0.start = nd.start; c0.count = nd.count; c0.dstart = nd.start; c0.dcount = nd.count;
        c0.key = a ? kl : kr; c0.leaf = nd.count <= MAX - 2;
        return 1;
    }
    if (min(a, r) < MIN) {
        const bool left_big = a >= r;
        c0.start = nd.start; c0.count = nd.count;
        c0.dstart = left_big ? nd.start : nd.start + a;
        c0.dcount = left_big ? a : r;
        c0.key = left_big ? kl : kr; c0.leaf = nd.count <= MAX;
        return 1;
    }
    c0.start = nd.start; c0.count = a; c0.dstart = nd.start; c0.dcount = a;
    c0.key = kl; c0.leaf = a <= MAX - 2;
    c1.start = nd.start + a; c1.count = r; c1.dstart = nd.start + a; c1.dcount = r;
    c1.key = kr; c1.leaf = r <= MAX - 2;
    return 2;
}

// Index of the tree (TreeRec): reserve the records of the children of node nd and write nd's own record.
// recs / n_rec belong to the tree of nd.  p1, p2: the drawn pair.  A node with one child (an empty side, or the
// min-size merge) routes every query the same way: it leaves no record and its child takes over its place, so a
// tree has fewer than twice as many records as buckets whatever its depth.
__device__ __forceinline__ void index_split(TreeRec* recs, int* n_rec, int rec_cap, int my_rec, int p1, int p2, int nc,
                                            int& rec0, int& rec1, LevelCounters* ctr)
{
    if (nc != 2) {
        rec0 = rec1 = my_rec;
        return;
    }
    const int base = atomicAdd(n_rec, 2);
    rec0 = base;
    rec1 = base + 1;
    if (base + 2 <= rec_cap && my_rec < rec_cap) {
        TreeRec r;
        r.a = p1; r.b = p2; r.c0 = rec0; r.c1 = rec1;
        recs[my_rec] = r;
    } else {
        ctr->overflow = 1;
    }
}

__device__ __forceinline__ void index_bucket(TreeRec* recs, int rec_cap, int my_rec, int start, int count, LevelCounters* ctr)
{
    if (my_rec < rec_cap) {
        TreeRec r;
        r.a = start; r.b = count; r.c0 = -1; r.c1 = -1;
        recs[my_rec] = r;
    } else {
        ctr->overflow = 1;
    }
}

// ---------------------------------------------------------------------------
// wide phase kernels
// ---------------------------------------------------------------------------

__global__ void k_init_perm(int* __restrict__ perm, int N, int B)
{
    const size_t total = (size_t)N * (size_t)B;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        perm[i] = (int)(i % (size_t)N);
}

__global__ void k_init_roots(TreeNode* nodes, TreeNode* tail, LevelCounters* ctr, TreeParams P, int B, int seed0,
                             int* n_rec, int* pmap)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= B) return;
    if (n_rec) n_rec[t] = 1;               // record 0 is the root
    TreeNode r;
    r.tree = t; r.start = 0; r.count = P.N; r.dstart = 0; r.dcount = P.N; r.depth = 0; r.buf = 0; r.leaf = 0;
    r.rec = 0; r.pad_ = 0;
    r.key = root_key(seed0 + t);
    // the root is never a leaf (src/kernels/build_tree_init.cu:79) unless the depth limit forces it
    const int at = emit_node(r, P, nodes, B, tail, B, ctr);
    if (pmap) pmap[t * pm::kPaths] = at;      // path 0 of level 0 = the root, if it is split at all
}

// chunk_base[i] = number of chunks of nodes [0,i); one workgroup.
__global__ __launch_bounds__(1024) void k_scan_chunks(const TreeNode* __restrict__ nodes, int node_cap, int chunk,
                                                      int* __restrict__ chunk_base, LevelCounters* ctr,
                                                      unsigned long long* __restrict__ stat)
{
    __shared__ int wsum[16];
    __shared__ int carry_s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_nodes = min(ctr->n_next, node_cap);       // nodes of the level, left by the previous level's scatter
    if (tid == 0) {
        carry_s = 0;
        phase_tick(ctr, 2);
    }
    __syncthreads();
    int members = 0;                                      // points of the nodes this thread looked at
    for (int base = 0; base < n_nodes; base += 1024) {
        const int i = base + tid;
        const int cnt_i = i < n_nodes ? nodes[i].count : 0;
        members += cnt_i;
        const int v = (cnt_i + chunk - 1) / chunk;
        // inclusive scan inside the wavefront
        int x = v;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int y = __shfl_up(x, o, 64);
            if (lane >= o) x += y;
        }
        if (lane == 63) wsum[wave] = x;
        __syncthreads();
        int woff = 0;
        for (int w = 0; w < wave; ++w) woff += wsum[w];
        const int carry = carry_s;
        if (i < n_nodes) chunk_base[i] = carry + woff + x - v;
        __syncthreads();
        if (tid == 1023) carry_s = carry + woff + x;
        __syncthreads();
    }
    if (tid == 0) { chunk_base[n_nodes] = carry_s; ctr->n_chunks = carry_s; }
    members = wave_sum_i(members);
    if (lane == 0) stat_add(stat, wave, 0, members);
}

// (also empties the queue of the level being produced, which the scatter kernel of this level fills)
__global__ void k_fill_chunks(const int* __restrict__ chunk_base, int n_nodes, int n_chunks, int* __restrict__ chunk2node,
                              LevelCounters* ctr)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c == 0) {
        phase_tick(ctr, 0);
        ctr->n_next = 0;
    }
    if (c >= n_chunks) return;
    int lo = 0, hi = n_nodes - 1;          // last node with chunk_base <= c
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (chunk_base[mid] <= c) lo = mid; else hi = mid - 1;
    }
    chunk2node[c] = lo;
}

// Hyperplanes of the nodes of a wide level, one wavefront per node: record ni of the table is
// [offset, bound of the 1-norm, sum of the components, 0 | normal, nvec_len(D) floats].  The workgroups of a node
// (one per chunk, up to a thousand at the first levels) fetch the record instead of each making the hyperplane again.
__global__ __launch_bounds__(256) void k_level_planes(const float* __restrict__ points, TreeParams P,
                                                      const int* __restrict__ perm0, const int* __restrict__ perm1,
                                                      const TreeNode* __restrict__ nodes, int n_nodes,
                                                      float* __restrict__ table, LevelCounters* ctr)
{
    extern __shared__ __align__(16) float lds_p[];          // per wavefront: 4 + nvec_len(D) floats
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (blockIdx.x == 0 && threadIdx.x == 0) phase_tick(ctr, -1);
    const int ni = blockIdx.x * (blockDim.x >> 6) + wave;
    if (ni >= n_nodes) return;
    const int rec = 4 + nvec_len(P.D);
    float* mine = lds_p + (size_t)wave * rec;
    const TreeNode nd = nodes[ni];
    const int* perm = (nd.buf ? perm1 : perm0) + (size_t)nd.tree * (size_t)P.N;
    int r1, r2;
    pick_pair(nd.key, nd.dcount, r1, r2);
    const int p1 = perm[nd.dstart + r1] & kIdMask;
    const int p2 = perm[nd.dstart + r2] & kIdMask;
    if (lane == 0) mine[3] = 0.0f;
    make_hyperplane_wave(points + (size_t)p1 * P.D, points + (size_t)p2 * P.D, P.D, mine + 4, mine);
    wave_lds_sync();
    float* out = table + (size_t)ni * rec;
    for (int i = lane; i < rec; i += 64) out[i] = mine[i];
}

// Side test of one chunk of one node: sets bit 31 of the permutation entry of
// every member on the right side and counts the members on the left.
template <bool Q8, int LPP>
__global__ __launch_bounds__(kBlock) void k_side(const float* __restrict__ points,
                                                 const uint16_t* __restrict__ pb16, const uint8_t* __restrict__ q8,
                                                 TreeParams P,
                                                 int* __restrict__ perm0, int* __restrict__ perm1,
                                                 const TreeNode* __restrict__ nodes, const int* __restrict__ chunk_base,
                                                 const int* __restrict__ chunk2node, int* __restrict__ chunk_left,
                                                 const float* __restrict__ planes, unsigned long long* __restrict__ stat)
{
    extern __shared__ __align__(16) float side_lds[];      // record of the node's hyperplane (k_level_planes)
    float* hp_s = side_lds;                                 // offset, bound of the 1-norm, sum of the components
    float* nvec = side_lds + 4;                             // nvec_len(D) floats
    __shared__ int left_s, n_def_s;
    __shared__ int deferred[1024];                          // points of the chunk left to the exact test (chunk <= 1024)
    const int c = blockIdx.x;
    const int ni = chunk2node[c];
    const TreeNode nd = nodes[ni];
    const int k = c - chunk_base[ni];
    int* perm = (nd.buf ? perm1 : perm0) + (size_t)nd.tree * (size_t)P.N;
    if (threadIdx.x == 0) { left_s = 0; n_def_s = 0; }
    {
        const int rec4 = (4 + nvec_len(P.D)) >> 2;          // 16-byte pieces of the record
        const float4* src = reinterpret_cast<const float4*>(planes + (size_t)ni * (size_t)(4 * rec4));
        for (int i = threadIdx.x; i < rec4; i += kBlock) reinterpret_cast<float4*>(side_lds)[i] = src[i];
    }
    __syncthreads();
    const float b = hp_s[0], n1 = hp_s[1], sn = hp_s[2];
    const int pos0 = nd.start + k * P.chunk;
    const int pos1 = min(nd.start + nd.count, pos0 + P.chunk);
    constexpr int kGroupsL = kBlock / LPP;                           // groups of LPP lanes, one point each
    const int grp = threadIdx.x / LPP, sub8 = threadIdx.x & (LPP - 1);
    const int iters = (pos1 - pos0 + kGroupsL - 1) / kGroupsL;
    int lefts = 0;
    for (int it = 0; it < iters; it += kSideBatch) {
        int id[kSideBatch], jz[kSideBatch], pos[kSideBatch];
        float bb[kSideBatch], h1[kSideBatch], h2[kSideBatch];
        bool valid[kSideBatch], right[kSideBatch], redo[kSideBatch];
#pragma unroll
        for (int u = 0; u < kSideBatch; ++u) {
            pos[u] = pos0 + (it + u) * kGroupsL + grp;
            valid[u] = pos[u] < pos1;
            id[u] = valid[u] ? (perm[pos[u]] & kIdMask) : 0;
            jz[u] = 0;
            bb[u] = b;
            h1[u] = n1;
            h2[u] = sn;
        }
        side_screen8<kSideBatch, Q8, LPP>(nvec, 0, jz, bb, h1, h2, pb16, q8, id, P.D, P.band, valid, right, redo);
#pragma unroll
        for (int u = 0; u < kSideBatch; ++u) {
            if (valid[u] && sub8 == 0) {
                if (redo[u]) {
                    deferred[atomicAdd(&n_def_s, 1)] = pos[u] - pos0;
                } else {
                    perm[pos[u]] = right[u] ? (id[u] | (int)0x80000000) : id[u];
                    lefts += right[u] ? 0 : 1;
                }
            }
        }
    }
    __syncthreads();
    resolve_exact(deferred, n_def_s, nvec, 0, hp_s, points, P.D,
                  [&](int local) { return perm[pos0 + local] & kIdMask; },
                  [&](int local, bool right) {
                      const int id = perm[pos0 + local] & kIdMask;
                      perm[pos0 + local] = right ? (id | (int)0x80000000) : id;      // build_tree_check_points_side.cu:149
                      lefts += right ? 0 : 1;
                  });
    if (lefts) atomicAdd(&left_s, lefts);
    __syncthreads();
    if (threadIdx.x == 0) {
        chunk_left[c] = left_s;
        stat_add(stat, c, 1, n_def_s);
    }
}

// Stable scatter of one chunk into the other permutation buffer; the workgroup
// of chunk 0 also applies the split rules and appends the children.
__global__ __launch_bounds__(kBlock) void k_scatter(TreeParams P, int* __restrict__ perm0, int* __restrict__ perm1,
                                                    const TreeNode* __restrict__ nodes, const int* __restrict__ chunk_base,
                                                    const int* __restrict__ chunk2node, const int* __restrict__ chunk_left,
                                                    TreeNode* __restrict__ next, int next_cap,
                                                    TreeNode* __restrict__ tail, int tail_cap, LevelCounters* ctr,
                                                    TreeRec* __restrict__ recs, int* __restrict__ n_rec, int rec_cap,
                                                    int2* __restrict__ child)
{
    __shared__ int red[2][kBlock / 64];
    const int c = blockIdx.x;
    if (c == 0 && threadIdx.x == 0) phase_tick(ctr, 1);
    const int ni = chunk2node[c];
    const TreeNode nd = nodes[ni];
    const int first = chunk_base[ni];
    const int nch = chunk_base[ni + 1] - first;
    const int k = c - first;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    const size_t toff = (size_t)nd.tree * (size_t)P.N;
    const int* src = (nd.buf ? perm1 : perm0) + toff;
    int* dst = (nd.buf ? perm0 : perm1) + toff;
    const int pos0 = nd.start + k * P.chunk;
    const int pos1 = min(nd.start + nd.count, pos0 + P.chunk);
    // rounds of four entries per thread (entry u of a thread at r0 + u kBlock + tid: loads and stores stay coalesced,
    // four loads in flight, one exchange of the wavefronts' counts per round); the entries of the first round (the
    // only one with chunks of 1024) are requested before the counts of the node's chunks are added up, so that the
    // two trips to memory go side by side
    constexpr int kPer = 4;
    int v[kPer];
    auto request = [&](int r0) {
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int pos = r0 + u * kBlock + tid;
            v[u] = pos < pos1 ? src[pos] : -1;            // (beyond the chunk: counts as a right one, is not stored)
        }
    };
    request(pos0);

    // lefts in the chunks before this one, and in the whole node
    int before = 0, all = 0;
    for (int j = tid; j < nch; j += kBlock) {
        const int x = chunk_left[first + j];
        all += x;
        if (j < k) before += x;
    }
    before = wave_sum_i(before);
    all = wave_sum_i(all);
    if (lane == 0) { red[0][wave] = before; red[1][wave] = all; }
    __syncthreads();
    before = 0; all = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) { before += red[0][w]; all += red[1][w]; }

    int lbase = before;                                   // lefts of the node before the current round
    __shared__ int wcnt4[kPer][kBlock / 64];
    for (int r0 = pos0; r0 < pos1; r0 += kPer * kBlock) {
        if (r0 > pos0) request(r0);
        uint64_t m[kPer];
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            m[u] = ballot64(v[u] >= 0);
            if (lane == 0) wcnt4[u][wave] = __popcll(m[u]);
        }
        __syncthreads();
        int run = lbase;                                  // lefts before entry (u, wavefront 0)
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            int woff = 0, tot = 0;
#pragma unroll
            for (int w = 0; w < kBlock / 64; ++w) { const int x = wcnt4[u][w]; if (w < wave) woff += x; tot += x; }
            const int pos = r0 + u * kBlock + tid;
            if (pos < pos1) {
                const int lrank = run + woff + mask_prefix(m[u]);      // lefts of the node before this position
                const bool right = v[u] < 0;
                const int dest = right ? nd.start + all + (pos - nd.start) - lrank : nd.start + lrank;
                dst[dest] = v[u] & kIdMask;
            }
            run += tot;
        }
        lbase = run;
        __syncthreads();
    }
    if (k == 0 && tid == 0) {
        TreeNode c0, c1;
        const int nc = split_rules(nd, all, P.MIN, P.MAX, nd.buf ^ 1, c0, c1);
        if (recs) {
            int r1, r2;
            pick_pair(nd.key, nd.dcount, r1, r2);
            index_split(recs + (size_t)nd.tree * rec_cap, n_rec + nd.tree, rec_cap, nd.rec, src[nd.dstart + r1] & kIdMask,
                        src[nd.dstart + r2] & kIdMask, nc, c0.rec, c1.rec, ctr);
        }
        const int at0 = emit_node(c0, P, next, next_cap, tail, tail_cap, ctr);
        const int at1 = nc == 2 ? emit_node(c1, P, next, next_cap, tail, tail_cap, ctr) : at0;
        // where the members of either side are at the next level (a node with one child keeps them together)
        if (child) child[ni] = make_int2(at0, at1);
    }
}

// What k_side leaves behind, from sides that are already known (one bit per point of the tree, pm::k_pm_sweep and
// pm::k_pm_resolve): bit 31 of the permutation entries of a chunk and the number of its left members.
__global__ __launch_bounds__(kBlock) void k_pm_mark(TreeParams P, int* __restrict__ perm0, int* __restrict__ perm1,
                                                    const TreeNode* __restrict__ nodes, const int* __restrict__ chunk_base,
                                                    const int* __restrict__ chunk2node, int* __restrict__ chunk_left,
                                                    const uint32_t* __restrict__ sidebits, int W)
{
    __shared__ int part[kBlock / 64];
    const int c = blockIdx.x;
    const int ni = chunk2node[c];
    const TreeNode nd = nodes[ni];
    const int k = c - chunk_base[ni];
    int* perm = (nd.buf ? perm1 : perm0) + (size_t)nd.tree * (size_t)P.N;
    const uint32_t* bits = sidebits + (size_t)nd.tree * (size_t)W;
    const int pos0 = nd.start + k * P.chunk;
    const int pos1 = min(nd.start + nd.count, pos0 + P.chunk);
    int lefts = 0;
    for (int r0 = pos0; r0 < pos1; r0 += 4 * kBlock) {
        int id[4];
        uint32_t w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int pos = r0 + u * kBlock + (int)threadIdx.x;
            id[u] = pos < pos1 ? (perm[pos] & kIdMask) : -1;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) w[u] = id[u] >= 0 ? bits[id[u] >> 5] : 0u;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int pos = r0 + u * kBlock + (int)threadIdx.x;
            if (id[u] >= 0) {
                const bool right = (w[u] >> (id[u] & 31)) & 1u;
                perm[pos] = right ? (id[u] | (int)0x80000000) : id[u];
                lefts += right ? 0 : 1;
            }
        }
    }
    lefts = wave_sum_i(lefts);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = lefts;
    __syncthreads();
    if (threadIdx.x == 0) {
        int all = 0;
#pragma unroll
        for (int i = 0; i < kBlock / 64; ++i) all += part[i];
        chunk_left[c] = all;
    }
}

// ---------------------------------------------------------------------------
// tail phase: one workgroup per small node, whole subtree in LDS
// ---------------------------------------------------------------------------
struct SmallNode {
    int start, count, dstart, dcount;     // offsets inside the task's segment
    int depth, leaf;
    int rec, pad_;                        // record of the node in the index of the tree, if one is written
    uint64_t key;
};

struct TreeStats {          // one per tree of the batch
    int n_leaves;           // buckets of at most kBucketSplit points, stored from the front of the leaf table
    int n_big;              // larger buckets, stored from the back of the leaf table
    int levels;
    int max_leaf;
    int min_leaf;
};

// Entry of the leaf table that the `at`-th bucket of its kind takes: small buckets fill the table of the tree from the
// front, large ones from the back, so that each kind can be handed to its own kernel as a plain (start, size) array.
__device__ __forceinline__ void store_leaf(int tree, int gstart, int count, int at, int leaf_cap,
                                           int* __restrict__ leaf_start, int* __restrict__ leaf_size, LevelCounters* ctr)
{
    if (at < leaf_cap) {
        const int slot = count > kBucketSplit ? leaf_cap - 1 - at : at;
        leaf_start[(size_t)tree * leaf_cap + slot] = gstart;
        leaf_size[(size_t)tree * leaf_cap + slot] = count;
    } else {
        ctr->overflow = 1;
    }
}

// One bucket straight to the table (nodes that became buckets in the wide phase).
__device__ __forceinline__ void emit_leaf(int tree, int gstart, int count, int depth, int leaf_cap,
                                          int* __restrict__ leaf_start, int* __restrict__ leaf_size,
                                          TreeStats* stats, LevelCounters* ctr)
{
    TreeStats* st = stats + tree;
    const int at = atomicAdd(count > kBucketSplit ? &st->n_big : &st->n_leaves, 1);
    store_leaf(tree, gstart, count, at, leaf_cap, leaf_start, leaf_size, ctr);
    atomicMax(&st->levels, depth + 1);
    atomicMax(&st->max_leaf, count);
    atomicMin(&st->min_leaf, count);
}

constexpr int kMaxGroup = 16;        // nodes of one level of a subtree worked on together

// One workgroup finishes the subtree of a task level by level: the nodes of a level are taken kMaxGroup (or
// fewer, G) at a time -- their hyperplanes are made together (one wavefront each), all their points are tested in
// one sweep, and each node is partitioned by one wavefront -- so the number of dependent trips to memory per
// subtree is a few per level instead of a few per node.
// TB = threads per workgroup: 256, or 1024 for launches over so few subtrees that workgroups of 256 would leave
// most of the device idle (the phases of a level then have four times the lanes).
template <bool Q8, int TB>
__global__ __launch_bounds__(TB) void k_tail(const float* __restrict__ points,
                                                 const uint16_t* __restrict__ pb16, const uint8_t* __restrict__ q8, TreeParams P,
                                                 const int* __restrict__ perm0, const int* __restrict__ perm1,
                                                 int* __restrict__ perm_out,
                                                 const TreeNode* __restrict__ tasks, int n_tasks, int node_cap, int G,
                                                 int leaf_cap, int* __restrict__ leaf_start, int* __restrict__ leaf_size,
                                                 TreeStats* stats, LevelCounters* ctr,
                                                 TreeRec* __restrict__ recs_all, int* __restrict__ n_rec_all, int rec_cap,
                                                 unsigned long long* __restrict__ stat)
{
    // dynamic LDS: seg[small] | tmp[small] | nvec[G][nvec_len(D)] | lrec[node_cap] | level lists 2 x node_cap | fmap[small]
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int Dv = nvec_len(P.D);
    int* seg = reinterpret_cast<int*>(lds_raw);
    int* tmp = seg + P.small;
    float* nvec = reinterpret_cast<float*>(tmp + P.small);
    // buckets of this subtree, written to the table of the tree together at the end (one reservation per
    // workgroup instead of one atomic round trip per bucket): x = start, y = size | rank among its kind << 16
    int2* lrec = reinterpret_cast<int2*>(nvec + (size_t)G * Dv);
    SmallNode* cur = reinterpret_cast<SmallNode*>(lrec + node_cap);
    SmallNode* nxt = cur + node_cap;
    unsigned char* fmap = reinterpret_cast<unsigned char*>(nxt + node_cap);
    __shared__ float b_s[kMaxGroup], hp_s[kMaxGroup][3];
    __shared__ int left_s[kMaxGroup], pre_s[kMaxGroup + 1], start_s[kMaxGroup], pair_s[kMaxGroup][2];
    __shared__ int n_cur_s, n_nxt_s, nrec_s, kind_s[2], base_s[2], lev_s, mx_s, mn_s, n_def_s;
    __shared__ int seen_s, unsure_s;        // points tested over all levels of the subtree, and left to the exact test

    const int task = blockIdx.x;
    if (task >= n_tasks) return;
    const TreeNode tk = tasks[task];
    const size_t toff = (size_t)tk.tree * (size_t)P.N;
    const int* src = (tk.buf ? perm1 : perm0) + toff;
    int* dst = perm_out + toff;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    if (tk.leaf) {
        // already a bucket (any size): move it to the output buffer and record it
        if (src != dst)
            for (int i = tid; i < tk.count; i += TB) dst[tk.start + i] = src[tk.start + i] & kIdMask;
        if (tid == 0) {
            emit_leaf(tk.tree, tk.start, tk.count, tk.depth, leaf_cap, leaf_start, leaf_size, stats, ctr);
            if (recs_all) index_bucket(recs_all + (size_t)tk.tree * rec_cap, rec_cap, tk.rec, tk.start, tk.count, ctr);
        }
        return;
    }
    TreeRec* recs = recs_all ? recs_all + (size_t)tk.tree * rec_cap : nullptr;
    int* n_rec = recs_all ? n_rec_all + tk.tree : nullptr;
    for (int i = tid; i < tk.count; i += TB) seg[i] = src[tk.start + i] & kIdMask;
    if (tid == 0) {
        SmallNode r;
        r.start = 0; r.count = tk.count; r.dstart = tk.dstart - tk.start; r.dcount = tk.dcount;
        r.depth = tk.depth; r.leaf = 0; r.key = tk.key; r.rec = tk.rec; r.pad_ = 0;
        cur[0] = r;
        n_cur_s = 1; n_nxt_s = 0; nrec_s = 0; kind_s[0] = 0; kind_s[1] = 0; lev_s = 0; mx_s = 0; mn_s = 0x7fffffff;
        seen_s = 0; unsure_s = 0;
    }
    __syncthreads();

    auto record_leaf = [&](int start, int count, int depth, int rec) {
        if (recs) index_bucket(recs, rec_cap, rec, tk.start + start, count, ctr);
        const int at = atomicAdd(&nrec_s, 1);
        const int rank = atomicAdd(&kind_s[count > kBucketSplit ? 1 : 0], 1);
        if (at < node_cap) lrec[at] = make_int2(tk.start + start, count | (rank << 16)); else ctr->overflow = 1;
        atomicMax(&lev_s, depth + 1);
        atomicMax(&mx_s, count);
        atomicMin(&mn_s, count);
    };

    const int grp = tid >> 3, sub8 = tid & 7;       // 32 groups of 8 lanes, one point each per iteration
    while (true) {
        const int n_cur = n_cur_s;
        if (n_cur == 0) break;
        for (int b0 = 0; b0 < n_cur; b0 += G) {
            const int nb = min(G, n_cur - b0);
            // the drawn pairs of the nodes of the group, and where their points sit in the flat numbering
            if (tid < nb) {
                const SmallNode nd = cur[b0 + tid];
                int r1, r2;
                pick_pair(nd.key, nd.dcount, r1, r2);
                pair_s[tid][0] = seg[nd.dstart + r1];
                pair_s[tid][1] = seg[nd.dstart + r2];
                start_s[tid] = nd.start;
            }
            if (tid == 0) {
                n_def_s = 0;
                int run = 0;
                for (int j = 0; j < nb; ++j) { pre_s[j] = run; run += cur[b0 + j].count; }
                pre_s[nb] = run;
            }
            __syncthreads();
            for (int j = wave; j < nb; j += TB / 64) {
                make_hyperplane_wave(points + (size_t)pair_s[j][0] * P.D, points + (size_t)pair_s[j][1] * P.D, P.D,
                                     nvec + (size_t)j * Dv, hp_s[j]);
                if (lane == 0) b_s[j] = hp_s[j][0];       // written by this lane just above
            }
            for (int j = 0; j < nb; ++j) {
                const int c = pre_s[j + 1] - pre_s[j];
                for (int t = tid; t < c; t += TB) fmap[pre_s[j] + t] = (unsigned char)j;
            }
            __syncthreads();
            // side of every point of the group's nodes
            const int total = pre_s[nb];
            constexpr int kTailGroups = TB / 8;
            const int iters = (total + kTailGroups - 1) / kTailGroups;
            for (int it = 0; it < iters; it += kTailBatch) {
                int id[kTailBatch], jj[kTailBatch], pos[kTailBatch];
                float bb[kTailBatch], h1[kTailBatch], h2[kTailBatch];
                bool valid[kTailBatch], right[kTailBatch], redo[kTailBatch];
#pragma unroll
                for (int u = 0; u < kTailBatch; ++u) {
                    const int f = (it + u) * kTailGroups + grp;
                    valid[u] = f < total;
                    jj[u] = valid[u] ? fmap[f] : 0;
                    pos[u] = valid[u] ? start_s[jj[u]] + f - pre_s[jj[u]] : 0;
                    id[u] = valid[u] ? seg[pos[u]] : 0;
                    bb[u] = b_s[jj[u]];
                    h1[u] = hp_s[jj[u]][1];
                    h2[u] = hp_s[jj[u]][2];
                }
                side_screen8<kTailBatch, Q8>(nvec, Dv, jj, bb, h1, h2, pb16, q8, id, P.D, P.band, valid, right, redo);
#pragma unroll
                for (int u = 0; u < kTailBatch; ++u) {
                    if (valid[u] && sub8 == 0) {
                        if (redo[u]) tmp[atomicAdd(&n_def_s, 1)] = pos[u] | (jj[u] << 16);      // tmp is free until the partition
                        else if (right[u]) seg[pos[u]] = id[u] | (int)0x80000000;
                    }
                }
            }
            __syncthreads();
            if (tid == 0) { seen_s += total; unsure_s += n_def_s; }
            resolve_exact(tmp, n_def_s, nvec, Dv, b_s, points, P.D, [&](int pos) { return seg[pos] & kIdMask; },
                          [&](int pos, bool right) { if (right) seg[pos] |= (int)0x80000000; });
            __syncthreads();
            // stable partition, one wavefront per node: seg -> tmp -> seg
            for (int j = wave; j < nb; j += TB / 64) {
                const int st = start_s[j], cnt = pre_s[j + 1] - pre_s[j];
                int a = 0;
                for (int r0 = 0; r0 < cnt; r0 += 64) a += __popcll(ballot64(r0 + lane < cnt && seg[st + r0 + lane] >= 0));
                int lbase = 0;
                for (int r0 = 0; r0 < cnt; r0 += 64) {
                    const int i = r0 + lane;
                    const bool valid = i < cnt;
                    const int v = valid ? seg[st + i] : 0;
                    const bool right = v < 0;
                    const uint64_t m = ballot64(valid && !right);
                    const int lrank = lbase + mask_prefix(m);
                    if (valid) tmp[st + (right ? a + i - lrank : lrank)] = v & kIdMask;
                    lbase += __popcll(m);
                }
                wave_lds_sync();
                for (int i = lane; i < cnt; i += 64) seg[st + i] = tmp[st + i];
                if (lane == 0) left_s[j] = a;
            }
            __syncthreads();
            // children: buckets are recorded, the others wait for the next level
            if (tid < nb) {
                const SmallNode nd = cur[b0 + tid];
                TreeNode full, c[2];
                full.tree = tk.tree; full.start = nd.start; full.count = nd.count; full.dstart = nd.dstart;
                full.dcount = nd.dcount; full.depth = nd.depth; full.buf = 0; full.leaf = 0; full.key = nd.key;
                const int nc = split_rules(full, left_s[tid], P.MIN, P.MAX, 0, c[0], c[1]);
                if (recs) index_split(recs, n_rec, rec_cap, nd.rec, pair_s[tid][0], pair_s[tid][1], nc, c[0].rec, c[1].rec, ctr);
                for (int q = 0; q < nc; ++q) {
                    if (c[q].leaf || c[q].depth >= P.MAX_DEPTH - 1) {
                        record_leaf(c[q].start, c[q].count, c[q].depth, c[q].rec);
                    } else {
                        const int at = atomicAdd(&n_nxt_s, 1);
                        if (at < node_cap) {
                            SmallNode sn;
                            sn.start = c[q].start; sn.count = c[q].count; sn.dstart = c[q].dstart; sn.dcount = c[q].dcount;
                            sn.depth = c[q].depth; sn.leaf = 0; sn.key = c[q].key; sn.rec = c[q].rec; sn.pad_ = 0;
                            nxt[at] = sn;
                        } else {
                            ctr->overflow = 1;
                        }
                    }
                }
            }
            __syncthreads();
        }
        if (tid == 0) { n_cur_s = min(n_nxt_s, node_cap); n_nxt_s = 0; }
        SmallNode* t = cur; cur = nxt; nxt = t;
        __syncthreads();
    }
    for (int i = tid; i < tk.count; i += TB) dst[tk.start + i] = seg[i];
    if (tid == 0) {
        TreeStats* st = stats + tk.tree;
        base_s[0] = kind_s[0] ? atomicAdd(&st->n_leaves, kind_s[0]) : 0;
        base_s[1] = kind_s[1] ? atomicAdd(&st->n_big, kind_s[1]) : 0;
        atomicMax(&st->levels, lev_s);
        atomicMax(&st->max_leaf, mx_s);
        atomicMin(&st->min_leaf, mn_s);
        stat_add(stat, task, 0, seen_s);
        stat_add(stat, task, 1, unsure_s);
    }
    __syncthreads();
    const int nrec = min(nrec_s, node_cap);
    for (int i = tid; i < nrec; i += TB) {
        const int2 r = lrec[i];
        const int count = r.y & 0xffff, rank = r.y >> 16;
        store_leaf(tk.tree, r.x, count, base_s[count > kBucketSplit ? 1 : 0] + rank, leaf_cap, leaf_start, leaf_size, ctr);
    }
}

template <typename T>
int dmalloc(T** p, size_t n)
{
    return ws_alloc(reinterpret_cast<void**>(p), std::max<size_t>(n, 1) * sizeof(T));
}

}  // namespace

// ---------------------------------------------------------------------------
// host driver
// ---------------------------------------------------------------------------
struct TreeBatchWorkspace {
    int B = 0, N = 0;
    int leaf_cap = 0, node_cap = 0, tail_cap = 0, chunk_cap = 0;
    int* perm[2] = {nullptr, nullptr};   // perm[0] is also the output
    TreeNode* nodes[2] = {nullptr, nullptr};
    TreeNode* tail = nullptr;
    int* chunk_base = nullptr;
    int* chunk2node = nullptr;
    int* chunk_left = nullptr;
    float* planes = nullptr;             // hyperplanes of the nodes of the current wide level: node_cap x (4 + nvec_len(D))
    int* leaf_start = nullptr;
    int* leaf_size = nullptr;
    TreeStats* stats = nullptr;
    LevelCounters* ctr = nullptr;
    int D = 0;
    LevelCounters* h_ctr = nullptr;      // pinned
    TreeStats* h_stats = nullptr;        // pinned
    unsigned long long* stat = nullptr;  // kStatSlots x kStatPitch: counts for the report (stat_add)
    unsigned long long* h_stat = nullptr;        // pinned
    unsigned long long counts[2] = {0, 0};       // of the last batch: points the side tests looked at, undecided ones
    // index of the trees for routing query points (allocated by tree_ws_enable_index)
    TreeRec* recs = nullptr;             // B x rec_cap
    int* n_rec = nullptr;                // B
    int rec_cap = 0;
    // events around the kernels of a wide level (hyperplanes | side test | scatter) and around the tail kernel
    hipEvent_t ev[2] = {nullptr, nullptr};          // around the tail kernel
    float phase_s[4] = {0.f, 0.f, 0.f, 0.f};   // of the last batch: side tests, hyperplanes, scatter, tail kernel
    // side tests of the first levels taken point by point (tree_sweep.hpp); allocated when D allows it
    int pm_ks = 0;                       // 32-dimension steps of a row as matrix-core operands (1, 2, 4, 8), 0 = not available
    int pm_W = 0;                        // tiles of 32 points (even)
    int pm_Bs = 0;                       // B rounded up to 16
    uint8_t* pm_path = nullptr;          // 32 W x Bs
    uint32_t* pm_side = nullptr;         // B x W
    uint32_t* pm_undec = nullptr;        // B x W
    int* pm_map[2] = {nullptr, nullptr}; // B x pm::kPaths, this level's and the next one's
    pm::PlaneQ* pm_sc = nullptr;         // B x pm::kPaths
    int8_t* pm_aq = nullptr;             // B x pm::kMaxGroups x 32 x 32 pm_ks
    int2* pm_child = nullptr;            // node_cap
};

static void free_ws(TreeBatchWorkspace& w)
{
    void* dev[] = {w.perm[0], w.perm[1], w.nodes[0], w.nodes[1], w.tail, w.chunk_base, w.chunk2node,
                   w.chunk_left, w.leaf_start, w.leaf_size, w.stats, w.ctr, w.recs, w.n_rec, w.planes,
                   w.pm_path, w.pm_side, w.pm_undec, w.pm_map[0], w.pm_map[1], w.pm_sc, w.pm_aq, w.pm_child, w.stat};
    for (void* p : dev) ws_free(p);
    if (w.h_ctr) (void)hipHostFree(w.h_ctr);
    if (w.h_stat) (void)hipHostFree(w.h_stat);
    if (w.h_stats) (void)hipHostFree(w.h_stats);
    for (hipEvent_t e : w.ev)
        if (e) (void)hipEventDestroy(e);
    w = TreeBatchWorkspace();
}

void tree_ws_free(TreeBatchWorkspace* w)
{
    if (!w) return;
    free_ws(*w);
    delete w;
}

int tree_ws_leaf_cap(const TreeBatchWorkspace* w) { return w->leaf_cap; }
const int* tree_ws_perm(const TreeBatchWorkspace* w, int t) { return w->perm[0] + (size_t)t * w->N; }
const int* tree_ws_leaf_start(const TreeBatchWorkspace* w, int t) { return w->leaf_start + (size_t)t * w->leaf_cap; }
const int* tree_ws_leaf_size(const TreeBatchWorkspace* w, int t) { return w->leaf_size + (size_t)t * w->leaf_cap; }

// Nodes of at most this many points are finished by one workgroup (k_tail): 1024, or 2048 for short rows, where a
// wide level costs more per byte of row it reads (the permutation entries it moves weigh more) -- measured on 10M x 32
// points 4.46 against 4.81 ms per tree, on 1M x 100 points 0.548 against 0.520 -- and for batches so small (N x B below
// 2^21 points) that the subtrees do not fill the device anyway: a wide level then costs its launches and little else
// (70,000 x 784, 10 trees: 0.964 against 0.996 ms per tree).  RSFK_TREE_SMALL overrides (tests).
int tree_small_threshold(int D, int N, int B)
{
    const char* e = std::getenv("RSFK_TREE_SMALL");
    const bool few = (size_t)N * (size_t)std::max(B, 1) < ((size_t)1 << 21);
    const int v = e && *e ? std::atoi(e) : (D <= 48 || few ? 2048 : 1024);
    return std::min(2048, std::max(64, v));
}
constexpr int kWideChunk = 1024;         // points per workgroup in the wide passes (k_side keeps a chunk's undecided points in LDS)

// bytes of device memory a batch of B trees needs
size_t tree_ws_bytes(int N, int D, int MIN, int B)
{
    const size_t lc = (size_t)N / (size_t)std::max(MIN, 1) + 2;
    return bf16_copy_bytes(N, D) + (size_t)B * ((size_t)N * 8 + (size_t)N * 2 + 512 * 1024 + lc * (8 + sizeof(TreeNode)) + ((size_t)N / 1024 + 2) * (2 * sizeof(TreeNode) + 24 + (size_t)(4 + nvec_len(D)) * 4));
}

// From now on every build with this workspace also writes the index of each tree (TreeRec records).
int tree_ws_enable_index(TreeBatchWorkspace* w, int MIN, int MAX_DEPTH)
{
    if (w->recs) return 0;
    // buckets <= N / MIN + 1 and two-child nodes fewer than buckets (one-child nodes leave no record)
    (void)MAX_DEPTH;
    const size_t cap = (size_t)2 * ((size_t)w->N / (size_t)std::max(MIN, 1) + 2) + 64;
    RSFK_CHECK(cap < ((size_t)1 << 30), "tree index: too many nodes");
    w->rec_cap = (int)cap;
    if (dmalloc(&w->recs, (size_t)w->B * cap)) return 1;
    if (dmalloc(&w->n_rec, (size_t)w->B)) return 1;
    return 0;
}
const TreeRec* tree_ws_recs(const TreeBatchWorkspace* w, int t) { return w->recs + (size_t)t * w->rec_cap; }
int tree_ws_rec_cap(const TreeBatchWorkspace* w) { return w->rec_cap; }
const int* tree_ws_n_rec(const TreeBatchWorkspace* w, int t) { return w->n_rec + t; }

int tree_ws_alloc(TreeBatchWorkspace** out, int N, int D, int MIN, int B)
{
    TreeBatchWorkspace* w = new TreeBatchWorkspace();
    *out = w;
    w->B = B; w->N = N; w->D = D;
    const int small = tree_small_threshold(D, N, B);
    w->leaf_cap = N / std::max(MIN, 1) + 2;
    w->node_cap = B * (N / small + 2);
    w->tail_cap = B * w->leaf_cap;
    w->chunk_cap = B * (N / kWideChunk + N / small + 4) + 16;      // sum ceil(count/chunk) <= N/chunk + nodes
    if (dmalloc(&w->perm[0], (size_t)B * N)) return 1;
    if (dmalloc(&w->perm[1], (size_t)B * N)) return 1;
    if (dmalloc(&w->nodes[0], (size_t)w->node_cap)) return 1;
    if (dmalloc(&w->nodes[1], (size_t)w->node_cap)) return 1;
    if (dmalloc(&w->tail, (size_t)w->tail_cap)) return 1;
    if (dmalloc(&w->chunk_base, (size_t)w->node_cap + 1)) return 1;
    if (dmalloc(&w->chunk2node, (size_t)w->chunk_cap)) return 1;
    if (dmalloc(&w->chunk_left, (size_t)w->chunk_cap)) return 1;
    if (dmalloc(&w->planes, (size_t)w->node_cap * (size_t)(4 + nvec_len(D)))) return 1;
    if (dmalloc(&w->leaf_start, (size_t)B * w->leaf_cap)) return 1;
    if (dmalloc(&w->leaf_size, (size_t)B * w->leaf_cap)) return 1;
    if (dmalloc(&w->stats, (size_t)B)) return 1;
    if (dmalloc(&w->ctr, (size_t)1)) return 1;
    if (dmalloc(&w->stat, (size_t)kStatSlots * kStatPitch)) return 1;
    if (D <= 256 && N > small && B <= 64) {
        w->pm_ks = D <= 32 ? 1 : D <= 64 ? 2 : D <= 128 ? 4 : 8;
        w->pm_W = 2 * ((N + 63) / 64);                     // an even number of 32-point tiles
        w->pm_Bs = (B + 15) & ~15;
        if (dmalloc(&w->pm_path, (size_t)w->pm_Bs * w->pm_W * 32)) return 1;
        if (dmalloc(&w->pm_side, (size_t)w->pm_Bs * w->pm_W)) return 1;
        if (dmalloc(&w->pm_undec, (size_t)w->pm_Bs * w->pm_W)) return 1;
        if (dmalloc(&w->pm_map[0], (size_t)B * pm::kPaths)) return 1;
        if (dmalloc(&w->pm_map[1], (size_t)B * pm::kPaths)) return 1;
        if (dmalloc(&w->pm_sc, (size_t)B * pm::kPaths)) return 1;
        if (dmalloc(&w->pm_aq, (size_t)B * pm::kMaxGroups * 32 * 32 * w->pm_ks)) return 1;
        if (dmalloc(&w->pm_child, (size_t)w->node_cap)) return 1;
    }
    RSFK_HIP(hipHostMalloc(reinterpret_cast<void**>(&w->h_ctr), sizeof(LevelCounters)));
    RSFK_HIP(hipHostMalloc(reinterpret_cast<void**>(&w->h_stats), sizeof(TreeStats) * (size_t)B));
    RSFK_HIP(hipHostMalloc(reinterpret_cast<void**>(&w->h_stat), sizeof(unsigned long long) * kStatSlots * kStatPitch));
    for (hipEvent_t& e : w->ev) RSFK_HIP(hipEventCreate(&e));
    return 0;
}

// seconds the last batch spent in: side tests, hyperplanes of the wide levels, scatter, tail kernel
const float* tree_ws_phase_seconds(const TreeBatchWorkspace* w) { return w->phase_s; }
// of the last batch: [0] points the side tests of all levels and trees looked at (the sum over the levels of the
// members of the nodes that were split), [1] those the screen left to the exact fp32 test
const unsigned long long* tree_ws_counts(const TreeBatchWorkspace* w) { return w->counts; }
// bytes of a row of the copy the side tests are screened on
int tree_screen_row_bytes(int D, bool q8) { return q8 ? q8_pitch(D) : 2 * bf16_pitch(D); }

// Builds nb (<= B) trees with seeds seed0 .. seed0+nb-1.  pb16 = rows of the bfloat16 copy of the points (may be
// null: every side test then reads the fp32 row).  On return perm[0] of
// tree t holds the point ids grouped by bucket and (leaf_start, leaf_size)[t]
// the buckets, in no particular order: those of at most kBucketSplit points in entries [0, n_small), the
// larger ones in entries [leaf_cap - n_big, leaf_cap).  host_stats receives 5 ints per tree: number of
// buckets, number of levels, largest and smallest bucket, number of large buckets.
int build_tree_batch(TreeBatchWorkspace* w, const float* points, const uint16_t* pb16, const uint8_t* q8, int N, int D, int MIN, int MAX,
                     int MAX_DEPTH, int seed0, int nb, int* host_stats, hipStream_t stream)
{
    RSFK_CHECK(nb >= 1 && nb <= w->B && N == w->N && D == w->D, "tree batch: workspace does not match the request");
    RSFK_CHECK(N >= 1 && D >= 1, "tree batch: N and D must be positive");
    TreeParams P;
    P.N = N; P.D = D; P.MIN = MIN; P.MAX = MAX; P.MAX_DEPTH = MAX_DEPTH;
    P.small = tree_small_threshold(D, N, w->B);
    P.chunk = kWideChunk;
    // bfloat16 rounding 2^-8 (1 + 2^-7), plus the summation errors of the screen (D/8 terms per lane and a 3-step
    // tree) and of the exact test (D/32 terms per lane and a 5-step tree), 1 % on top
    P.band = 1.01f * ((1.0f + 1.0f / 128.0f) / 256.0f + (float)(D / 8 + D / 32 + 16) / 16777216.0f);

    {
        const size_t total = (size_t)N * nb;
        const int grid = (int)std::min<size_t>((total + 255) / 256, 65536);
        hipLaunchKernelGGL(k_init_perm, dim3(grid), dim3(256), 0, stream, w->perm[0], N, nb);
    }
    std::vector<TreeStats> init((size_t)nb);
    for (auto& s : init) { s.n_leaves = 0; s.n_big = 0; s.levels = 0; s.max_leaf = 0; s.min_leaf = 0x7fffffff; }
    std::memcpy(w->h_stats, init.data(), sizeof(TreeStats) * (size_t)nb);
    RSFK_HIP(hipMemcpyAsync(w->stats, w->h_stats, sizeof(TreeStats) * (size_t)nb, hipMemcpyHostToDevice, stream));
    RSFK_HIP(hipMemsetAsync(w->ctr, 0, sizeof(LevelCounters), stream));
    RSFK_HIP(hipMemsetAsync(w->stat, 0, sizeof(unsigned long long) * kStatSlots * kStatPitch, stream));
    // Levels whose side tests are taken point by point (needs the 8-bit copy).  RSFK_PM_LEVELS overrides (0 = none).
    // The sweep multiplies every tile of points with every block of 16 hyperplanes of a tree, so its cost doubles
    // per level from the fifth on; measured, the seventh level is the last one it takes faster than k_side.
    int pm_levels = 0;
    if (q8 && w->pm_ks) {
        pm_levels = pm::kMaxLevels - 1;
        if (const char* e = std::getenv("RSFK_PM_LEVELS")) pm_levels = std::max(0, std::min(pm::kMaxLevels, std::atoi(e)));
    }
    hipLaunchKernelGGL(k_init_roots, dim3((nb + 63) / 64), dim3(64), 0, stream, w->nodes[0], w->tail, w->ctr, P, nb, seed0,
                       w->n_rec, pm_levels > 0 ? w->pm_map[0] : nullptr);
    RSFK_HIP(hipGetLastError());

    int cur = 0;
    const size_t side_lds = (size_t)(4 + nvec_len(D)) * sizeof(float);
    RSFK_CHECK(side_lds <= 150 * 1024, "tree batch: D too large for the LDS of the side test");
    // k_level_planes: four nodes per workgroup while their records fit in 48 KB, else one
    const int plane_waves = 4 * side_lds <= 48 * 1024 ? 4 : 1;
    if (side_lds > 48 * 1024) {
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_level_planes), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)side_lds));
        if (q8) {
            RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_side<true, 8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)side_lds));
        } else {
            RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_side<false, 8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)side_lds));
        }
    }
    for (float& v : w->phase_s) v = 0.0f;
    // wide levels
    int level = 0;
    while (true) {
        // one trip to the host per level: the chunk table of the level is made first (from the node count on the
        // device), then both counts come back together
        hipLaunchKernelGGL(k_scan_chunks, dim3(1), dim3(1024), 0, stream, w->nodes[cur], w->node_cap, P.chunk, w->chunk_base, w->ctr,
                           w->stat);
        RSFK_HIP(hipMemcpyAsync(w->h_ctr, w->ctr, sizeof(LevelCounters), hipMemcpyDeviceToHost, stream));
        RSFK_HIP(hipStreamSynchronize(stream));
        RSFK_CHECK(!w->h_ctr->overflow, "tree batch: node queue overflow");
        const int n_nodes = w->h_ctr->n_next;
        if (std::getenv("RSFK_TREE_TRACE")) {
            static double t_prev = 0.0;
            const double t_now = std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
            std::fprintf(stderr, "level %d: %d nodes, %d chunks, tail %d, previous level %.3f ms\n", level, n_nodes,
                         w->h_ctr->n_chunks, w->h_ctr->n_tail, level ? (t_now - t_prev) * 1e3 : 0.0);
            t_prev = t_now;
        }
        if (n_nodes == 0) break;
        RSFK_CHECK(n_nodes <= w->node_cap, "tree batch: node queue overflow");
        const int n_chunks = w->h_ctr->n_chunks;
        RSFK_CHECK(n_chunks <= w->chunk_cap, "tree batch: chunk table overflow");
        hipLaunchKernelGGL(k_level_planes, dim3((unsigned)((n_nodes + plane_waves - 1) / plane_waves)), dim3(64 * plane_waves),
                           plane_waves * side_lds, stream, points, P, w->perm[0], w->perm[1], w->nodes[cur], n_nodes, w->planes,
                           w->ctr);
        // (also sets n_next := 0 for the level being produced)
        hipLaunchKernelGGL(k_fill_chunks, dim3((n_chunks + 255) / 256), dim3(256), 0, stream, w->chunk_base, n_nodes, n_chunks,
                           w->chunk2node, w->ctr);
        const bool swept = level < pm_levels;
        if (swept) {
            // the sides of every point in all trees of the batch, then their marks in the permutations
            const int n_paths = 1 << level, ks = w->pm_ks, W = w->pm_W;
            const int rec = 4 + nvec_len(D);
            hipLaunchKernelGGL(pm::k_pm_planes, dim3((unsigned)((nb * n_paths + 3) / 4)), dim3(256), 0, stream, w->planes, rec, D,
                               32 * ks, w->pm_map[level & 1], n_paths, nb, w->pm_sc, w->pm_aq);
            const dim3 sgrid((unsigned)((W + 7) / 8));          // two tiles per wavefront, four wavefronts
#define RSFK_SWEEP_LAUNCH(KS)                                                                                                \
            hipLaunchKernelGGL((pm::k_pm_sweep<KS>), sgrid, dim3(256), 0, stream, q8, N, D, nb, w->pm_Bs, level, W, w->pm_path, \
                               w->pm_side, w->pm_undec, w->pm_aq, w->pm_sc)
            if (ks == 1) RSFK_SWEEP_LAUNCH(1);
            else if (ks == 2) RSFK_SWEEP_LAUNCH(2);
            else if (ks == 4) RSFK_SWEEP_LAUNCH(4);
            else RSFK_SWEEP_LAUNCH(8);
#undef RSFK_SWEEP_LAUNCH
            const size_t words = (size_t)nb * W;
            hipLaunchKernelGGL(pm::k_pm_resolve, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, points, D, W,
                               w->pm_Bs, words, w->pm_path, w->pm_sc, w->planes, rec, w->pm_side, w->pm_undec, w->stat);
            hipLaunchKernelGGL(k_pm_mark, dim3(n_chunks), dim3(kBlock), 0, stream, P, w->perm[0], w->perm[1], w->nodes[cur],
                               w->chunk_base, w->chunk2node, w->chunk_left, w->pm_side, W);
        } else {
        // lanes per point in the 8-bit screen: a lane takes 16 coordinates per step
        const int q8_pieces = q8_padded(D) >> 4;
#define RSFK_SIDE_LAUNCH(Q, L)                                                                                              \
        hipLaunchKernelGGL((k_side<Q, L>), dim3(n_chunks), dim3(kBlock), side_lds, stream, points, pb16, q8, P, w->perm[0],    \
                           w->perm[1], w->nodes[cur], w->chunk_base, w->chunk2node, w->chunk_left, w->planes, w->stat)
        if (!q8) RSFK_SIDE_LAUNCH(false, 8);
        else if (q8_pieces <= 2) RSFK_SIDE_LAUNCH(true, 2);
        else if (q8_pieces <= 4) RSFK_SIDE_LAUNCH(true, 4);
        else RSFK_SIDE_LAUNCH(true, 8);
#undef RSFK_SIDE_LAUNCH
        }
        const bool map_next = level + 1 < pm_levels;
        hipLaunchKernelGGL(k_scatter, dim3(n_chunks), dim3(kBlock), 0, stream, P, w->perm[0], w->perm[1], w->nodes[cur],
                           w->chunk_base, w->chunk2node, w->chunk_left, w->nodes[cur ^ 1], w->node_cap, w->tail, w->tail_cap, w->ctr,
                           w->recs, w->n_rec, w->rec_cap, map_next ? w->pm_child : nullptr);
        if (map_next) {
            const int n_paths = 1 << level;
            hipLaunchKernelGGL(pm::k_pm_next_map, dim3((unsigned)((nb * n_paths + 255) / 256)), dim3(256), 0, stream,
                               w->pm_map[level & 1], w->pm_map[(level + 1) & 1], w->pm_child, n_paths, nb);
        }
        RSFK_HIP(hipGetLastError());
        cur ^= 1;
        ++level;
    }
    // tail
    const int n_tail = w->h_ctr->n_tail;
    RSFK_CHECK(n_tail <= w->tail_cap, "tree batch: tail queue overflow");
    if (n_tail > 0) {
        // (the tail kernel keeps the bfloat16 screen: measured, it is not faster with the 8-bit one)
        // nodes of a level of a subtree (and its buckets): at most small / MIN + 1; hyperplanes kept together:
        // as many as 24 KB hold, at most kMaxGroup
        const int node_cap = P.small / std::max(MIN, 1) + 4;
        const int G = std::max(1, std::min(kMaxGroup, (int)(24 * 1024 / ((size_t)nvec_len(D) * 4))));
        const size_t lds = (size_t)(2 * P.small) * 4 + (size_t)G * nvec_len(D) * 4 + (size_t)node_cap * sizeof(int2) +
                           2 * (size_t)node_cap * sizeof(SmallNode) + (size_t)P.small;
        RSFK_CHECK(lds <= 150 * 1024, "tree batch: D too large for the tail kernel's LDS budget");
        const bool tail_q8 = q8 != nullptr && std::getenv("RSFK_TAIL_BF16") == nullptr;
        (void)hipEventRecord(w->ev[0], stream);
        // few subtrees (small inputs, few trees): workgroups of 1024 threads, so that a subtree's levels take less time
        // (70,000 x 784, 10 trees: 1.24 -> 1.00 ms per tree).  RSFK_TAIL_BLOCK=256 / 1024 overrides.
        bool wide_wg = n_tail < 8 * 256;
        if (const char* e = std::getenv("RSFK_TAIL_BLOCK")) wide_wg = std::atoi(e) >= 1024;
#define RSFK_TAIL_LAUNCH(Q, T)                                                                                             \
        do {                                                                                                               \
            RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_tail<Q, T>),                                      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                          \
            hipLaunchKernelGGL((k_tail<Q, T>), dim3(n_tail), dim3(T), lds, stream, points, pb16, q8, P, w->perm[0],         \
                               w->perm[1], w->perm[0], w->tail, n_tail, node_cap, G, w->leaf_cap, w->leaf_start,            \
                               w->leaf_size, w->stats, w->ctr, w->recs, w->n_rec, w->rec_cap, w->stat);                    \
        } while (0)
        if (tail_q8 && wide_wg) RSFK_TAIL_LAUNCH(true, 1024);
        else if (tail_q8) RSFK_TAIL_LAUNCH(true, 256);
        else if (wide_wg) RSFK_TAIL_LAUNCH(false, 1024);
        else RSFK_TAIL_LAUNCH(false, 256);
#undef RSFK_TAIL_LAUNCH
        (void)hipEventRecord(w->ev[1], stream);
        RSFK_HIP(hipGetLastError());
    }
    RSFK_HIP(hipMemcpyAsync(w->h_stats, w->stats, sizeof(TreeStats) * (size_t)nb, hipMemcpyDeviceToHost, stream));
    RSFK_HIP(hipMemcpyAsync(w->h_ctr, w->ctr, sizeof(LevelCounters), hipMemcpyDeviceToHost, stream));
    RSFK_HIP(hipMemcpyAsync(w->h_stat, w->stat, sizeof(unsigned long long) * kStatSlots * kStatPitch, hipMemcpyDeviceToHost, stream));
    RSFK_HIP(hipStreamSynchronize(stream));
    w->counts[0] = w->counts[1] = 0;
    for (int sl = 0; sl < kStatSlots; ++sl) {
        w->counts[0] += w->h_stat[kStatPitch * sl];
        w->counts[1] += w->h_stat[kStatPitch * sl + 1];
    }
    if (n_tail > 0) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, w->ev[0], w->ev[1]) == hipSuccess) w->phase_s[3] = ms * 1e-3f;
    }
    {
        // the steps of the wide levels, from the device's clock (events between the kernels of a level would cost
        // more than some of the kernels)
        int dev = 0, khz = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) == hipSuccess &&
            khz > 0) {
            const float s_per_tick = 1e-3f / (float)khz;
            w->phase_s[1] = (float)w->h_ctr->phase_ticks[0] * s_per_tick;       // hyperplanes
            w->phase_s[0] = (float)w->h_ctr->phase_ticks[1] * s_per_tick;       // side tests
            w->phase_s[2] = (float)w->h_ctr->phase_ticks[2] * s_per_tick;       // scatter
        }
    }
    RSFK_CHECK(!w->h_ctr->overflow, "tree batch: queue overflow in the tail phase");
    for (int t = 0; t < nb; ++t) {
        const int total = w->h_stats[t].n_leaves + w->h_stats[t].n_big;
        host_stats[5 * t + 0] = total;
        host_stats[5 * t + 1] = w->h_stats[t].levels;
        host_stats[5 * t + 2] = w->h_stats[t].max_leaf;
        host_stats[5 * t + 3] = total ? w->h_stats[t].min_leaf : 0;
        host_stats[5 * t + 4] = w->h_stats[t].n_big;
        RSFK_CHECK(total <= w->leaf_cap, "tree batch: leaf table overflow");
    }
    return 0;
}

}  // namespace rsfk
