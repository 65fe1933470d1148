// Neighbourhood exploration: every point looks at the neighbours of its
// neighbours (taken from a snapshot of the index array) and merges the closer
// ones into its own row.  Replaces nearest_neighbors_exploring
// (src/kernels/nearest_neighbors_exploring.cu:41-146) and its host loop
// (src/rsfk.cu:2100-2135).
//
// One wavefront per point, in three stages:
//
//  1. collect.  The K*K candidate ids are read with coalesced row reads of the
//     snapshot (16 rows of 64 ids in flight at a time) and put into a hash set in
//     LDS that was seeded with the point itself and its current row.  Only ids
//     that are new to the set survive, so each distinct candidate is looked at
//     once.  (The reference re-evaluates repeats; the result is the same because
//     a rejected candidate stays rejected -- the row maximum only decreases -- and
//     an accepted one is found in the row afterwards.)  The set is then compacted
//     in place into the list of candidates.  When the set cannot hold all K*K ids
//     (large K) the neighbours are processed in groups, each with a fresh set.
//
//  2. screen, on the bfloat16 copy of the points.  64 candidates at a time: their
//     rows (up to 128 dimensions = 256 bytes each) are requested with coalesced
//     128-byte segments, 8 lanes per row, while the previous 64 are being
//     evaluated (two batches of loads are in flight per wavefront: the stage is
//     bound by gather latency, so memory-level parallelism is what counts).  Rows
//     are transposed through LDS and each lane accumulates for "its" candidate
//     the approximate squared distance d~ and the quantity T below; a candidate
//     with d~ - E >= row maximum cannot enter the row and is dropped without its
//     fp32 row ever being touched.
//
//  3. exact.  The few candidates that pass get the exact distance from the fp32
//     rows (same gather/transposition, sequential fused multiply-add chain per
//     candidate: the arithmetic of the bucket kernel, compute_knn_from_buckets.cu:40-54,
//     so a pair has one distance value everywhere) and are offered to the sorted row.
//
// Error bound of the screen.  bfloat16 keeps 8 significant bits, so c~ = c + e with
// |e_d| <= 2^-8 |c_d| <= 2^-8 (1+2^-7) |c~_d| (round to nearest).  From
// (x-c)^2 = (x-c~)^2 + 2(x-c~)e + e^2:
//     |d~ - d| <= 2^-7 (1+2^-7) T + 2^-16 (1+2^-6) Q,   T = sum |x_d - c~_d| |c~_d|,  Q = sum c~_d^2.
// Both fp32 sums (d~ here, d in the exact path) are sums of non-negative terms, so
// each is within D 2^-24 (relative) of its real value.  E below is larger than the
// total; Q comes precomputed with the copy.
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"
#include "exact_batch.hpp"
#include <algorithm>

namespace rsfk {

namespace {

constexpr int kPitch = kChunk + 4;      // 36 words = 9 x 16 B: conflict-free b128 reads down a column of rows
constexpr int kBlockB = 128;            // bfloat16 dimensions per pipeline stage of the screen (2 x 64)
constexpr int kQueue2 = 128;            // candidates waiting for the exact distance
constexpr int kIdRows = 16;             // batches of 64 candidate ids loaded back to back
constexpr int kEmpty = (int)0x80000000; // free slot of the hash set

__device__ __forceinline__ uint32_t hash_id(int c)
{
    uint32_t h = (uint32_t)c * 0x9E3779B1u;
    return h ^ (h >> 15);
}

// Set of ids with open addressing.  Seeds (ids that must not become candidates) are
// stored as -id-1, candidates as id.  Returns true when c was new.  The caller
// guarantees a free slot exists.
__device__ __forceinline__ bool set_insert(int* table, int mask, int c, bool seed)
{
    uint32_t h = hash_id(c) & (uint32_t)mask;
    const int stored = seed ? -c - 1 : c;
    for (int i = 0; i <= mask; ++i) {
        const int old = atomicCAS(&table[h], kEmpty, stored);
        if (old == kEmpty) return true;
        if (old == c || old == -c - 1) return false;
        h = (h + 1) & (uint32_t)mask;
    }
    return false;
}

// The same for a candidate, returning its place in the table (whether new or already there), or -1 when the id is a
// seed (or the table is full).
__device__ __forceinline__ int set_insert_at(int* table, int mask, int c)
{
    uint32_t h = hash_id(c) & (uint32_t)mask;
    for (int i = 0; i <= mask; ++i) {
        const int old = atomicCAS(&table[h], kEmpty, c);
        if (old == kEmpty || old == c) return (int)h;
        if (old == -c - 1) return -1;
        h = (h + 1) & (uint32_t)mask;
    }
    return -1;
}

__device__ __forceinline__ void screen_pair(uint32_t w, float x0, float x1, float& da, float& ta)
{
    const float c0 = __uint_as_float(w << 16);
    const float c1 = __uint_as_float(w & 0xffff0000u);
    const float f0 = x0 - c0, f1 = x1 - c1;
    da = __builtin_fmaf(f0, f0, da);
    da = __builtin_fmaf(f1, f1, da);
    ta = __builtin_fmaf(fabsf(f0), fabsf(c0), ta);
    ta = __builtin_fmaf(fabsf(f1), fabsf(c1), ta);
}

// One pipeline stage of the screen = 128 bfloat16 dimensions of 64 candidate rows.
struct ScreenLoads {
    uint4 v[16];             // v[h*8+i]: half h (64 dimensions), rows i*8+sub, piece lane&7
};

__device__ __forceinline__ void screen_issue(ScreenLoads& S, const int* list, int n, const uint16_t* __restrict__ rows,
                                             int Db, int Dv, int b0)
{
    const int lane = lane_id();
    const int sub = lane >> 3, piece = lane & 7;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = i * 8 + sub;
        const uint16_t* rp = rows + (size_t)list[r < n ? r : 0] * (size_t)Db + b0 + piece * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            S.v[h * 8 + i] = make_uint4(0, 0, 0, 0);
            if (b0 + h * 64 + piece * 8 < Dv) S.v[h * 8 + i] = *reinterpret_cast<const uint4*>(rp + h * 64);
        }
    }
}

// Accumulate one stage into (da, ta) of this lane's candidate.
__device__ __forceinline__ void screen_consume(const ScreenLoads& S, const ExploreLds& L, int Db, int b0, float& da,
                                               float& ta)
{
    const int lane = lane_id();
    const int sub = lane >> 3, piece = lane & 7;
    uint32_t* tile = reinterpret_cast<uint32_t*>(L.tile);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int d0 = b0 + h * 64;
        if (d0 >= Db) break;
        wave_lds_sync();                 // previous reads of the tile are done
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *reinterpret_cast<uint4*>(&tile[(i * 8 + sub) * kPitch + piece * 4]) = S.v[h * 8 + i];
        wave_lds_sync();
        const int pieces = min(8, (Db - d0) >> 3);
        const uint32_t* mine = &tile[lane * kPitch];
        const float* xs = &L.xrow[d0];
        for (int q = 0; q < pieces; ++q) {
            const uint4 w = *reinterpret_cast<const uint4*>(mine + 4 * q);
            const float4 xa = *reinterpret_cast<const float4*>(xs + 8 * q);
            const float4 xb = *reinterpret_cast<const float4*>(xs + 8 * q + 4);
            screen_pair(w.x, xa.x, xa.y, da, ta);
            screen_pair(w.y, xa.z, xa.w, da, ta);
            screen_pair(w.z, xb.x, xb.y, da, ta);
            screen_pair(w.w, xb.z, xb.w, da, ta);
        }
    }
}

// Count of the exact distances of a launch, for the report of a build: one addition per wavefront, to one of 256
// slots a cache line apart (stat may be null).
__device__ __forceinline__ void count_exact(unsigned long long* stat, int n)
{
    if (stat && n > 0 && lane_id() == 0) atomicAdd(&stat[32 * (blockIdx.x & 255)], (unsigned long long)n);
}

// Stages are numbered s = batch * nblk + block; list holds U candidates.
struct ScreenCtx {
    const int* list;
    int U, nblk, Db, Dv, D;
};

template <int SL>
__device__ __forceinline__ void screen_stage_finish(const ScreenCtx& C, const ExploreLds& L, const Bf16Copy& bf, int batch,
                                                    float da, float ta, KnnRow<SL>& row, int& queued2,
                                                    const float* __restrict__ points, bool vec_ok, int& n_exact)
{
    const int lane = lane_id();
    const int n = min(64, C.U - batch * 64);
    const int my_c = C.list[batch * 64 + (lane < n ? lane : 0)];
    const float qn = bf.norms[my_c];
    const float slack = (float)(C.D + 8) * (1.0f / 4194304.0f);      // (D+8) 2^-22: fp32 summation error of both sums
    const float e = ta * (1.02f / 128.0f) + qn * (1.05f / 65536.0f) + da * slack;
    const bool may = lane < n && (da - e <= row.tau);
    const uint64_t pm = ballot64(may);
    if (pm == 0) return;
    if (may) L.queue2[queued2 + mask_prefix(pm)] = my_c;
    queued2 += __popcll(pm);
    if (queued2 >= 64) {
        wave_lds_sync();
        exact_batch<SL>(L, L.queue2, 64, points, C.D, vec_ok, row);
        n_exact += 64;
        const int rest = queued2 - 64;
        const int mv = lane < rest ? L.queue2[64 + lane] : 0;
        wave_lds_sync();
        if (lane < rest) L.queue2[lane] = mv;
        queued2 = rest;
        wave_lds_sync();
    }
}

template <int SL>
__device__ __forceinline__ void screen_all(const ScreenCtx& C, const ExploreLds& L, const Bf16Copy& bf, KnnRow<SL>& row,
                                           int& queued2, const float* __restrict__ points, bool vec_ok, int& n_exact)
{
    const int nb = (C.U + 63) >> 6;
    const int stages = nb * C.nblk;
    ScreenLoads A, B;
    float da = 0.0f, ta = 0.0f;
    auto issue = [&](ScreenLoads& S, int s) {
        const int batch = s / C.nblk, blk = s - batch * C.nblk;
        screen_issue(S, C.list + batch * 64, min(64, C.U - batch * 64), bf.rows, C.Db, C.Dv, blk * kBlockB);
    };
    auto consume = [&](const ScreenLoads& S, int s) {
        const int batch = s / C.nblk, blk = s - batch * C.nblk;
        if (blk == 0) { da = 0.0f; ta = 0.0f; }
        screen_consume(S, L, C.Dv, blk * kBlockB, da, ta);
        if (blk == C.nblk - 1) screen_stage_finish<SL>(C, L, bf, batch, da, ta, row, queued2, points, vec_ok, n_exact);
    };
    if (stages > 0) issue(A, 0);
    for (int s = 0; s < stages; s += 2) {
        if (s + 1 < stages) issue(B, s + 1);
        consume(A, s);
        if (s + 1 < stages) {
            if (s + 2 < stages) issue(A, s + 2);
            consume(B, s + 1);
        }
    }
}

template <int SL, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void k_explore(const float* __restrict__ points, Bf16Copy bf, int N, int D, int K,
                                                         const int* __restrict__ old_idx, int* __restrict__ knn_idx,
                                                         float* __restrict__ knn_dist, int table_size, int wave_lds_ints,
                                                         int dpad, int rows_per_group, const int* __restrict__ todo,
                                                         int n_todo, unsigned long long* __restrict__ stat)
{
    extern __shared__ __align__(16) int lds_i[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int slot = blockIdx.x * WAVES + wave;
    if (slot >= (todo ? n_todo : N)) return;              // whole wavefront leaves together
    const int p = todo ? todo[slot] : slot;               // all points, or the listed ones
    int* base = lds_i + (size_t)wave * (size_t)wave_lds_ints;
    ExploreLds L;
    L.tile = reinterpret_cast<float*>(base);                        // 64*kPitch words, 16-byte aligned
    L.xrow = reinterpret_cast<float*>(base + 64 * kPitch);          // dpad floats (multiple of 8)
    L.queue2 = base + 64 * kPitch + dpad;
    L.table = L.queue2 + kQueue2;
    L.srow = L.table + table_size;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const bool use_screen = bf.rows != nullptr;
    const int mask = table_size - 1;

    KnnRow<SL> row;
    row.load(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
    for (int k = lane; k < K; k += 64) L.srow[k] = old_idx[(size_t)p * K + k];
    const float* xp = points + (size_t)p * D;
    for (int d = lane; d < dpad; d += 64) L.xrow[d] = d < D ? xp[d] : 0.0f;

    ScreenCtx C;
    C.list = L.table;
    C.Db = bf16_pitch(D);
    C.Dv = bf16_valid(D);
    C.D = D;
    C.nblk = (C.Dv + kBlockB - 1) / kBlockB;
    int queued2 = 0;                                       // wave-uniform
    int n_exact = 0;                                       // exact distances of this point (wave-uniform)

    for (int i0 = 0; i0 < K; i0 += rows_per_group) {
        const int i1 = min(K, i0 + rows_per_group);
        // ---- collect -----------------------------------------------------------------
        wave_lds_sync();
        for (int i = lane; i < table_size; i += 64) L.table[i] = kEmpty;
        wave_lds_sync();
        if (lane == 0) set_insert(L.table, mask, p, true);
#pragma unroll
        for (int s = 0; s < SL; ++s)
            if (row.idx[s] >= 0) set_insert(L.table, mask, row.idx[s], true);
        const int e_begin = i0 * K, e_end = i1 * K;
        for (int g0 = e_begin; g0 < e_end; g0 += 64 * kIdRows) {
            int cand[kIdRows];
#pragma unroll
            for (int b = 0; b < kIdRows; ++b) {
                const int e = g0 + b * 64 + lane;
                int c = -1;
                if (e < e_end) {
                    const int i = e / K, k = e - i * K;
                    const int q = L.srow[i];
                    if (q >= 0 && q < N) c = old_idx[(size_t)q * K + k];
                }
                cand[b] = c;
            }
#pragma unroll
            for (int b = 0; b < kIdRows; ++b) {
                if (g0 + b * 64 >= e_end) break;
                const int c = cand[b];
                if (c >= 0 && c < N) set_insert(L.table, mask, c, false);
            }
        }
        wave_lds_sync();
        // ---- compact the set in place into the candidate list --------------------------
        int U = 0;
        for (int t0 = 0; t0 < table_size; t0 += 64) {
            const int v = L.table[t0 + lane];
            const bool is_cand = v >= 0;
            const uint64_t m = ballot64(is_cand);
            wave_lds_sync();             // all reads of this block are done before the front is overwritten
            if (is_cand) L.table[U + mask_prefix(m)] = v;
            U += __popcll(m);
        }
        wave_lds_sync();
        C.U = U;
        // ---- screen / exact ------------------------------------------------------------
        if (use_screen) {
            screen_all<SL>(C, L, bf, row, queued2, points, vec_ok, n_exact);
        } else {
            for (int off = 0; off < U; off += 64) {
                wave_lds_sync();
                exact_batch<SL>(L, L.table + off, min(64, U - off), points, D, vec_ok, row);
            }
            n_exact += U;
        }
    }
    // drain the second queue (at most 127 entries)
    for (int off = 0; off < queued2; off += 64) {
        wave_lds_sync();
        exact_batch<SL>(L, L.queue2 + off, min(64, queued2 - off), points, D, vec_ok, row);
    }
    n_exact += queued2;
    count_exact(stat, n_exact);
    if (row.changed) row.store(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K);
}

// Exploration of the points whose candidates the join has marked (explore_join.hip): entry (p, k) of
// the graph has the mask of neighbour slots at pass[p K + k] (entries without a valid neighbour have none).  One wavefront per point: gather
// the marked ids, drop repeats and ids the row holds (hash set), exact distances, merge.  Points with
// more marks than the LDS of this launch takes are appended to todo_out (for a launch with more LDS
// per wavefront, or for the general kernel).  todo_in: the points to work on, or null for all.
// Per-wavefront LDS (ints): tile[64*20] | xrow[dpad] | table[table_size] | srow[K] | marked[3/4 table_size].
// Number of entry (p, k) of the graph snapshot, p K + k, or -1 when the slot holds no valid neighbour (the join writes
// nothing for such an entry).
__device__ __forceinline__ int graph_entry(const int* __restrict__ old_idx, int N, int K, int p, int k)
{
    const int q = old_idx[(size_t)p * K + k];
    return q >= 0 && q < N ? p * K + k : -1;
}

constexpr int kMergeChunk = 16;
// 16-byte pieces of a candidate's row a lane requests from the tile together (exact_batch): 16 dimensions per wait for
// LDS.  (Measured: 1M x 256 pass 26.2 -> 24.8 ms, 70k x 784 pass 26.2 -> 25.0 ms; eight pieces cost the workgroup
// kernel its second wavefront per SIMD: 39 ms.)
constexpr int kChainGroup = 4;
constexpr int kMergeTile = 64 * (kMergeChunk + 4);
// Rows of at most this many (padded) dimensions are read by the lane that runs their chain, 32 dimensions at a time,
// without the transposing tile in LDS (exact_direct): the LDS of a wavefront shrinks by the tile.
__host__ __device__ inline int merge_tile_ints(int dpad, int direct_max) { return dpad <= direct_max ? 0 : kMergeTile; }
int merge_direct_max()
{
    static const int v = [] {
        // measured: 1M x 100 merge 4.4 -> 3.4 ms, 10M x 32 43 -> 27 ms; 1M x 256 slower (eight steps, each a trip)
        const char* e = std::getenv("RSFK_MERGE_DIRECT");
        return e ? std::atoi(e) : 128;
    }();
    return v;
}


// TILE: the candidates' rows go through the transposing tile (rows longer than direct_max dimensions); the two forms
// are kernels of their own, so that the shorter one does not carry the registers of the other.
template <int SL, int WAVES, bool TILE>
__global__ __launch_bounds__(64 * WAVES) void k_explore_merge(const float* __restrict__ points, int N, int D, int K,
                                                               const int* __restrict__ old_idx, int* __restrict__ knn_idx,
                                                               float* __restrict__ knn_dist, int table_size,
                                                               int wave_lds_ints, int dpad, int direct_max,
                                                               const uint32_t* __restrict__ pass,
                                                               const uint16_t* __restrict__ bounds,
                                                               const int* __restrict__ todo_in, int n_in,
                                                               int* __restrict__ todo_out, int* __restrict__ n_out,
                                                               unsigned long long* __restrict__ stat,
                                                               const int* __restrict__ order)
{
    extern __shared__ __align__(16) int lds_m[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int slot = die_local_place(blockIdx.x, gridDim.x) * WAVES + wave;
    if (slot >= (todo_in ? n_in : N)) return;             // whole wavefront leaves together
    const int p = todo_in ? todo_in[slot] : (order ? order[slot] : slot);
    const int MW = (K + 31) >> 5;
    int* base = lds_m + (size_t)wave * (size_t)wave_lds_ints;
    // Rows of at most 64 neighbours (one slot per lane): everything the point needs from memory before its candidates
    // are known -- its K-NN row, the snapshot of its neighbours, its mark words, its coordinates -- is requested at once;
    // none of these addresses depends on another's data.  (Longer rows: one after the other, as they are needed.)
    constexpr bool kEarly = SL == 1;
    KnnRow<SL> row;
    int q_own = -1;
    uint32_t pw[2] = {0u, 0u};
    if (kEarly) {
        const size_t at = (size_t)p * K + (lane < K ? lane : 0);
        row.idx[0] = knn_idx[at];
        row.dist[0] = knn_dist[at];
        q_own = old_idx[at];
        pw[0] = pass[at * MW];
        if (MW > 1) pw[1] = pass[at * MW + 1];
        const float* xp0 = points + (size_t)p * D;
        float* xr = reinterpret_cast<float*>(base + merge_tile_ints(dpad, direct_max));
        for (int d = lane; d < dpad; d += 64) xr[d] = d < D ? xp0[d] : 0.0f;
        if (lane >= K) { row.idx[0] = -2; row.dist[0] = INFINITY; q_own = -1; }
        if (!(q_own >= 0 && q_own < N)) { pw[0] = 0u; pw[1] = 0u; }          // the join writes nothing for such an entry
    }
    int bits = 0;
    if (kEarly) {
        bits = __popc(pw[0]) + __popc(pw[1]);
    } else {
        for (int k = lane; k < K; k += 64) {
            const int j = graph_entry(old_idx, N, K, p, k);
            if (j >= 0)
                for (int w = 0; w < MW; ++w) bits += __popc(pass[(size_t)j * MW + w]);
        }
    }
    const int n_given = wave_sum_i(bits);
    if (n_given == 0) return;
    if (n_given + K + 1 > table_size / 4 * 3) {
        if (lane == 0) todo_out[atomicAdd(n_out, 1)] = p;
        return;
    }
    ExploreLds L;
    L.tile = reinterpret_cast<float*>(base);
    const int tile_ints = merge_tile_ints(dpad, direct_max);
    L.xrow = reinterpret_cast<float*>(base + tile_ints);
    L.queue2 = nullptr;
    L.table = base + tile_ints + dpad;
    L.srow = L.table + table_size;
    // with bounds: the smallest lower bound seen for the id in the same place of the set (bfloat16 bits), behind the
    // list of marks
    int* tbound = bounds ? L.srow + K + table_size / 4 * 3 : nullptr;
    const int KP = (K + 31) & ~31;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);

    if (kEarly) {
        row.init_from_regs(K);
        if (lane < K) L.srow[lane] = q_own;
    } else {
        row.load(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
        for (int k = lane; k < K; k += 64) L.srow[k] = old_idx[(size_t)p * K + k];
        const float* xp = points + (size_t)p * D;
        for (int d = lane; d < dpad; d += 64) L.xrow[d] = d < D ? xp[d] : 0.0f;
    }

    int ts = 64;
    while (ts < 2 * (n_given + K + 1)) ts <<= 1;
    ts = min(ts, table_size);
    const int mask = ts - 1;
    for (int i = lane; i < ts; i += 64) {
        L.table[i] = kEmpty;
        if (tbound) tbound[i] = 0x7fffffff;
    }
    wave_lds_sync();
    if (lane == 0) set_insert(L.table, mask, p, true);
#pragma unroll
    for (int s = 0; s < SL; ++s)
        if (row.idx[s] >= 0) set_insert(L.table, mask, row.idx[s], true);
    // list of the marked (neighbour, slot) pairs, so that the ids can be gathered by all lanes at once
    // instead of one after the other per neighbour
    int* marked = L.srow + K;
    int n_marked = 0;                                     // wave-uniform
    for (int k0 = 0; k0 < K; k0 += 64) {
        const int k = k0 + lane;
        const int j = kEarly ? (q_own >= 0 && q_own < N ? p * K + k : -1) : (k < K ? graph_entry(old_idx, N, K, p, k) : -1);
        int mine = 0;
        if (kEarly) mine = bits;
        else if (j >= 0)
            for (int w = 0; w < MW; ++w) mine += __popc(pass[(size_t)j * MW + w]);
        int at = n_marked + wave_excl_scan_i(mine);
        if (j >= 0) {
            for (int w = 0; w < MW; ++w) {
                uint32_t m = kEarly ? pw[w & 1] : pass[(size_t)j * MW + w];
                while (m) {
                    const int b = __ffs(m) - 1;
                    m &= m - 1;
                    marked[at++] = k | ((32 * w + b) << 8);
                }
            }
        }
        n_marked += wave_sum_i(mine);
    }
    wave_lds_sync();
    // (the ids of 256 marks are requested together: a point's marks then cost one trip to memory, not one per 64)
    for (int i0 = 0; i0 < n_marked; i0 += 256) {
        int c[4], lb[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + 64 * u + lane;
            c[u] = -1;
            lb[u] = 0;
            if (i < n_marked) {
                const int e = marked[i];
                c[u] = old_idx[(size_t)L.srow[e & 255] * K + (e >> 8)];
                // the join's lower bound of the pair: entry p K + k of the graph, column = slot in the neighbour's row
                if (bounds) lb[u] = bounds[((size_t)p * K + (e & 255)) * (size_t)KP + (e >> 8)];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (c[u] >= 0 && c[u] < N) {
                if (tbound) {
                    const int at = set_insert_at(L.table, mask, c[u]);
                    if (at >= 0) atomicMin(&tbound[at], lb[u]);
                } else {
                    set_insert(L.table, mask, c[u], false);
                }
            }
        }
    }
    wave_lds_sync();
    // compact the set in place into the candidate list (and the bounds with it)
    int U = 0;
    for (int t0 = 0; t0 < ts; t0 += 64) {
        const int v = L.table[t0 + lane];
        const int vb = tbound ? tbound[t0 + lane] : 0;
        const bool is_cand = v >= 0;
        const uint64_t m = ballot64(is_cand);
        wave_lds_sync();
        if (is_cand) {
            L.table[U + mask_prefix(m)] = v;
            if (tbound) tbound[U + mask_prefix(m)] = vb;
        }
        U += __popcll(m);
    }
    wave_lds_sync();
    int n_exact = 0;                                      // exact distances of this point (wave-uniform)
    auto batch = [&](const int* list, int n) {
        n_exact += n;
        if (!TILE) exact_direct<SL>(L, list, n, points, D, vec_ok, row);
        else exact_batch<SL, kMergeChunk, true, kChainGroup>(L, list, n, points, D, vec_ok, row);    // two steps of gathers in flight
    };
    if (tbound == nullptr || U <= 64) {
        for (int off = 0; off < U; off += 64) {
            wave_lds_sync();
            batch(L.table + off, min(64, U - off));
        }
    } else {
        // Nearer bounds first: a round takes the candidates that are left, whose bound is not above the row's last
        // slot (it shrinks from round to round) and -- while more than a batch of them is left -- not above the
        // mean of these bounds.  A candidate whose bound is above the last slot cannot enter the row and is never
        // read.  The ids of a round are gathered in the list of marks, which is no longer needed.  (Taking exactly
        // the 64 nearest bounds of every round, found by bisection, was measured slower: the bounds of a point take
        // few distinct values at 16 bits, and the search costs more than the order gains.)
        constexpr int kDone = 0x7fffffff;
        int* round_ids = marked;
        while (true) {
            const float tau_now = row.tau;
            int n_el = 0, sum = 0;
            for (int t0 = 0; t0 < U; t0 += 64) {
                const int b = t0 + lane < U ? tbound[t0 + lane] : kDone;
                const bool el = b != kDone && !(__uint_as_float((uint32_t)b << 16) > tau_now);
                n_el += __popcll(ballot64(el));
                sum += el ? b : 0;
            }
            if (n_el == 0) break;
            sum = wave_sum_i(sum);
            const int cut = n_el <= 64 ? 0xffff : sum / n_el;           // (the smallest bound is never above the mean)
            int n_round = 0;
            for (int t0 = 0; t0 < U; t0 += 64) {
                const int b = t0 + lane < U ? tbound[t0 + lane] : kDone;
                const bool take = b != kDone && !(__uint_as_float((uint32_t)b << 16) > tau_now) && b <= cut;
                const uint64_t m = ballot64(take);
                if (take) {
                    round_ids[n_round + mask_prefix(m)] = L.table[t0 + lane];
                    tbound[t0 + lane] = kDone;
                }
                n_round += __popcll(m);
            }
            for (int off = 0; off < n_round; off += 64) {
                wave_lds_sync();
                batch(round_ids + off, min(64, n_round - off));
            }
            wave_lds_sync();
        }
    }
    count_exact(stat, n_exact);
    if (row.changed) row.store(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K);
}

// The same for rows so long that the set of one point takes most of the LDS a wavefront could get (K above about 45:
// a point has up to K^2 marks): one workgroup of four wavefronts per point, and the candidates are taken in the
// order of their lower bounds.
//
// A candidate can only end up in the row if its exact distance is at most the row's last slot at the end, and that
// slot falls fast once the nearest candidates are in.  In the order of the marks most candidates enter at some
// moment and are pushed out again later (three quarters of them on 70,000 x 784 rows with K = 90), each at the price
// of gathering a whole fp32 row.  Here:
//   1. all threads list the marked (neighbour, slot) pairs of the point together with the lower bound L the join
//      kept for each (explore_join.hip; 0 when it kept none), one 32-bit word per pair;
//   2. every wavefront walks its quarter of the list in rounds with a rising limit: the smallest limit that takes 64
//      marks it has not taken yet (found by bisection on the 16 bits of the bounds), never above the shared last
//      slot -- near candidates first, without sorting anything.  A pair whose bound is above the shared last slot at
//      its turn is never looked at.  The others have their id read, pass through a hash set (seeded with the row;
//      drops repeats -- only a saving: a repeated candidate would be rejected by the row), get the exact distance,
//      64 at a time and what is left at the end of the round, and are merged into the wavefront's copy of the row.
//      Between the rounds the wavefronts work out what the last slot of their four rows taken together would be
//      (shared_last_slot below, no merge needed), which is the limit nobody goes beyond: measured on 70,000 x 784 rows
//      with K = 90, 184 exact distances per point instead of 544 with a limit from each wavefront's own row, for the
//      85 entries of a row that change;
//   3. the four rows become one in two steps (2 -> 0 and 3 -> 1, then 1 -> 0), entries above that limit left out,
//      and the first wavefront stores the result.
// A bound is below the exact distance of its pair, the shared last slot is never below the final one: a dropped
// candidate could not have been in the final row, so the result is the one of any other order.
// (Sorting the list by the bounds first, a bitonic network over up to 4096 words in LDS, cost more than it saved.)
// LDS (ints): table[kWgTable] | srow[K] | jrow[K] | xrow[dpad] | marked[cap] | 4 tiles | 3 rows for the exchange | 4 x 128 ids
// | distances of the row as loaded [K] | distances of the four rows as last shown [4][K].
constexpr int kWgChunk = 32;
constexpr int kWgTile = 64 * (kWgChunk + 4);
constexpr int kWgTable = 2048;              // hash set; when three quarters are taken, new ids are no longer recorded
constexpr int kWgMinCap = 1024;             // the kernel is not used when fewer marks than this would fit

constexpr int kWgMaxRounds = 12;            // the last one takes everything that is left below the last slot
constexpr int kWgMaxCap = 6656;             // marks per point: 26 steps of the walk of a wavefront
constexpr int kWgMaxSteps = kWgMaxCap / 256;

// distance in slot k of a row (k is the same in all lanes)
template <int SL>
__device__ __forceinline__ float row_slot_dist(const KnnRow<SL>& row, int k)
{
    float v = INFINITY;
#pragma unroll
    for (int s = 0; s < SL; ++s)
        if ((k >> 6) == s) v = read_lane_f(row.dist[s], k & 63);
    return v;
}

template <int SL>
__global__ __launch_bounds__(256) void k_explore_merge_wg(const float* __restrict__ points, int N, int D, int K,
                                                          const int* __restrict__ old_idx, int* __restrict__ knn_idx,
                                                          float* __restrict__ knn_dist, int cap, int dpad,
                                                          const uint32_t* __restrict__ pass,
                                                          const uint16_t* __restrict__ bounds,
                                                          const int* __restrict__ todo_in, int n_in,
                                                          int* __restrict__ todo_out, int* __restrict__ n_out,
                                                          unsigned long long* __restrict__ stat)
{
    extern __shared__ __align__(16) int lds_w[];
    __shared__ int wave_tot[4];
    __shared__ int n_set_s;
    __shared__ uint32_t tau_s;                                    // bits of the smallest last slot reached so far
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // (the list of points a launch before this one left over is in the order in which that launch came to them)
    const int slot = die_local_place(blockIdx.x, gridDim.x);
    if (slot >= (todo_in ? n_in : N)) return;
    const int p = todo_in ? todo_in[slot] : slot;
    const int MW = (K + 31) >> 5, KP = MW * 32;
    int* table = lds_w;
    int* srow = table + kWgTable;
    int* jrow = srow + ((K + 3) & ~3);                            // number of graph entry (p, k), -1 without a valid neighbour
    float* xrow = reinterpret_cast<float*>(jrow + ((K + 3) & ~3));
    uint32_t* marked = reinterpret_cast<uint32_t*>(xrow + dpad);
    int* tiles = reinterpret_cast<int*>(marked + cap);
    int* xch = tiles + 4 * kWgTile;                               // rows on their way to another wavefront: [3][idx | dist][64 SL]
    int* ids = xch + 6 * 64 * SL + 128 * wave;                    // this wavefront's candidates: a batch and what is left over
    const int kq = (K + 3) & ~3;
    float* old_d = reinterpret_cast<float*>(xch + 6 * 64 * SL + 4 * 128);  // distances of the row as it was loaded
    float* seen_d = old_d + kq;                                   // [4][kq]: the rows of the wavefronts as they last showed them
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);

    // thread k takes neighbour k (K <= 256): its entry of the snapshot and its mark words are requested together with
    // the point's row and coordinates (none of these addresses depends on another's data)
    const int k = threadIdx.x;
    const size_t entry = (size_t)p * K + (k < K ? k : 0);
    const int q_own = old_idx[entry];
    uint32_t pw[8];                                               // MW <= 8
#pragma unroll
    for (int w = 0; w < 8; ++w) pw[w] = w < MW ? pass[entry * MW + w] : 0u;
    KnnRow<SL> row;
    row.load(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
    const float* xp = points + (size_t)p * D;
    for (int d = threadIdx.x; d < dpad; d += 256) xrow[d] = d < D ? xp[d] : 0.0f;
    for (int i = threadIdx.x; i < kWgTable; i += 256) table[i] = kEmpty;

    // ---- 1. the marked pairs of the point
    const int j = k < K && q_own >= 0 && q_own < N ? (int)entry : -1;     // (the join writes nothing for other entries)
    if (k < K) {
        srow[k] = q_own;
        jrow[k] = j;
    }
#pragma unroll
    for (int s = 0; s < SL; ++s) {
        if (lane + 64 * s < K) {
            seen_d[wave * kq + lane + 64 * s] = row.dist[s];      // every wavefront starts from the same sorted row
            if (wave == 0) old_d[lane + 64 * s] = row.dist[s];
        }
    }
    int mine = 0;
    if (j >= 0) {
#pragma unroll
        for (int w = 0; w < 8; ++w) mine += __popc(pw[w]);
    }
    const int in_wave = wave_excl_scan_i(mine);
    if (lane == 63) wave_tot[wave] = in_wave + mine;
    if (threadIdx.x == 0) {
        n_set_s = 0;
        tau_s = __float_as_uint(row.tau);
    }
    __syncthreads();
    int at = in_wave, n_marked = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        if (w < wave) at += wave_tot[w];
        n_marked += wave_tot[w];
    }
    if (n_marked == 0) return;
    if (n_marked > cap) {
        if (threadIdx.x == 0) todo_out[atomicAdd(n_out, 1)] = p;
        return;
    }
    if (j >= 0) {
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            uint32_t m = pw[w];
            while (m) {
                const int b = __ffs(m) - 1;
                m &= m - 1;
                marked[at++] = (uint32_t)((32 * w + b) << 8) | (uint32_t)k;
            }
        }
    }
    if (wave == 0) {                                              // seeds: ids that are in the row already
        const int mask = kWgTable - 1;
        int seeded = 0;
#pragma unroll
        for (int s = 0; s < SL; ++s)
            if (row.idx[s] >= 0) { set_insert(table, mask, row.idx[s], true); ++seeded; }
        seeded = wave_sum_i(seeded);
        if (lane == 0) atomicAdd(&n_set_s, seeded);
    }
    __syncthreads();
    if (bounds) {
        // the bounds of the listed pairs, by all threads (a thread's own marks one after the other would wait for
        // one 2-byte read at a time)
        for (int i0 = threadIdx.x; i0 < n_marked; i0 += 4 * 256) {
            uint32_t e[4], lb[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = i0 + 256 * u;
                e[u] = i < n_marked ? marked[i] : 0u;
                lb[u] = i < n_marked ? (uint32_t)bounds[(size_t)jrow[e[u] & 255u] * KP + ((e[u] >> 8) & 255u)] : 0u;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (i0 + 256 * u < n_marked) marked[i0 + 256 * u] = e[u] | (lb[u] << 16);
        }
        __syncthreads();
    }

    // ---- 2. my quarter of the list, nearer bounds first
    ExploreLds L;
    L.tile = reinterpret_cast<float*>(tiles + wave * kWgTile);
    L.xrow = xrow;
    L.queue2 = nullptr;
    L.table = nullptr;
    L.srow = nullptr;
    int have = 0;                                                 // candidates waiting in ids (wave-uniform)
    int n_exact = 0;                                              // exact distances this wavefront asked for
    auto run_batch = [&]() {
        wave_lds_sync();
        const int n_now = min(64, have);
        n_exact += n_now;
        const float cap_now = __uint_as_float(*reinterpret_cast<volatile uint32_t*>(&tau_s));
        exact_batch<SL, kWgChunk, true, kChainGroup>(L, ids, n_now, points, D, vec_ok, row, cap_now);
        if (lane == 0) atomicMin(&tau_s, __float_as_uint(row.tau));   // non-negative floats order like their bits
        have -= n_now;
        const int left = lane < have ? ids[64 + lane] : 0;        // the candidates beyond the batch move to the front
        wave_lds_sync();
        if (lane < have) ids[lane] = left;
    };
    // The last slot of the four rows taken together, without merging them.  The wavefronts evaluate disjoint sets of
    // new candidates (the hash set, as long as it records), none of them in the row as loaded, so for any t the
    // candidates and old entries at a distance <= t number at least sum_w c_w(t) - 3 o(t), with c_w(t) the entries
    // <= t of the row of wavefront w and o(t) those of the row as loaded (a row holds every old entry below its own
    // last slot, and what it dropped is above it).  The smallest t among this wavefront's own entries for which
    // that number reaches K is at least the last slot of the final row.  Rows of the other wavefronts are read as
    // they were last shown, possibly half-way through being shown again: entries only fall, the search only moves
    // past an entry it has seen to be <= t, so a stale or mixed row gives a smaller count and a larger t.
    auto shared_last_slot = [&]() {
#pragma unroll
        for (int s = 0; s < SL; ++s)
            if (lane + 64 * s < K) seen_d[wave * kq + lane + 64 * s] = row.dist[s];
        wave_lds_sync();
        int top = 1;
        while (2 * top <= K) top *= 2;
        // the searches of a lane (its SL entries in the three other rows and in the row as loaded) advance together:
        // their reads do not wait for each other
        int pos[SL][4];
#pragma unroll
        for (int s = 0; s < SL; ++s)
#pragma unroll
            for (int w = 0; w < 4; ++w) pos[s][w] = 0;
        const volatile float* arr[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const int other = w + (w >= wave ? 1 : 0);            // 0..3 without this wavefront, then 4 = the row as loaded
            arr[w] = other < 4 ? seen_d + other * kq : old_d;
        }
        for (int b = top; b > 0; b >>= 1) {
#pragma unroll
            for (int s = 0; s < SL; ++s) {
                const float t = row.dist[s];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const int np = pos[s][w] + b;
                    if (np <= K && arr[w][np - 1] <= t) pos[s][w] = np;
                }
            }
        }
        float best = INFINITY;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const int slot = lane + 64 * s;
            const float t = row.dist[s];
            // (arr[0..2]: the other wavefronts, arr[3]: the row as loaded)
            const int total = slot + 1 + pos[s][0] + pos[s][1] + pos[s][2] - 3 * pos[s][3];
            const uint64_t okm = ballot64(slot < K && t < INFINITY && total >= K);
            if (okm != 0 && best == INFINITY) best = read_lane_f(t, first_lane(okm));   // rows are sorted: the first is the smallest
        }
        // (read after the rows: once the set no longer records, two wavefronts may hold the same candidate)
        const bool recording = *reinterpret_cast<volatile int*>(&n_set_s) < kWgTable / 4 * 3;
        if (recording && lane == 0 && best < INFINITY) atomicMin(&tau_s, __float_as_uint(best));
    };
    // the bounds of this wavefront's marks (upper 16 bits of the fp32 number; non-negative floats order like their bits)
    int lb16[kWgMaxSteps];
#pragma unroll
    for (int u = 0; u < kWgMaxSteps; ++u) {
        const int at = 64 * wave + 256 * u + lane;
        lb16[u] = at < n_marked ? (int)(marked[at] >> 16) : 0x7fffffff;
    }
    auto marks_upto = [&](int from, int upto) {                   // marks with from < bound <= upto
        int n = 0;
#pragma unroll
        for (int u = 0; u < kWgMaxSteps; ++u) {
            if (64 * wave + 256 * u >= n_marked) break;
            n += __popcll(ballot64(lb16[u] > from && lb16[u] <= upto));
        }
        return n;
    };
    int least = 0x7fffffff;                                       // the smallest bound of this wavefront's marks
#pragma unroll
    for (int u = 0; u < kWgMaxSteps; ++u) least = min(least, lb16[u]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) least = min(least, __shfl_xor(least, o, 64));
    int prev = -1;                                                // bounds up to here have been taken
    bool rows_moved = false;                                      // a batch has run since the last slots were compared
    for (int r = 0; r < kWgMaxRounds; ++r) {
        if (rows_moved) {
            shared_last_slot();
            rows_moved = false;
        }
        const int lim = (int)(*reinterpret_cast<volatile uint32_t*>(&tau_s) >> 16);   // bound <= last slot iff its 16 bits <= lim
        if (lim <= prev) break;
        // the smallest limit that takes a batch; everything up to the last slot when that is less (or in the last round)
        int lo = max(prev + 1, min(least, lim)), hi = lim;
        if (r + 1 < kWgMaxRounds) {
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (marks_upto(prev, mid) >= 64 - have) hi = mid;
                else lo = mid + 1;
            }
        } else {
            lo = lim;
        }
        const int upto = lo;
        // first the ids of everything this round takes (all reads travel together), then the candidates one step
        // of the walk after the other
        int c[kWgMaxSteps];
#pragma unroll
        for (int u = 0; u < kWgMaxSteps; ++u) {
            const int at = 64 * wave + 256 * u + lane;
            c[u] = -1;
            if (lb16[u] > prev && lb16[u] <= upto) {              // (false beyond the list)
                const uint32_t e = marked[at];
                c[u] = old_idx[(size_t)srow[e & 255u] * K + ((e >> 8) & 255u)];
            }
        }
#pragma unroll
        for (int u = 0; u < kWgMaxSteps; ++u) {
            if (64 * wave + 256 * u >= n_marked) break;
            bool fresh = c[u] >= 0 && c[u] < N && c[u] != p;
            if (ballot64(fresh) == 0) continue;
            // the shared last slot may have fallen since the ids were requested
            const float tau_now = __uint_as_float(*reinterpret_cast<volatile uint32_t*>(&tau_s));
            if (fresh && __uint_as_float((uint32_t)lb16[u] << 16) > tau_now) fresh = false;
            if (fresh && *reinterpret_cast<volatile int*>(&n_set_s) < kWgTable / 4 * 3) {
                fresh = set_insert(table, kWgTable - 1, c[u], false);
                if (fresh) atomicAdd(&n_set_s, 1);
            }
            const uint64_t fm = ballot64(fresh);
            if (fresh) ids[have + mask_prefix(fm)] = c[u];        // have < 64 here: at most 127 entries
            have += __popcll(fm);
            if (have >= 64) {
                run_batch();
                rows_moved = true;
            }
        }
        prev = upto;
        if (have > 0) {                                           // the next round's limit comes from the rows
            run_batch();
            rows_moved = true;
        }
    }
    if (have > 0) run_batch();
    count_exact(stat, n_exact);

    // ---- 3. one row out of four: wavefronts 0 and 1 take the rows of 2 and 3, then 0 takes the row of 1
    float tau_all = INFINITY;
    auto put_row = [&](int at) {
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            xch[(at * 2 + 0) * (64 * SL) + lane + 64 * s] = row.idx[s];
            xch[(at * 2 + 1) * (64 * SL) + lane + 64 * s] = __float_as_int(row.dist[s]);
        }
    };
    auto take_row = [&](int at) {
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const int c = xch[(at * 2 + 0) * (64 * SL) + lane + 64 * s];
            const float d = __int_as_float(xch[(at * 2 + 1) * (64 * SL) + lane + 64 * s]);
            row.merge(lane + 64 * s < K && c >= 0 && d <= tau_all, c, d);
        }
    };
    // The last slot of the four rows together, once more with all batches done: entries above it (most of what the
    // rows still share with the row as loaded) need not be offered to the row that takes them.
    __syncthreads();
    shared_last_slot();
    __syncthreads();
    tau_all = __uint_as_float(tau_s);
    if (wave >= 2) put_row(wave - 2);
    __syncthreads();
    if (wave < 2) take_row(wave);
    if (wave == 1) put_row(2);
    __syncthreads();
    if (wave == 0) {
        take_row(2);
        if (row.changed) row.store(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K);
    }
}

// marks per point the workgroup-per-point merge can take with the LDS of a compute unit shared by two workgroups
int merge_wg_cap(int dpad, int K, int sl)
{
    const int budget = 78 * 1024 / 4;
    const int fixed = kWgTable + 2 * ((K + 3) & ~3) + dpad + 4 * kWgTile + 6 * 64 * sl + 4 * 128 + 5 * ((K + 3) & ~3);
    return std::min(std::min(budget - fixed, K * K), kWgMaxCap);
}

int merge_wg_ints(int cap, int dpad, int K, int sl)
{
    return (kWgTable + 2 * ((K + 3) & ~3) + dpad + cap + 4 * kWgTile + 6 * 64 * sl + 4 * 128 + 5 * ((K + 3) & ~3) + 3) / 4 * 4;
}

template <int SL>
int launch_merge_wg(const float* points, int N, int D, int K, const int* old_idx, int* knn_idx, float* knn_dist, int cap,
                    int dpad, const uint32_t* pass, const uint16_t* bounds, const int* todo_in, int n_in,
                    int* todo_out, int* n_out, unsigned long long* stat, hipStream_t stream)
{
    const size_t lds = (size_t)merge_wg_ints(cap, dpad, K, SL) * sizeof(int);
    RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore_merge_wg<SL>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    const int n_work = todo_in ? n_in : N;
    hipLaunchKernelGGL((k_explore_merge_wg<SL>), dim3(grid_for_dies((size_t)n_work)), dim3(256), lds, stream, points, N, D, K, old_idx,
                       knn_idx, knn_dist, cap, dpad, pass, bounds, todo_in, n_in, todo_out, n_out, stat);
    RSFK_HIP(hipGetLastError());
    return 0;
}

int next_pow2(int v)
{
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

template <int SL, int WAVES>
int launch_merge(const float* points, int N, int D, int K, const int* old_idx, int* knn_idx, float* knn_dist, int table,
                 int wave_ints, int dpad, const uint32_t* pass, const uint16_t* bounds, const int* todo_in, int n_in,
                 int* todo_out, int* n_out, unsigned long long* stat, const int* order, hipStream_t stream)
{
    const size_t lds = (size_t)WAVES * (size_t)wave_ints * sizeof(int);
    const int n_work = todo_in ? n_in : N;
    dim3 grid(grid_for_dies(((size_t)n_work + WAVES - 1) / WAVES)), block(64 * WAVES);
    if (merge_tile_ints(dpad, merge_direct_max()) == 0) {
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore_merge<SL, WAVES, false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL((k_explore_merge<SL, WAVES, false>), grid, block, lds, stream, points, N, D, K, old_idx, knn_idx,
                           knn_dist, table, wave_ints, dpad, merge_direct_max(), pass, bounds, todo_in, n_in, todo_out, n_out,
                           stat, order);
    } else {
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore_merge<SL, WAVES, true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL((k_explore_merge<SL, WAVES, true>), grid, block, lds, stream, points, N, D, K, old_idx, knn_idx,
                           knn_dist, table, wave_ints, dpad, merge_direct_max(), pass, bounds, todo_in, n_in, todo_out, n_out,
                           stat, order);
    }
    RSFK_HIP(hipGetLastError());
    return 0;
}

// ints of LDS a wavefront of the merge kernel needs for a set of `table` entries: tile | point | set | row | list of
// marks | with_bounds: a bound per place of the set
int merge_wave_ints(int table, int dpad, int K, bool with_bounds = false)
{
    return (merge_tile_ints(dpad, merge_direct_max()) + dpad + table + K + table / 4 * 3 + (with_bounds ? table : 0) + 3) / 4 * 4;
}

int dispatch_merge(int sl, int waves, const float* points, int N, int D, int K, const int* old_idx, int* knn_idx,
                   float* knn_dist, int table, int dpad, const uint32_t* pass, const uint16_t* bounds, const int* todo_in,
                   int n_in, int* todo_out, int* n_out, unsigned long long* stat, const int* order, hipStream_t stream)
{
    const int wi = merge_wave_ints(table, dpad, K, bounds != nullptr);
#define RSFK_MERGE_CASE(SLV, WV)                                                                                        \
    if (sl == SLV && waves == WV)                                                                                       \
        return launch_merge<SLV, WV>(points, N, D, K, old_idx, knn_idx, knn_dist, table, wi, dpad, pass, bounds, \
                                     todo_in, n_in, todo_out, n_out, stat, order, stream);
    RSFK_MERGE_CASE(1, 4) RSFK_MERGE_CASE(1, 2) RSFK_MERGE_CASE(1, 1)
    RSFK_MERGE_CASE(2, 4) RSFK_MERGE_CASE(2, 2) RSFK_MERGE_CASE(2, 1)
    RSFK_MERGE_CASE(4, 4) RSFK_MERGE_CASE(4, 2) RSFK_MERGE_CASE(4, 1)
#undef RSFK_MERGE_CASE
    RSFK_CHECK(false, "exploration: no merge kernel for this configuration");
}

template <int SL, int WAVES>
int launch_one(const float* points, const Bf16Copy& b, int N, int D, int K, const int* old_idx, int* knn_idx,
               float* knn_dist, int table, int wave_ints, int dpad, int rows_per_group, const int* todo, int n_todo,
               unsigned long long* stat, hipStream_t stream)
{
    const size_t lds = (size_t)WAVES * (size_t)wave_ints * sizeof(int);
    RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore<SL, WAVES>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    const int n_work = todo ? n_todo : N;
    dim3 grid((unsigned)((n_work + WAVES - 1) / WAVES)), block(64 * WAVES);
    hipLaunchKernelGGL((k_explore<SL, WAVES>), grid, block, lds, stream, points, b, N, D, K, old_idx, knn_idx, knn_dist,
                       table, wave_ints, dpad, rows_per_group, todo, n_todo, stat);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace

// Does the join keep the lower bounds of the pairs it marks (N K KP 2-byte words)?  Yes for the rows that go to the
// workgroup-per-point merge (below), and for rows of more than 128 dimensions while the array stays below 4 GB: the
// wavefront-per-point merge then takes the candidates of a point nearer bounds first (their rows are long, and every
// candidate that a tighter last slot turns away is a row not read; at 100 dimensions a point has fewer than 64
// candidates, one batch, and the bounds only cost: merge 4.05 against 3.67 ms, join 6.0 against 3.6 ms at 1M x 100).
// RSFK_MERGE_ORDER=0 switches the second case off.
bool explore_join_keeps_bounds(int N, int D, int K)
{
    if (explore_merge_uses_bounds(D, K)) return true;
    static const bool on = [] {
        const char* e = std::getenv("RSFK_MERGE_ORDER");
        return !(e && e[0] == '0');
    }();
    const size_t KP = (size_t)((K + 31) & ~31);
    return on && D > 128 && K <= 64 && (size_t)N * (size_t)K * KP * 2 <= ((size_t)4 << 30);
}

bool explore_merge_uses_bounds(int D, int K)
{
    const int dpad = bf16_valid(D);
    const int lds_ints = 150 * 1024 / 4;
    const int sl = K <= 64 ? 1 : (K <= 128 ? 2 : 4);
    const int want = std::max(next_pow2(K * K + K + 2), next_pow2(4 * K + 66));
    int big_waves = 4;
    while (big_waves > 1 && merge_wave_ints(want, dpad, K) > lds_ints / big_waves) big_waves >>= 1;
    return big_waves < 4 && merge_wg_cap(dpad, K, sl) >= kWgMinCap;
}


// One exploration pass.  old_idx is scratch of N*K ints (receives the snapshot).
// bf may be null (or hold null rows): every candidate then gets the exact distance.
// Rows short enough for the LDS of the merge kernels: the exploration then takes its candidates from the join, and
// the general kernel (the only user of the uncentred copy) only sees what the merge kernels hand back.
bool explore_merge_fits(int D, int K)
{
    const int small_table = std::min(4096, std::max(256, next_pow2(16 * K)));
    return K <= kMaxKJoin && 4 * merge_wave_ints(small_table, bf16_valid(D), K) <= 150 * 1024 / 4;
}

// ws may be null; with a workspace and a bfloat16 copy for the join (bf_join, may be centred; bf must not be)
// the candidates come from the join over the reversed graph (explore_join.hip), which needs rows sorted by
// distance.
int launch_explore(const float* points, const Bf16Copy* bf, const Bf16Copy* bf_join, int N, int D, int K, int* knn_idx,
                   float* knn_dist, int* old_idx, ExploreWorkspace* ws, hipStream_t stream, bool rows_sorted,
                   unsigned long long* stat, const int* order)
{
    if (N <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= kMaxK, "exploration: K must be in 1..1024");
    RSFK_CHECK(bf == nullptr || bf->mu == nullptr, "exploration: the general kernel needs an uncentred copy");
    const int dpad = bf16_valid(D);
    const int small_table = std::min(4096, std::max(256, next_pow2(16 * K)));
    // (rows too long for the LDS of the merge kernel: every point enumerates its own candidates)
    const bool join = ws != nullptr && bf_join != nullptr && bf_join->rows != nullptr && explore_merge_fits(D, K);
    // (rows_sorted: the caller knows that every row is in order, e.g. after the bucket step of a forest)
    if (join && !rows_sorted && launch_sort_rows(knn_idx, knn_dist, N, K, stream)) return 1;
    RSFK_HIP(hipMemcpyAsync(old_idx, knn_idx, sizeof(int) * (size_t)N * (size_t)K, hipMemcpyDeviceToDevice, stream));
    const int fixed = 64 * kPitch + dpad + kQueue2 + K;                 // ints per wavefront besides the set
    const int lds_ints = 150 * 1024 / 4;                                // usable LDS per workgroup
    // The set must hold the seeds (K+1) and all candidates of a group of neighbours with room to
    // spare.  Prefer 4 wavefronts per workgroup; shrink the workgroup, then the group of
    // neighbours, when K is large.
    // (the kernel walks the set 64 entries at a time: it must never be smaller than 64)
    const int floor_table = next_pow2(4 * K + 66);
    const int want = std::max(next_pow2(K * K + K + 2), floor_table);
    RSFK_CHECK(fixed + floor_table <= lds_ints, "exploration: D or K too large for the LDS budget");
    int waves = 4;
    int table = want;
    while (waves > 1 && fixed + table > lds_ints / waves) waves >>= 1;
    while (table > floor_table && fixed + table > lds_ints / waves) table >>= 1;
    int rows_per_group = K;
    if (table < want) rows_per_group = std::max(1, (table * 3 / 4 - K - 1) / K);
    RSFK_CHECK(table >= 64 && (table & (table - 1)) == 0 && rows_per_group >= 1, "exploration: bad set size");
    const int wave_ints = (fixed + table + 3) / 4 * 4;
    Bf16Copy b;
    if (bf) b = *bf;
    const int sl = row_slots(K);
    const int* todo = nullptr;
    int n_todo = 0;
    if (join) {
        // Marks from the join, then the merge kernel with a small set (little LDS, many wavefronts per CU).
        // The points it cannot take come back in a list and get a second launch with the largest set that
        // fits; what is left after that goes to the general kernel below.
        if (launch_explore_join(ws, *bf_join, N, D, K, old_idx, knn_dist, stream, order)) return 1;
        const uint32_t* pass = explore_ws_pass(ws);
        int* listA = explore_ws_todo(ws, 0);
        int* listB = explore_ws_todo(ws, 1);
        int* host_n = explore_ws_host_count(ws);
        // (the bounds of the join, when it kept them and the set with a bound per place still fits)
        const uint16_t* wave_bounds = explore_ws_bounds(ws);
        if (4 * merge_wave_ints(small_table, dpad, K, true) > lds_ints) wave_bounds = nullptr;
        int big_table = want, big_waves = 4;
        while (big_waves > 1 && merge_wave_ints(big_table, dpad, K) > lds_ints / big_waves) big_waves >>= 1;
        // fewer than four wavefronts per workgroup would leave the compute units nearly empty: such sets get one
        // workgroup per point instead
        const bool per_wg = big_waves < 4;
        const int wg_cap = merge_wg_cap(dpad, K, sl);
        if (!per_wg)
            while (big_table > small_table && merge_wave_ints(big_table, dpad, K) > lds_ints / big_waves) big_table >>= 1;
        const bool second = per_wg ? wg_cap >= kWgMinCap : big_table > small_table;
        auto merge_wg = [&](const int* list, int n) {
            const uint16_t* bounds = explore_ws_bounds(ws);
            if (sl == 1)
                return launch_merge_wg<1>(points, N, D, K, old_idx, knn_idx, knn_dist, wg_cap, dpad, pass, bounds, list, n, listB,
                                          listB + N, stat, stream);
            if (sl == 2)
                return launch_merge_wg<2>(points, N, D, K, old_idx, knn_idx, knn_dist, wg_cap, dpad, pass, bounds, list, n, listB,
                                          listB + N, stat, stream);
            return launch_merge_wg<4>(points, N, D, K, old_idx, knn_idx, knn_dist, wg_cap, dpad, pass, bounds, list, n, listB,
                                      listB + N, stat, stream);
        };
        // Where the workgroup-per-point kernel may follow, the small set is first tried on a sample (the first points of
        // the order they are taken in): when it has to hand most of them back -- rows of many neighbours that are far
        // from done have thousands of marks each -- the launch over all points would only find that out for every
        // one of them (70,000 x 784, K = 90, 10 trees: all of them, 0.9 ms of a 25 ms pass).
        constexpr int kSample = 2048;
        int first = 0;                                    // points the small set has been tried on
        bool rest_per_wg = false;
        if (second && per_wg && order != nullptr && N > 2 * kSample) {
            if (dispatch_merge(sl, 4, points, N, D, K, old_idx, knn_idx, knn_dist, small_table, dpad, pass, wave_bounds, order,
                               kSample, listA, listA + N, stat, nullptr, stream))
                return 1;
            RSFK_HIP(hipMemcpyAsync(host_n, listA + N, sizeof(int), hipMemcpyDeviceToHost, stream));
            RSFK_HIP(hipStreamSynchronize(stream));
            first = kSample;
            rest_per_wg = *host_n > kSample / 2;
        }
        if (rest_per_wg) {
            // everything but the sample straight to the workgroup-per-point kernel (its list: the rest of the order)
            if (merge_wg(order + first, N - first)) return 1;
        } else if (dispatch_merge(sl, 4, points, N, D, K, old_idx, knn_idx, knn_dist, small_table, dpad, pass, wave_bounds,
                                  first > 0 ? order + first : nullptr, first > 0 ? N - first : 0, listA, listA + N, stat,
                                  first > 0 ? nullptr : order, stream)) {
            return 1;
        }
        RSFK_HIP(hipMemcpyAsync(host_n, listA + N, sizeof(int), hipMemcpyDeviceToHost, stream));
        RSFK_HIP(hipStreamSynchronize(stream));
        n_todo = *host_n;                                 // what the small set handed back (of the sample, or of all points)
        todo = listA;
        if (n_todo == 0 && !rest_per_wg) return 0;
        if (second) {
            int rc = 0;
            if (n_todo == 0)
                rc = 0;
            else if (!per_wg)
                rc = dispatch_merge(sl, big_waves, points, N, D, K, old_idx, knn_idx, knn_dist, big_table, dpad, pass,
                                    nullptr, listA, n_todo, listB, listB + N, stat, nullptr, stream);
            else
                rc = merge_wg(listA, n_todo);
            if (rc)
                return 1;
            RSFK_HIP(hipMemcpyAsync(host_n, listB + N, sizeof(int), hipMemcpyDeviceToHost, stream));
            RSFK_HIP(hipStreamSynchronize(stream));
            n_todo = *host_n;
            if (n_todo == 0) return 0;
            todo = listB;
        }
    }
#define RSFK_EXPLORE_CASE(SLV, WV)                                                                                      \
    if (sl == SLV && waves == WV)                                                                                       \
        return launch_one<SLV, WV>(points, b, N, D, K, old_idx, knn_idx, knn_dist, table, wave_ints, dpad,              \
                                   rows_per_group, todo, n_todo, stat, stream);
    RSFK_EXPLORE_CASE(1, 4) RSFK_EXPLORE_CASE(1, 2) RSFK_EXPLORE_CASE(1, 1)
    RSFK_EXPLORE_CASE(2, 4) RSFK_EXPLORE_CASE(2, 2) RSFK_EXPLORE_CASE(2, 1)
    RSFK_EXPLORE_CASE(4, 4) RSFK_EXPLORE_CASE(4, 2) RSFK_EXPLORE_CASE(4, 1)
    RSFK_EXPLORE_CASE(8, 4) RSFK_EXPLORE_CASE(8, 2) RSFK_EXPLORE_CASE(8, 1)
    RSFK_EXPLORE_CASE(16, 4) RSFK_EXPLORE_CASE(16, 2) RSFK_EXPLORE_CASE(16, 1)
#undef RSFK_EXPLORE_CASE
    RSFK_CHECK(false, "exploration: no kernel for this configuration");
}

}  // namespace rsfk
