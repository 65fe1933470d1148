// Bucket K-NN for buckets of at most 64 points and K <= 64 with the pair matrix
// bounded on the matrix cores first: same function and same results as the kernel in
// bucket_knn_small.hip (see bucket_knn.hip for the reference kernels both replace),
// same decomposition (one bucket per workgroup of two wavefronts, many workgroups
// per compute unit), but the sequential fp32 chains -- nearly all of the arithmetic
// of that kernel, and what bounds it -- are only run for the pairs that may change a
// row.
//
// A pair (i, j) changes nothing unless its distance is at most the last slot of row
// i or of row j.  Once the rows are good that holds for a small share of the pairs
// (none at all in most buckets of clustered high-dimensional data), so:
//
//   1. the fp32 rows pass through LDS, kChunk dimensions at a time, the next chunk
//      travelling while this one is used; the wavefronts read them as matrix-core
//      operands, every value split into two bfloat16 numbers (mfma_split.hpp), and
//      accumulate the three 32 x 32 quadrants of the upper triangle of the Gram
//      matrix (wavefront 0: the first diagonal quadrant and the off-diagonal one,
//      wavefront 1: the second diagonal quadrant) and the squared norms;
//   2. with S = n_i + n_j and d~ = S - 2 G_ij the real-number distance is at least
//      d~ - c S (c: split_gram_error_coefficient) and the fp32 chain of the exact
//      path returns at least (1 - gamma) times the real-number distance,
//      gamma = (D + 8) 2^-22: the pair is dropped iff
//      (d~ - c S)(1 - gamma) > max(last slot of row i, last slot of row j).
//      NaN or infinite intermediate values never drop a pair;
//   3. the pairs that are left go to a list in LDS.  If it is empty the workgroup is
//      done.  Otherwise the rows pass through LDS once more (not when D <= kChunk:
//      they are still there) and each thread runs the sequential fused multiply-add
//      chains of its pairs of the list (arithmetic of euclidean_distance_sqr,
//      compute_knn_from_buckets.cu:40-54: a pair has the same distance value as in
//      every other kernel);
//   4. an exact distance that is not above the last slot of a row goes into the
//      bucket's distance matrix in LDS and sets the member's bit in that row's
//      candidate set (nothing else of the matrix is written or read); the rows
//      with a candidate are merged as in the other kernel.
//
// Requires every K-NN row to be sorted on entry (the last slot is its maximum);
// launch_sort_rows establishes that once per build.
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"
#include "mfma_split.hpp"
#include "bucket_small_body.hpp"
#include <algorithm>
#include <cstdlib>

namespace rsfk {

namespace {

constexpr int kCap = kBucketSplit;          // largest bucket this kernel takes
static_assert(kCap == 64, "two 32-row operand blocks and lane-per-candidate merge assume 64");
constexpr int kThreads = 128;
constexpr int kDistPitch = kCap + 1;
constexpr int kChunk = 64;                 // dimensions staged at once (a multiple of 16)
constexpr int kMaxPairs = kCap * (kCap - 1) / 2;
constexpr int kMaxRounds = (kMaxPairs + kThreads - 1) / kThreads;     // listed pairs per thread
// Pairs the list holds.  A bucket with more pairs to evaluate (nearly half of those of a full bucket: the first trees
// of a build) evaluates all its pairs, which then need no list.  With this size the workgroup's LDS is 20 KB and eight
// workgroups share a compute unit.
constexpr int kListCap = 752;

// LDS after the row / distance region: ids, last slots, candidate sets, norms as seen by either wavefront, pair
// counter, list
struct alignas(16) ScreenMeta {
    int lids[kCap];
    float tau[kCap];
    unsigned long long cand[kCap];          // bit j of cand[i]: member j is at a distance not above the last slot of row i
    float nrm[2][kCap];
    int n_pairs[4];
    uint16_t list[kListCap];
};

// The rows of the bucket on their way from HBM to LDS: 16 lanes (a quarter wavefront) per row, a lane moves 16 bytes
// of kLoads rows.  Zeros beyond D and for the rows beyond s.
struct RowLoads {
    static constexpr int kPieces = kChunk / 4;
    static constexpr int kRowsPerPass = kThreads / kPieces;
    static constexpr int kLoads = kCap / kRowsPerPass;
    float4 v[kLoads];

    __device__ __forceinline__ void request(const int* __restrict__ lids, int s, const float* __restrict__ points, int D,
                                            int d0, bool vec_ok)
    {
        const int piece = threadIdx.x & (kPieces - 1);
        const int r0 = threadIdx.x / kPieces;
        const int d = d0 + 4 * piece;
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int m = r0 + i * kRowsPerPass;
            v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < s && d < D) {
                const float* src = points + (size_t)lids[m] * (size_t)D + d;
                if (vec_ok) {
                    v[i] = *reinterpret_cast<const float4*>(src);
                } else {
                    v[i].x = src[0];
                    if (d + 1 < D) v[i].y = src[1];
                    if (d + 2 < D) v[i].z = src[2];
                    if (d + 3 < D) v[i].w = src[3];
                }
            }
        }
    }

    __device__ __forceinline__ void commit(float* __restrict__ rows, int pitch) const
    {
        const int piece = threadIdx.x & (kPieces - 1);
        const int r0 = threadIdx.x / kPieces;
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
            *reinterpret_cast<float4*>(&rows[(r0 + i * kRowsPerPass) * pitch + 4 * piece]) = v[i];
    }
};

// SINGLE: D <= kChunk, the rows are staged once and stay in LDS until the exact chains have run.  Otherwise the Gram
// pass takes the chunks from the last to the first, so that the first one is still in LDS when the exact chains --
// which must run from dimension 0 upwards -- begin; only the chunks after it pass through LDS a second time, and the
// first of those is requested before the bounds are evaluated.
// stats (may be null): the workgroups whose number is a multiple of 2^stat_shift add pairs of the bucket << 32 | pairs
// that got an exact distance to one of its 8 words (a sample of the buckets, see small_bucket_body).
// The work of one workgroup on bucket blockIdx.x; lds: kScreenLdsBytes bytes of LDS.
constexpr int kPitch = kChunk + 4;                        // an odd number of 16-byte units: rows start in different banks
constexpr int kRegion = kCap * kPitch > kCap * kDistPitch ? kCap * kPitch : kCap * kDistPitch;
constexpr size_t kScreenLdsBytes = sizeof(float) * kRegion + sizeof(ScreenMeta);
static_assert(kScreenLdsBytes <= 160 * 1024 / 8, "eight workgroups per compute unit");

template <bool SINGLE>
__device__ __forceinline__ void screen_bucket_body(float* __restrict__ lds, const float* __restrict__ points, int D, int K,
                                                   const int* __restrict__ ids, const int* __restrict__ starts,
                                                   const int* __restrict__ sizes, int stride, int* __restrict__ knn_idx,
                                                   float* __restrict__ knn_dist, float c_err, float one_minus_gamma,
                                                   unsigned long long* __restrict__ stats, int stat_shift)
{
    float* rows = lds;                                    // kRegion floats: the rows, later the distance matrix
    float* dist = lds;
    ScreenMeta& M = *reinterpret_cast<ScreenMeta*>(lds + kRegion);

    const int bkt = blockIdx.x;
    const int s = sizes[bkt];
    const size_t first = starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride;     // (asked for together with s)
    if (s < 2 || s > kCap) return;
    const int* bid = ids + first;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int n_chunks = SINGLE ? 1 : (D + kChunk - 1) / kChunk;
    const int fm = wave + 2 * lane;                       // bit u of a member set: member wave + 2 u
    const int* lids = M.lids;

    // (a member's last slot is requested here and put into LDS once the rows have been requested too: the two trips to
    // memory then overlap; nobody reads the last slots before the bounds)
    float tau_own = 0.0f;
    if (tid < kCap) {
        const int id = tid < s ? bid[tid] : -1;
        M.lids[tid] = id;
        if (id >= 0) tau_own = knn_dist[(size_t)id * (size_t)K + (K - 1)];
        M.cand[tid] = 0ull;
    }
    if (tid == kCap) M.n_pairs[0] = 0;
    __syncthreads();
    // ---- 1. Gram quadrants and norms
    const bool two_blocks = s > 32;
    const bool act0 = wave == 0 || two_blocks;            // this wavefront's diagonal quadrant (block `wave`)
    const bool act1 = wave == 0 && two_blocks;            // quadrant (block 0, block 1)
    RowLoads ld;
    {
        f32x16 g0, g1;
#pragma unroll
        for (int i = 0; i < 16; ++i) { g0[i] = 0.0f; g1[i] = 0.0f; }
        float n0 = 0.0f, n1 = 0.0f;
        const float* pa = rows + (32 * wave + (lane & 31)) * kPitch + 8 * (lane >> 5);
        const float* pb = rows + (32 + (lane & 31)) * kPitch + 8 * (lane >> 5);
        ld.request(lids, s, points, D, (n_chunks - 1) * kChunk, vec_ok);
        if (tid < kCap) M.tau[tid] = tau_own;
        for (int step = 0; step < n_chunks; ++step) {
            const int c = n_chunks - 1 - step;           // the last chunk first
            if (!SINGLE && step > 0) __syncthreads();    // the previous chunk has been consumed
            ld.commit(rows, kPitch);
            __syncthreads();
            // the next chunk of this pass; after the last one (chunk 0) the first chunk of the second pass
            if (!SINGLE) ld.request(lids, s, points, D, (c > 0 ? c - 1 : 1) * kChunk, vec_ok);
            const int ksteps = min(kChunk, (D - c * kChunk + 15) & ~15) >> 4;
            if (act0) {
                for (int k = 0; k < ksteps; ++k) {
                    bf16x8 ah, al;
                    load_split(pa + 16 * k, ah, al, n0);
                    g0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, ah, g0, 0, 0, 0);
                    g0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, al, g0, 0, 0, 0);
                    g0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, ah, g0, 0, 0, 0);
                    if (act1) {
                        bf16x8 bh, bl;
                        load_split(pb + 16 * k, bh, bl, n1);
                        g1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh, g1, 0, 0, 0);
                        g1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl, g1, 0, 0, 0);
                        g1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh, g1, 0, 0, 0);
                    }
                }
            }
        }
        // a lane holds the squares of half of the dimensions of its row: add the two halves
        n0 += __shfl_xor(n0, 32, 64);
        n1 += __shfl_xor(n1, 32, 64);
        float* nrm = M.nrm[wave];                     // a wavefront only reads back what it wrote itself
        if (lane < 32) {
            nrm[32 * wave + lane] = n0;
            if (wave == 0) nrm[32 + lane] = n1;
        }
        wave_lds_sync();

        // ---- 2. screen.  Accumulator i of lane l is pair (m, n), m = 32 qi + 8 (i / 4) + i % 4 + 4 (l / 32),
        //         n = 32 qj + l % 32; in a diagonal quadrant only m < n counts
        auto screen = [&](const f32x16& g, int qi, int qj) {
            const int n = 32 * qj + (lane & 31);
            const float nn = nrm[n];
            const float tn = M.tau[n];
            const int mbase = 32 * qi + 4 * (lane >> 5);
            uint32_t bits = 0;
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                // four consecutive members at a time (16-byte reads of their norms and last slots)
                const int m0 = mbase + 8 * i4;
                const float4 nm4 = *reinterpret_cast<const float4*>(&nrm[m0]);
                const float4 tm4 = *reinterpret_cast<const float4*>(&M.tau[m0]);
                const float nm[4] = {nm4.x, nm4.y, nm4.z, nm4.w}, tm[4] = {tm4.x, tm4.y, tm4.z, tm4.w};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int i = 4 * i4 + c, m = m0 + c;
                    const float S = nm[c] + nn;
                    const float dt = __builtin_fmaf(-2.0f, g[i], S);
                    const float lower = (dt - __builtin_fmaf(c_err, S, 1e-35f)) * one_minus_gamma;
                    // a NaN bound never drops a pair (the comparison is false); a NaN last slot cannot occur: rows
                    // only hold what passed `distance < last slot`, +inf where they are empty
                    const bool drop = lower > fmaxf(tm[c], tn);
                    const bool valid = n < s && (qi == qj ? m < n : m < s);
                    if (valid && !drop) bits |= 1u << i;
                }
            }
            const int cnt = __popc(bits);
            int at = cnt ? atomicAdd(&M.n_pairs[0], cnt) : 0;
            while (bits) {
                const int i = __ffs(bits) - 1;
                bits &= bits - 1;
                const int m = mbase + 8 * (i >> 2) + (i & 3);
                if (at < kListCap) M.list[at] = (uint16_t)(m | (n << 6));
                ++at;
            }
        };
        if (act0) screen(g0, wave, wave);
        if (act1) screen(g1, 0, 1);
    }
    __syncthreads();
    const int n_passed = M.n_pairs[0];
    if (stats && tid == 0 && (bkt & ((1 << stat_shift) - 1)) == 0)
        atomicAdd(&stats[(bkt >> stat_shift) & 7], ((unsigned long long)(s * (s - 1) / 2) << 32) | (unsigned long long)n_passed);
    if (n_passed == 0) return;                        // no pair of this bucket can change a row

    // ---- 3. exact distances of the listed pairs: thread t takes entries t, t + 128, ...
    // More pairs than the list holds: all pairs, in the order (a, a + o mod s) for o = 1 .. (s - 1) / 2 and all a, then
    // o = s / 2 with a < s / 2 when s is even: pair number p has o = p / s + 1, a = p mod s.
    const bool all_pairs = n_passed > kListCap;
    const int n_list = all_pairs ? s * (s - 1) / 2 : n_passed;
    const int rounds = (n_list + kThreads - 1) / kThreads;
    const float inv_s = 1.0f / (float)s;
    float acc[kMaxRounds];
#pragma unroll
    for (int r = 0; r < kMaxRounds; ++r) acc[r] = 0.0f;
    auto entry = [&](int r) {                         // idle threads compute pair (0, 0)
        const int p = tid + r * kThreads;
        if (p >= n_list) return 0u;
        if (!all_pairs) return (uint32_t)M.list[p];
        // p / s (exact: p < 2048 and (p + 0.5) / s is never within 1 / 128 of an integer)
        const int q = (int)(((float)p + 0.5f) * inv_s);
        const int a = p - q * s;
        int b = a + q + 1;
        if (b >= s) b -= s;
        return (uint32_t)(a | (b << 6));
    };
    auto chains = [&](int np) {
#pragma unroll
        for (int r = 0; r < kMaxRounds; ++r) {
            if (r < rounds) {
                const uint32_t e = entry(r);
                const float* ra = rows + (e & 63u) * (uint32_t)kPitch;
                const float* rb = rows + (e >> 6) * (uint32_t)kPitch;
                float a = acc[r];
                // (not unrolled all the way: with a whole chunk's reads hoisted the registers do not suffice)
#pragma unroll 4
                for (int q = 0; q < np; ++q) {
                    const float4 x = *reinterpret_cast<const float4*>(ra + 4 * q);
                    const float4 y = *reinterpret_cast<const float4*>(rb + 4 * q);
                    float df;
                    df = x.x - y.x; a = __builtin_fmaf(df, df, a);
                    df = x.y - y.y; a = __builtin_fmaf(df, df, a);
                    df = x.z - y.z; a = __builtin_fmaf(df, df, a);
                    df = x.w - y.w; a = __builtin_fmaf(df, df, a);
                }
                acc[r] = a;
            }
        }
    };
    if (SINGLE) {
        chains((D + 3) >> 2);                         // the rows are still in LDS
    } else {
        chains(kChunk >> 2);                          // so is the first chunk; the second is on its way
        for (int c = 1; c < n_chunks; ++c) {
            __syncthreads();
            ld.commit(rows, kPitch);
            __syncthreads();
            if (c + 1 < n_chunks) ld.request(lids, s, points, D, (c + 1) * kChunk, vec_ok);
            chains(min(kChunk, (D - c * kChunk + 3) & ~3) >> 2);
        }
    }
    __syncthreads();                                  // rows no longer needed: the region becomes the distance matrix
    // (only the entries a row may take are written, and cand says which they are: nothing else of the matrix is read)
#pragma unroll
    for (int r = 0; r < kMaxRounds; ++r) {
        if (tid + r * kThreads < n_list) {
            const uint32_t e = entry(r);
            const int i = (int)(e & 63u), j = (int)(e >> 6);
            const float d = acc[r];
            if (d <= M.tau[i]) {
                dist[i * kDistPitch + j] = d;
                atomicOr(&M.cand[i], 1ull << j);
            }
            if (d <= M.tau[j]) {
                dist[j * kDistPitch + i] = d;
                atomicOr(&M.cand[j], 1ull << i);
            }
        }
    }
    __syncthreads();

    // ---- 4. top-K update: a wavefront walks its members that have a candidate, eight at a time, with the rows of the
    //         next eight in flight
    const int my_id = lids[lane];
    uint32_t active = (uint32_t)ballot64(lane < 32 && M.cand[fm < kCap ? fm : 0] != 0ull);
    auto next_member = [&]() {
        if (active == 0) return -1;
        const int u = __ffs(active) - 1;
        active &= active - 1;
        return wave + 2 * u;
    };
    auto load_row = [&](int i, int& ri, float& rd) {
        ri = -2;
        rd = INFINITY;
        if (i >= 0 && lane < K) {
            const size_t at = (size_t)lids[i] * (size_t)K + lane;
            ri = knn_idx[at];
            rd = knn_dist[at];
        }
    };
    constexpr int kAhead = 8;
    int cur_i[kAhead], cur_ri[kAhead], nxt_i[kAhead], nxt_ri[kAhead];
    float cur_rd[kAhead], nxt_rd[kAhead];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
        cur_i[u] = next_member();
        load_row(cur_i[u], cur_ri[u], cur_rd[u]);
    }
    while (cur_i[0] >= 0) {
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            nxt_i[u] = next_member();
            load_row(nxt_i[u], nxt_ri[u], nxt_rd[u]);
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int i = cur_i[u];
            if (i < 0) break;
            KnnRow<1> row;
            row.idx[0] = cur_ri[u];
            row.dist[0] = cur_rd[u];
            row.init_sorted(K);
            const bool offered = (M.cand[i] >> lane) & 1ull;
            row.merge(offered, my_id, offered ? dist[i * kDistPitch + lane] : INFINITY);
            if (row.changed) {
                const size_t at = (size_t)lids[i] * (size_t)K;
                row.store(knn_idx + at, knn_dist + at);
            }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) { cur_i[u] = nxt_i[u]; cur_ri[u] = nxt_ri[u]; cur_rd[u] = nxt_rd[u]; }
    }
}

template <bool SINGLE>
__global__ __launch_bounds__(kThreads, 4) void k_bucket_knn_screen(const float* __restrict__ points, int D, int K,
                                                                   const int* __restrict__ ids,
                                                                   const int* __restrict__ starts,
                                                                   const int* __restrict__ sizes, int stride,
                                                                   int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                                   float c_err, float one_minus_gamma)
{
    extern __shared__ __align__(16) float lds_s[];
    screen_bucket_body<SINGLE>(lds_s, points, D, K, ids, starts, sizes, stride, knn_idx, knn_dist, c_err, one_minus_gamma,
                               nullptr, 0);
}

// The kernel of a forest's trees: every workgroup looks at the numbers of pairs the tree before this one left behind
// (prev: 8 words, pairs << 32 | pairs that had to be evaluated exactly, as both forms of the kernel count them in a
// sample of the buckets) and
// takes the screened form when fewer than share_q16 / 65536 of the pairs had to be, the direct form otherwise (and
// for the first tree, prev == null).  One scalar load and a few scalar instructions per workgroup; both forms leave
// their own numbers in stats for the next tree.  All K-NN rows sorted on entry.
template <bool SINGLE>
__global__ __launch_bounds__(kThreads, 4) void k_bucket_knn_auto(const float* __restrict__ points, int D, int K,
                                                                 const int* __restrict__ ids, const int* __restrict__ starts,
                                                                 const int* __restrict__ sizes, int* __restrict__ knn_idx,
                                                                 float* __restrict__ knn_dist, float c_err,
                                                                 float one_minus_gamma, int chunk, int pitch,
                                                                 int region_floats,
                                                                 const unsigned long long* __restrict__ prev,
                                                                 unsigned int share_q16,
                                                                 unsigned long long* __restrict__ stats, int stat_shift)
{
    extern __shared__ __align__(16) float lds_a[];
    bool screened = share_q16 == kScreenAlways;
    if (prev && !screened) {
        unsigned long long sum = 0;                      // (the halves cannot carry into each other: a tree has < 2^32 pairs)
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += prev[i];
        const unsigned long long listed = sum & 0xffffffffull, total = sum >> 32;
        screened = total > 0 && (listed << 16) < total * share_q16;
    }
    if (screened)
        screen_bucket_body<SINGLE>(lds_a, points, D, K, ids, starts, sizes, 0, knn_idx, knn_dist, c_err, one_minus_gamma, stats,
                                   stat_shift);
    else
        small_bucket::small_bucket_body<kCap, kThreads, 33>(lds_a, points, D, K, ids, starts, sizes, 0, 2, knn_idx, knn_dist,
                                                            chunk, pitch, region_floats, 1, stats, stat_shift);
}

// one wavefront per row: rows that are not sorted by distance are rebuilt by insertion
template <int SL>
__global__ __launch_bounds__(256) void k_sort_rows(int* __restrict__ knn_idx, float* __restrict__ knn_dist, int N, int K)
{
    const int row_id = (int)((blockIdx.x * (size_t)blockDim.x + threadIdx.x) >> 6);
    if (row_id >= N) return;
    KnnRow<SL> row;
    row.load(knn_idx + (size_t)row_id * K, knn_dist + (size_t)row_id * K, K);
    if (row.changed) row.store(knn_idx + (size_t)row_id * K, knn_dist + (size_t)row_id * K);
}

}  // namespace

int launch_sort_rows(int* knn_idx, float* knn_dist, int N, int K, hipStream_t stream)
{
    if (N <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= kMaxK, "sort rows: K must be in 1..1024");
    const dim3 grid((unsigned)((N + 3) / 4)), block(256);
    if (K <= 64) hipLaunchKernelGGL(k_sort_rows<1>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    else if (K <= 128) hipLaunchKernelGGL(k_sort_rows<2>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    else if (K <= 256) hipLaunchKernelGGL(k_sort_rows<4>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    else if (K <= 512) hipLaunchKernelGGL(k_sort_rows<8>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    else hipLaunchKernelGGL(k_sort_rows<16>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    RSFK_HIP(hipGetLastError());
    return 0;
}

// Buckets of 2..64 points (others are skipped); every K-NN row sorted on entry.
int launch_bucket_knn_screen(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                             int n_buckets, int stride, int* knn_idx, float* knn_dist, hipStream_t stream)
{
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 64 && D >= 1, "screened small-bucket kernel: K must be in 1..64 and D positive");
    const float c_err = split_gram_error_coefficient((D + 15) & ~15);
    const float one_minus_gamma = 1.0f - (float)(D + 8) * (1.0f / 4194304.0f);
    RSFK_CHECK(one_minus_gamma > 0.5f, "screened small-bucket kernel: D too large");
    const dim3 grid((unsigned)n_buckets), block(kThreads);
    if (D <= kChunk)
        hipLaunchKernelGGL(k_bucket_knn_screen<true>, grid, block, kScreenLdsBytes, stream, points, D, K, ids, starts, sizes,
                           stride, knn_idx, knn_dist, c_err, one_minus_gamma);
    else
        hipLaunchKernelGGL(k_bucket_knn_screen<false>, grid, block, kScreenLdsBytes, stream, points, D, K, ids, starts, sizes,
                           stride, knn_idx, knn_dist, c_err, one_minus_gamma);
    RSFK_HIP(hipGetLastError());
    return 0;
}

// The small buckets (2..64 points, starts / sizes form) of one tree of a forest; every K-NN row sorted on entry.
// prev: the 8 words a launch of this kind (or of either form) left for the tree before, or null for the first tree;
// stats: 8 zeroed words for this tree.  The form of the kernel is chosen on the device from prev (k_bucket_knn_auto).
int launch_bucket_knn_auto(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                           int n_buckets, int* knn_idx, float* knn_dist, const unsigned long long* prev,
                           unsigned long long* stats, hipStream_t stream)
{
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 64 && D >= 1, "small-bucket kernel: K must be in 1..64 and D positive");
    const float c_err = split_gram_error_coefficient((D + 15) & ~15);
    const float one_minus_gamma = 1.0f - (float)(D + 8) * (1.0f / 4194304.0f);
    RSFK_CHECK(one_minus_gamma > 0.5f, "small-bucket kernel: D too large");
    int chunk, pitch;
    small_bucket::small_bucket_shape(D, &chunk, &pitch);
    const int region_floats = small_bucket::small_bucket_region_floats<kCap, kThreads, 33>(pitch);
    const size_t lds = std::max(kScreenLdsBytes, small_bucket::small_bucket_lds_bytes<kCap, kThreads, 33>(pitch));
    const unsigned int share_q16 = bucket_screen_share_q16();
    // about 256 to 512 of the buckets are counted
    int stat_shift = 0;
    while ((n_buckets >> (stat_shift + 1)) >= 256) ++stat_shift;
    const dim3 grid((unsigned)n_buckets), block(kThreads);
    if (D <= kChunk)
        hipLaunchKernelGGL(k_bucket_knn_auto<true>, grid, block, lds, stream, points, D, K, ids, starts, sizes, knn_idx, knn_dist,
                           c_err, one_minus_gamma, chunk, pitch, region_floats, prev, share_q16, stats, stat_shift);
    else
        hipLaunchKernelGGL(k_bucket_knn_auto<false>, grid, block, lds, stream, points, D, K, ids, starts, sizes, knn_idx, knn_dist,
                           c_err, one_minus_gamma, chunk, pitch, region_floats, prev, share_q16, stats, stat_shift);
    RSFK_HIP(hipGetLastError());
    return 0;
}

// The small buckets of a tree take the screened form of the kernel when, in the tree before, less than this share
// (in 1 / 65536) of the pairs had to be evaluated exactly.  Every pair that passes the bound costs more in the
// screened form (its chain reads two rows from LDS on its own, where the direct form shares them among the four pairs
// of a block, and the rows pass through LDS twice), every pair that does not costs less: measured on uniform 100-
// dimensional and clustered 256-dimensional points the two forms take the same time when about four fifths of the
// pairs pass (the second tree of a build), and the screened form is ahead from the third tree on (43 to 48 %).  RSFK_BUCKET_SCREEN=<percent> overrides; "never" = 0; "always" = the screened form for every tree and for the
// stage-level call as well (kScreenAlways).
unsigned int bucket_screen_share_q16()
{
    double pct = 60.0;
    const char* e = std::getenv("RSFK_BUCKET_SCREEN");          // (read at every call: tests change it)
    if (e && *e) {
        if (e[0] == 'a') return kScreenAlways;
        pct = e[0] >= '0' && e[0] <= '9' ? std::atof(e) : 0.0;
    }
    pct = std::min(100.0, std::max(0.0, pct));
    return (unsigned int)(pct * 65536.0 / 100.0 + (pct >= 100.0 ? 1.0 : 0.0));
}

}  // namespace rsfk
