// The small-bucket K-NN kernel's work on one bucket, as a device function, so that the kernel of
// bucket_knn_small.hip and the kernel that chooses between this and the screened form (bucket_knn_screen.hip) share
// it.  See bucket_knn_small.hip for what it does.
#pragma once
#include "rsfk_common.hpp"
#include "knn_list.hpp"

namespace rsfk {
namespace small_bucket {

constexpr int kMaxChunk = 64;               // dimensions staged at once

// CAP = largest bucket, THREADS = workgroup size, SPACING = LDS rows between members 2t and 2t+1: the 2x2 block
// (a, b) reads rows a, a + SPACING, b, b + SPACING -- consecutive a (consecutive threads) give conflict-free 16-byte
// reads (the pitch is an odd number of 16-byte units).
// Does the row in the registers of the wavefront (slot k in lane k) hold nothing but, possibly, the point itself in
// slot 0?  Empty slots are (-1, +inf).
__device__ __forceinline__ bool fresh_row(int ri, float rd, int self_id, int K)
{
    const int lane = lane_id();
    const bool empty = ri == -1 && rd == INFINITY;
    const bool fine = lane >= K || empty || (lane == 0 && ri == self_id);
    return ballot64(!fine) == 0;
}

// dv[v] of lane l: distance of candidate l + 64 v of a fresh row (the point itself included, with the distance its row
// holds), +inf where there is none; n candidates in all.  When no two finite distances are equal, the place of a
// candidate in the row ordered by (distance, index) is the number of finite distances below its own: dv[v] is
// replaced by that number (as an integer; -1 for a candidate that is not finite) and the result is true.  With equal
// distances the result is false and dv is unchanged.
template <int CL>
__device__ __forceinline__ bool place_by_rank(float (&dv)[CL], int n)
{
    int rank[CL];
#pragma unroll
    for (int v = 0; v < CL; ++v) rank[v] = 0;
#pragma unroll
    for (int u = 0; u < CL; ++u) {
        const int nu = min(kWave, n - kWave * u);
        // four at a time (lanes past the last candidate hold +inf and count for nothing)
        for (int j = 0; j < nu; j += 4) {
            float dj[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) dj[x] = read_lane_f(dv[u], j + x);
#pragma unroll
            for (int x = 0; x < 4; ++x)
#pragma unroll
                for (int v = 0; v < CL; ++v) rank[v] += dj[x] < dv[v] ? 1 : 0;
        }
    }
    // equal distances give equal numbers: all numbers of the finite candidates must differ
    uint32_t seen[4] = {0u, 0u, 0u, 0u};                 // bit r of the 128-bit set: some candidate has number r
    int n_finite = 0;
#pragma unroll
    for (int v = 0; v < CL; ++v) {
        const bool fin = dv[v] < INFINITY;
        n_finite += __popcll(ballot64(fin));
#pragma unroll
        for (int w = 0; w < 2 * CL; ++w) seen[w] |= (fin && (rank[v] >> 5) == w) ? (1u << (rank[v] & 31)) : 0u;
        if (!fin) rank[v] = -1;
    }
    int n_seen = 0;
#pragma unroll
    for (int w = 0; w < 2 * CL; ++w) n_seen += __popc(wave_or_u32(seen[w]));
    if (n_seen != n_finite) return false;
#pragma unroll
    for (int v = 0; v < CL; ++v) dv[v] = __int_as_float(rank[v]);
    return true;
}

template <int CAP, int THREADS, int SPACING>
struct SmallCfg {
    static constexpr int kWaves = THREADS / 64;
    static constexpr int kBlocks = CAP / 2;
    static constexpr int kLdsRows = (kBlocks - 1) + SPACING + 1;
    static constexpr int kDistPitch = CAP + 1;
    static constexpr int kMaxLoads = (CAP * (kMaxChunk / 4) + THREADS - 1) / THREADS;   // 16-byte loads per thread and chunk
    static constexpr int kMaxRounds = (kBlocks * (kBlocks + 1) / 2 + THREADS - 1) / THREADS;  // 2x2 blocks per thread
    static_assert(CAP % 2 == 0 && CAP <= 128 && THREADS % 64 == 0 && THREADS >= CAP, "shape");
    static_assert(SPACING >= kBlocks, "LDS rows of different members must not collide");
    static_assert((CAP + kWaves - 1) / kWaves <= 32, "members of a wavefront must fit a 32-bit mask");
};

// The work of one workgroup (THREADS threads) on bucket blockIdx.x.  lds_f: the workgroup's LDS,
// small_bucket_lds_bytes<...>(pitch) bytes.  min_size: smaller buckets are left to another launch.
// stats (may be null): the workgroups whose number is a multiple of 2^stat_shift add pairs of the bucket << 32 | pairs
// whose distance is not above the last slot of one of the two rows (what the screened kernel would have to evaluate
// exactly) to one of its 8 words -- a sample of the buckets: one addition per workgroup to so few words would take
// longer than the kernel.
template <int CAP, int THREADS, int SPACING>
__device__ __forceinline__ void small_bucket_body(float* __restrict__ lds_f, const float* __restrict__ points, int D, int K,
                                                  const int* __restrict__ ids, const int* __restrict__ starts,
                                                  const int* __restrict__ sizes, int stride, int min_size,
                                                  int* __restrict__ knn_idx, float* __restrict__ knn_dist, int chunk,
                                                  int pitch, int region_floats, int rows_sorted,
                                                  unsigned long long* __restrict__ stats, int stat_shift)
{
    using Cfg = SmallCfg<CAP, THREADS, SPACING>;
    constexpr int kCap = CAP, kThreads = THREADS, kWaves = Cfg::kWaves, kSpacing = SPACING;
    constexpr int kDistPitch = Cfg::kDistPitch, kMaxLoads = Cfg::kMaxLoads;
    auto phys_row = [](int m) { return (m >> 1) + kSpacing * (m & 1); };     // LDS row of bucket member m
    // LDS: [rows | dist] (region_floats) | ids[CAP] | tau[CAP] | flag[CAP]
    float* rows = lds_f;
    float* dist = lds_f;                     // same storage, used after the last read of rows
    int* lids = reinterpret_cast<int*>(lds_f + region_floats);
    // last slot of each member's row when the rows are known to be sorted (else +inf): a member none of whose
    // candidates is below it is left alone -- its row is neither read nor written
    float* tau = reinterpret_cast<float*>(lids + kCap);
    int* flag = reinterpret_cast<int*>(tau + kCap);                    // member has such a candidate

    const int bkt = blockIdx.x;
    const int s = sizes[bkt];
    const size_t first = starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride;     // (asked for together with s)
    if (s < min_size || s > kCap) return;
    const int* bid = ids + first;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);

    // (a member's last slot is requested here and put into LDS once the first rows have been requested too: the two
    // trips to memory then overlap; nobody reads the last slots before the distances are there)
    float tau_own = INFINITY;
    if (tid < kCap) {
        const int id = tid < s ? bid[tid] : -1;
        lids[tid] = id;
        if (rows_sorted && id >= 0) tau_own = knn_dist[(size_t)id * (size_t)K + (K - 1)];
        flag[tid] = 0;
    }
    __syncthreads();

    // work assignment.  With n2 blocks of two members, the unordered block pairs (a, b) are (a, (a + o) mod n2) for
    // the offsets o = 0 .. (n2 - 1) / 2 and all a, plus o = n2 / 2 with a < n2 / 2 when n2 is even: block pair number
    // k = o n2 + a, k < n_tiles.  Thread t takes k = t, t + THREADS, ...
    constexpr int kMaxRounds = Cfg::kMaxRounds;
    const int n2 = (s + 1) >> 1;
    const int n_tiles = n2 * (((n2 - 1) >> 1) + 1) + ((n2 & 1) ? 0 : (n2 >> 1));
    const int rounds = (n_tiles + kThreads - 1) / kThreads;            // at most kMaxRounds
    const float inv_n2 = 1.0f / (float)n2;
    int tile_ab[kMaxRounds];                                           // a | b << 8, or -1
#pragma unroll
    for (int r = 0; r < kMaxRounds; ++r) {
        const int k = tid + r * kThreads;
        // k / n2 (exact: k < 1024 and (k + 0.5) / n2 is never within 1 / 128 of an integer)
        const int o = (int)(((float)k + 0.5f) * inv_n2);
        const int a = k - o * n2;
        int bb = a + o;
        if (bb >= n2) bb -= n2;
        tile_ab[r] = k < n_tiles ? (a | (bb << 8)) : -1;
    }
    float acc[kMaxRounds][4];
#pragma unroll
    for (int r = 0; r < kMaxRounds; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;

    for (int d0 = 0; d0 < D; d0 += chunk) {
        const int np = min(chunk, (D - d0 + 3) & ~3) >> 2;      // 16-byte pieces per row in this chunk
        const int items = s * np;
        // request everything, then move it to LDS
        float4 pre[kMaxLoads];
#pragma unroll
        for (int i = 0; i < kMaxLoads; ++i) {
            const int it = tid + i * kThreads;
            pre[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (it < items) {
                const int m = it / np, pc = it - m * np;
                const float* src = points + (size_t)lids[m] * (size_t)D + d0 + 4 * pc;
                if (vec_ok) {
                    pre[i] = *reinterpret_cast<const float4*>(src);
                } else {
                    const int left = D - d0 - 4 * pc;
                    pre[i].x = src[0];
                    if (left > 1) pre[i].y = src[1];
                    if (left > 2) pre[i].z = src[2];
                    if (left > 3) pre[i].w = src[3];
                }
            }
        }
        if (d0 == 0 && tid < kCap) tau[tid] = tau_own;
        if (d0 > 0) __syncthreads();                 // the previous chunk has been consumed
#pragma unroll
        for (int i = 0; i < kMaxLoads; ++i) {
            const int it = tid + i * kThreads;
            if (it < items) {
                const int m = it / np, pc = it - m * np;
                *reinterpret_cast<float4*>(&rows[phys_row(m) * pitch + 4 * pc]) = pre[i];
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kMaxRounds; ++r) {
            if (r < rounds && tile_ab[r] >= 0) {
                const float* ra = &rows[(tile_ab[r] & 255) * pitch];
                const float* rb = &rows[(tile_ab[r] >> 8) * pitch];
                for (int q = 0; q < np; ++q) {
                    float4 av[2], bv[2];
#pragma unroll
                    for (int x = 0; x < 2; ++x) av[x] = *reinterpret_cast<const float4*>(ra + kSpacing * x * pitch + 4 * q);
#pragma unroll
                    for (int y = 0; y < 2; ++y) bv[y] = *reinterpret_cast<const float4*>(rb + kSpacing * y * pitch + 4 * q);
#pragma unroll
                    for (int x = 0; x < 2; ++x)
#pragma unroll
                        for (int y = 0; y < 2; ++y) {
                            float df;
                            df = av[x].x - bv[y].x; acc[r][2 * x + y] = __builtin_fmaf(df, df, acc[r][2 * x + y]);
                            df = av[x].y - bv[y].y; acc[r][2 * x + y] = __builtin_fmaf(df, df, acc[r][2 * x + y]);
                            df = av[x].z - bv[y].z; acc[r][2 * x + y] = __builtin_fmaf(df, df, acc[r][2 * x + y]);
                            df = av[x].w - bv[y].w; acc[r][2 * x + y] = __builtin_fmaf(df, df, acc[r][2 * x + y]);
                        }
                }
            }
        }
    }
    __syncthreads();                           // rows no longer needed: the region becomes the distance matrix
    int n_pass = 0;                            // pairs of this thread that may change a row
    auto put = [&](int i, int j, float d) {
        dist[i * kDistPitch + j] = d;
        dist[j * kDistPitch + i] = d;
        if (d <= tau[i]) flag[i] = 1;            // plain stores of the same value: no ordering needed
        if (d <= tau[j]) flag[j] = 1;
        n_pass += (d <= tau[i] || d <= tau[j]) ? 1 : 0;
    };
#pragma unroll
    for (int r = 0; r < kMaxRounds; ++r) {
        if (r < rounds && tile_ab[r] >= 0) {
            const int a = tile_ab[r] & 255, bb = tile_ab[r] >> 8;
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int y = 0; y < 2; ++y) {
                    const int i = 2 * a + x, j = 2 * bb + y;
                    // a block on the diagonal holds one pair of distinct members
                    if (i < s && j < s && (a != bb || (x == 0 && y == 1))) put(i, j, acc[r][2 * x + y]);
                }
        }
    }

    if (stats && (blockIdx.x & ((1u << stat_shift) - 1u)) == 0) {
        n_pass = wave_sum_i(n_pass);
        if (lane == 0)
            atomicAdd(&stats[(blockIdx.x >> stat_shift) & 7],
                      (unsigned long long)n_pass | (wave == 0 ? (unsigned long long)(s * (s - 1) / 2) << 32 : 0ull));
    }
    __syncthreads();                           // distance matrix complete

    // top-K update: a wavefront walks its members that have a candidate, four at a time, with the rows of the
    // next four in flight (the loop is bound by the latency of these row reads otherwise)
    const int my_id = lids[lane];
    const int my_id2 = (kCap > 64 && 64 + lane < kCap) ? lids[64 + lane] : -1;      // second round of candidates
    // bit u: member wave + kWaves u has a candidate
    const int fm = wave + kWaves * lane;
    const bool has_cand = lane < 32 && fm < kCap && flag[fm < kCap ? fm : 0] != 0;
    uint32_t active = (uint32_t)ballot64(has_cand);
    auto load_row = [&](int i, int& ri, float& rd) {
        ri = -2;
        rd = INFINITY;
        if (i >= 0 && lane < K) {
            const size_t at = (size_t)lids[i] * (size_t)K + lane;
            ri = knn_idx[at];
            rd = knn_dist[at];
        }
    };
    // handle(i, ri, rd) for the members of the set, in ascending order
    auto walk = [&](uint32_t members, auto&& handle) {
        auto next_member = [&]() {
            if (members == 0) return -1;
            const int u = __ffs(members) - 1;
            members &= members - 1;
            return wave + kWaves * u;
        };
        constexpr int kAhead = 4;
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
                if (cur_i[u] < 0) break;
                handle(cur_i[u], cur_ri[u], cur_rd[u]);
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) { cur_i[u] = nxt_i[u]; cur_ri[u] = nxt_ri[u]; cur_rd[u] = nxt_rd[u]; }
        }
    };

    // Rows that are not full (last slot at +inf; every row in the first tree of a build) may hold nothing but the
    // point itself.  Such a row needs no insertions: the place of a candidate is the number of candidates below it.
    // Rows done that way leave the set; the others (and rows with two candidates at the same distance) are left to
    // the insertions below.
    const uint32_t maybe_fresh = (uint32_t)ballot64(has_cand && tau[fm < kCap ? fm : 0] == INFINITY);
    if (maybe_fresh != 0) {
        walk(maybe_fresh, [&](int i, int ri, float rd) {
            if (!fresh_row(ri, rd, lids[i], K)) return;
            const float self_d = read_lane_i(ri, 0) >= 0 ? read_lane_f(rd, 0) : INFINITY;
            constexpr int CL = kCap > 64 ? 2 : 1;
            const int j2 = 64 + lane;
            float cd[CL], place[CL];
            cd[0] = lane == i ? self_d : (lane < s ? dist[i * kDistPitch + lane] : INFINITY);
            if (CL > 1) cd[CL - 1] = j2 == i ? self_d : (j2 < s ? dist[i * kDistPitch + j2] : INFINITY);
#pragma unroll
            for (int v = 0; v < CL; ++v) place[v] = cd[v];
            if (!place_by_rank<CL>(place, s)) return;
            const size_t at = (size_t)lids[i] * (size_t)K;
            const int cv[2] = {my_id, my_id2};
#pragma unroll
            for (int v = 0; v < CL; ++v) {
                const int slot = __float_as_int(place[v]);
                if (slot >= 0 && slot < K) {
                    knn_idx[at + slot] = cv[v];
                    knn_dist[at + slot] = cd[v];
                }
            }
            active &= ~(1u << ((i - wave) / kWaves));
        });
    }

    walk(active, [&](int i, int ri, float rd) {
        const float d = dist[i * kDistPitch + lane];
        KnnRow<1> row;
        row.idx[0] = ri;
        row.dist[0] = rd;
        row.init_from_regs(K);                   // rows that arrive unsorted are rebuilt here
        if (kCap > 64) {
            const int j2 = 64 + lane;
            const float d2 = j2 < s ? dist[i * kDistPitch + j2] : INFINITY;
            const bool okv[2] = {lane < s && lane != i, j2 < s && j2 != i};
            const int cv[2] = {my_id, my_id2};
            const float dv[2] = {d, d2};
            row.template merge<2>(okv, cv, dv);
        } else {
            row.merge(lane < s && lane != i, my_id, d);
        }
        if (row.changed) {
            const size_t at = (size_t)lids[i] * (size_t)K;
            row.store(knn_idx + at, knn_dist + at);
        }
    });
}


// bytes of LDS a workgroup of small_bucket_body needs for rows of `pitch` floats (see small_bucket_shape)
template <int CAP, int THREADS, int SPACING>
inline int small_bucket_region_floats(int pitch)
{
    using Cfg = SmallCfg<CAP, THREADS, SPACING>;
    const int region = Cfg::kLdsRows * pitch > CAP * Cfg::kDistPitch ? Cfg::kLdsRows * pitch : CAP * Cfg::kDistPitch;
    return (region + 3) & ~3;
}
template <int CAP, int THREADS, int SPACING>
inline size_t small_bucket_lds_bytes(int pitch)
{
    return (size_t)small_bucket_region_floats<CAP, THREADS, SPACING>(pitch) * 4 + (size_t)(3 * CAP) * 4;
}
// dimensions staged at a time and LDS floats per row for points of D dimensions
inline void small_bucket_shape(int D, int* chunk, int* pitch)
{
    const int dpad = (D + 3) & ~3;
    *chunk = dpad < kMaxChunk ? dpad : kMaxChunk;
    *pitch = *chunk;
    if (((*pitch >> 2) & 1) == 0) *pitch += 4;              // odd number of 16-byte units
}

}  // namespace small_bucket
}  // namespace rsfk
