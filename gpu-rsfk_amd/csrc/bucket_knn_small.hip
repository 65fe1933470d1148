// Bucket K-NN for buckets of at most 64 points and K <= 64: the shape the
// default parameters (bucket size K+1 .. 2(K+1), K <= 32) produce.  Same function
// as the general kernel in bucket_knn.hip (see there for the reference kernels it
// replaces); two wavefronts per bucket.
//
//   1. the rows of the bucket, 64 dimensions at a time, are requested from HBM at
//      once and written to LDS; a row is read by consecutive lanes, 16 bytes each
//      (coalesced);
//   2. each thread owns one 4x4 block of the upper triangle of the pair matrix and
//      accumulates its 16 distances with sequential fused multiply-add chains
//      (arithmetic of euclidean_distance_sqr, compute_knn_from_buckets.cu:40-54);
//      the 6 pairs inside each diagonal block are done one per thread;
//   3. the distance matrix replaces the rows in LDS; a wavefront owns every second
//      point: per point, the candidates that are closer than the row's last slot
//      are inserted into the sorted row unless the row holds them already
//      (knn_list.hpp); the rows of the next two points are in flight meanwhile.
// Registers are kept near 100 and LDS near 20 KB per workgroup so that four
// wavefronts per SIMD are resident: the kernel alternates between an arithmetic
// phase and a latency-bound merge phase, and only other resident workgroups can
// fill the gaps.
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"

namespace rsfk {

namespace {

constexpr int kCap = kBucketSplit;          // largest bucket this kernel takes
static_assert(kCap == 64, "lane-per-candidate merge and 64-bit presence masks assume 64");
constexpr int kThreads = 128;
constexpr int kWaves = kThreads / 64;
constexpr int kSpacing = 17;                // LDS rows between members 4t, 4t+1, 4t+2, 4t+3
constexpr int kLdsRows = 15 + 3 * kSpacing + 1;
constexpr int kDistPitch = kCap + 1;
constexpr int kMaxChunk = 64;               // dimensions staged at once
constexpr int kMaxLoads = kCap * (kMaxChunk / 4) / kThreads;   // 16-byte loads per thread and chunk

// LDS row of bucket member m: the 4x4 block of thread t reads rows t, t+17, t+34,
// t+51 -- consecutive t give conflict-free 16-byte reads (the pitch is an odd
// number of 16-byte units) and the four rows of one block fall in different banks.
__device__ __forceinline__ int phys_row(int m) { return (m >> 2) + kSpacing * (m & 3); }

__global__ __launch_bounds__(kThreads, 4) void k_bucket_knn_small(const float* __restrict__ points, int D, int K,
                                                                  const int* __restrict__ ids,
                                                                  const int* __restrict__ starts,
                                                                  const int* __restrict__ sizes, int stride,
                                                                  int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                                  int chunk, int pitch, int region_floats, int rows_sorted)
{
    // dynamic LDS: [rows | dist] (region_floats) | ids[64] | tau[64] | flag[64]
    extern __shared__ __align__(16) float lds_f[];
    float* rows = lds_f;
    float* dist = lds_f;                     // same storage, used after the last read of rows
    int* lids = reinterpret_cast<int*>(lds_f + region_floats);
    // last slot of each member's row when the rows are known to be sorted (else +inf): a member none of whose
    // candidates is below it is left alone -- its row is neither read nor written
    float* tau = reinterpret_cast<float*>(lids + kCap);
    int* flag = reinterpret_cast<int*>(tau + kCap);                    // member has such a candidate

    const int bkt = blockIdx.x;
    const int s = sizes[bkt];
    if (s < 2 || s > kCap) return;
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);

    if (tid < kCap) {
        const int id = tid < s ? bid[tid] : -1;
        lids[tid] = id;
        tau[tid] = (rows_sorted && id >= 0) ? knn_dist[(size_t)id * (size_t)K + (K - 1)] : INFINITY;
        flag[tid] = 0;
    }
    __syncthreads();

    // work assignment: off-diagonal 4x4 blocks (ti < tj) one per thread, then the 6 pairs of each diagonal block
    const int n = (s + 3) >> 2;
    const int noff = n * (n - 1) / 2;
    int ti = 0, tj = 0;
    const bool has_tile = tid < noff;
    if (has_tile) {
        int rem = tid;
        while (rem >= n - 1 - ti) { rem -= n - 1 - ti; ++ti; }
        tj = ti + 1 + rem;
    }
    const bool has_diag = tid < 6 * n;
    const int dt = tid / 6, dq = tid - 6 * dt;
    const int dr = dq < 3 ? 0 : (dq < 5 ? 1 : 2);
    const int dc = dq < 3 ? dq + 1 : (dq < 5 ? dq - 1 : 3);

    float acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
    float dacc = 0.0f;

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
        if (has_tile) {
            const float* ra = &rows[ti * pitch];
            const float* rb = &rows[tj * pitch];
            for (int q = 0; q < np; ++q) {
                float4 av[4], bv[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) av[r] = *reinterpret_cast<const float4*>(ra + kSpacing * r * pitch + 4 * q);
#pragma unroll
                for (int c = 0; c < 4; ++c) bv[c] = *reinterpret_cast<const float4*>(rb + kSpacing * c * pitch + 4 * q);
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float df;
                        df = av[r].x - bv[c].x; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                        df = av[r].y - bv[c].y; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                        df = av[r].z - bv[c].z; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                        df = av[r].w - bv[c].w; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                    }
            }
        }
        if (has_diag) {
            const float* ra = &rows[(dt + kSpacing * dr) * pitch];
            const float* rb = &rows[(dt + kSpacing * dc) * pitch];
            for (int q = 0; q < np; ++q) {
                const float4 a = *reinterpret_cast<const float4*>(ra + 4 * q);
                const float4 b = *reinterpret_cast<const float4*>(rb + 4 * q);
                float df;
                df = a.x - b.x; dacc = __builtin_fmaf(df, df, dacc);
                df = a.y - b.y; dacc = __builtin_fmaf(df, df, dacc);
                df = a.z - b.z; dacc = __builtin_fmaf(df, df, dacc);
                df = a.w - b.w; dacc = __builtin_fmaf(df, df, dacc);
            }
        }
    }
    __syncthreads();                           // rows no longer needed: the region becomes the distance matrix
    auto put = [&](int i, int j, float d) {
        dist[i * kDistPitch + j] = d;
        dist[j * kDistPitch + i] = d;
        if (d < tau[i]) flag[i] = 1;             // plain stores of the same value: no ordering needed
        if (d < tau[j]) flag[j] = 1;
    };
    if (has_tile) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int i = 4 * ti + r, j = 4 * tj + c;
                if (i < s && j < s) put(i, j, acc[r][c]);
            }
    }
    if (has_diag) {
        const int i = 4 * dt + dr, j = 4 * dt + dc;
        if (j < s) put(i, j, dacc);
    }

    __syncthreads();                           // distance matrix complete

    // top-K update: a wavefront walks its members that have a candidate, four at a time, with the rows of the
    // next four in flight (the loop is bound by the latency of these row reads otherwise)
    const int my_id = lids[lane];
    // bit u: member wave + 2 u has a candidate
    uint32_t active = (uint32_t)ballot64(lane < 32 && flag[(wave + kWaves * lane) & (kCap - 1)] != 0);
    auto next_member = [&]() {
        if (active == 0) return -1;
        const int u = __ffs(active) - 1;
        active &= active - 1;
        return wave + kWaves * u;
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
            const int i = cur_i[u];
            if (i < 0) break;
            const float d = dist[i * kDistPitch + lane];
            KnnRow<1> row;
            row.idx[0] = cur_ri[u];
            row.dist[0] = cur_rd[u];
            row.init_from_regs(K);                   // rows that arrive unsorted are rebuilt here
            row.offer_lanes<true>(lane < s && lane != i, my_id, d);
            if (row.changed) {
                const size_t at = (size_t)lids[i] * (size_t)K;
                row.store(knn_idx + at, knn_dist + at);
            }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) { cur_i[u] = nxt_i[u]; cur_ri[u] = nxt_ri[u]; cur_rd[u] = nxt_rd[u]; }
    }
}

}  // namespace

int small_bucket_cap() { return kCap; }

// rows_sorted: every K-NN row is known to be sorted by distance (then members without a candidate below their
// last slot are skipped)
int launch_bucket_knn_small(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                            int n_buckets, int stride, bool rows_sorted, int* knn_idx, float* knn_dist, hipStream_t stream)
{
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 64, "small-bucket kernel: K must be in 1..64");
    const int dpad = (D + 3) & ~3;
    const int chunk = dpad < kMaxChunk ? dpad : kMaxChunk;
    int pitch = chunk;
    if (((pitch >> 2) & 1) == 0) pitch += 4;              // odd number of 16-byte units
    const int region = std::max(kLdsRows * pitch, kCap * kDistPitch);
    const int region_floats = (region + 3) & ~3;
    const size_t lds = (size_t)region_floats * 4 + (size_t)(3 * kCap) * 4;
    RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_bucket_knn_small),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(k_bucket_knn_small, dim3((unsigned)n_buckets), dim3(kThreads), lds, stream, points, D, K, ids,
                       starts, sizes, stride, knn_idx, knn_dist, chunk, pitch, region_floats, rows_sorted ? 1 : 0);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
