// Bucket K-NN for buckets whose points fit into LDS whole (low-dimensional points,
// buckets of up to 256): same function and same results as the general kernel in
// bucket_knn.hip (see there for the reference kernels all of them replace), K <= 64.
//
// The tiled kernel looks at a bucket of s points as ceil(s / 64)^2 / 2 tiles of the
// pair matrix and visits the K-NN row of a point once per tile it takes part in:
// with buckets of 64..256 points a row is read, merged into and written about three
// times per tree, and with few trees over many points nearly every visit changes it.
// Here a row is touched once:
//
//   1. the fp32 rows of the whole bucket are staged into LDS (coalesced 16-byte
//      pieces; pitch an odd number of 16-byte units);
//   2. a wavefront takes two members at a time.  Lane l runs the sequential fused
//      multiply-add chains (arithmetic of euclidean_distance_sqr,
//      compute_knn_from_buckets.cu:40-54: a pair has the same distance value as in every
//      other kernel) of candidates l, 64 + l, ... against both members: the
//      candidate's values are read from LDS once for the two, the members' values are
//      the same in all lanes (broadcast reads).  Every pair is computed from both
//      ends, which at these dimensions costs less than carrying a distance matrix
//      through LDS and a second visit of the rows;
//   3. all candidates of a member are then offered to its row (knn_list.hpp), held
//      in registers, and the row is stored if it changed.  When far more candidates
//      are below the row's last slot than the row has slots, a histogram of their
//      distances first removes those that cannot stay, and into a row that is new
//      the rest is written by rank (counted, not inserted).  The K-NN rows of the
//      next two members are requested before the chains of these two start.
//
// No distance matrix, no flags, no barrier after the staging; a row is owned by
// one wavefront (no locks).
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"
#include "bucket_small_body.hpp"
#include <algorithm>

namespace rsfk {

namespace {

constexpr int kRowsThreads = 256;
constexpr int kRowsWaves = kRowsThreads / 64;
constexpr int kRowsStep = 32;                 // dimensions of the two members held in registers at a time
constexpr int kRowsLdsBytes = 40 * 1024;      // four workgroups per compute unit

// NT = tiles of 64 candidates: buckets of up to 64 NT points.  Buckets outside min_size..max_size are left alone.
// DENSE: with the histogram step for members most of whose candidates are below the last slot (the first trees of a
// build; the code costs the later ones a few per cent when it is merely present).
template <int NT, bool DENSE>
__global__ __launch_bounds__(kRowsThreads) void k_bucket_knn_rows(const float* __restrict__ points, int D, int K,
                                                                   const int* __restrict__ ids, const int* __restrict__ starts,
                                                                   const int* __restrict__ sizes, int stride, int min_size,
                                                                   int max_size, int* __restrict__ knn_idx,
                                                                   float* __restrict__ knn_dist, int pitch, int rows_sorted)
{
    extern __shared__ __align__(16) float lds_r[];
    float* rows = lds_r;                                          // 64 NT rows of `pitch` floats
    int* lids = reinterpret_cast<int*>(lds_r + 64 * NT * pitch);
    int* hist = lids + 64 * NT + 192 * (threadIdx.x >> 6);        // this wavefront's histogram, then 64 distances and 64 ids

    const int bkt = blockIdx.x;
    const int s = sizes[bkt];
    if (s < min_size || s > max_size || s < 2) return;
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int np = (D + 3) >> 2;                                  // 16-byte pieces per row

    for (int i = tid; i < 64 * NT; i += kRowsThreads) lids[i] = i < s ? bid[i] : -1;
    __syncthreads();
    // rows beyond s stay as they are: their distances are never offered
    for (int it = tid; it < s * np; it += kRowsThreads) {
        const int m = it / np, pc = it - m * np;
        const float* src = points + (size_t)lids[m] * (size_t)D + 4 * pc;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (vec_ok) {
            v = *reinterpret_cast<const float4*>(src);
        } else {
            const int left = D - 4 * pc;
            v.x = src[0];
            if (left > 1) v.y = src[1];
            if (left > 2) v.z = src[2];
            if (left > 3) v.w = src[3];
        }
        *reinterpret_cast<float4*>(&rows[m * pitch + 4 * pc]) = v;
    }
    __syncthreads();

    const int nt = (s + 63) >> 6;
    int cid[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) cid[t] = lids[64 * t + lane];

    auto load_row = [&](int m, int& ri, float& rd) {
        ri = -2;
        rd = INFINITY;
        if (m < s && lane < K) {
            const size_t at = (size_t)lids[m] * (size_t)K + lane;
            ri = knn_idx[at];
            rd = knn_dist[at];
        }
    };
    auto finish = [&](int m, int ri, float rd, const float (&acc)[NT]) {
        KnnRow<1> row;
        row.idx[0] = ri;
        row.dist[0] = rd;
        if (rows_sorted) row.init_sorted(K);
        else row.init_from_regs(K);                               // rows that arrive unsorted are rebuilt here
        bool ok[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) ok[t] = t < nt && cid[t] >= 0 && 64 * t + lane != m;
        // the first 64 candidates tell whether most candidates are below the row's last slot
        // (the histogram below only ever sees candidates that passed enters(): a NaN distance would otherwise land in
        // its first interval and push finite candidates out)
        int n_ok = DENSE ? __popcll(ballot64(ok[0] && row.enters(cid[0], acc[0]))) : 0;
        if (DENSE && n_ok > min(40, K + 16)) {
            n_ok = 0;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                ok[t] = ok[t] && row.enters(cid[t], acc[t]);
                n_ok += __popcll(ballot64(ok[t]));
            }
        }
        if (DENSE && n_ok > K + 16) {
            // Many more candidates below the last slot than the row has slots (rows that are new or far from done):
            // inserting them one after the other would push most of them out again.  A histogram of their distances
            // over 64 equal intervals tells in which interval the K-th smallest lies; a candidate in a later interval
            // has K candidates below it and cannot stay in the row, so it is not inserted at all.
            float lo = INFINITY, hi = 0.0f;
#pragma unroll
            for (int t = 0; t < NT; ++t)
                if (ok[t]) { lo = fminf(lo, acc[t]); hi = fmaxf(hi, acc[t]); }
            lo = -wave_max(-lo);
            hi = wave_max(hi);
            if (hi > lo) {
                const float scale = 63.5f / (hi - lo);
                wave_lds_sync();
                hist[lane] = 0;
                wave_lds_sync();
                int bin[NT];
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    bin[t] = min(63, max(0, (int)((acc[t] - lo) * scale)));       // does not decrease when the distance grows
                    if (ok[t]) atomicAdd(&hist[bin[t]], 1);
                }
                wave_lds_sync();
                const int h = hist[lane];
                const int upto = wave_excl_scan_i(h) + h;
                const int cross = first_lane(ballot64(upto >= K));
#pragma unroll
                for (int t = 0; t < NT; ++t) ok[t] = ok[t] && bin[t] <= cross;
            }
        }
        if (DENSE && n_ok > 0 && small_bucket::fresh_row(ri, rd, lids[m], K)) {
            // A new row (nothing in it but, possibly, the point itself): the candidates that are left are not inserted
            // one after the other -- their places in the row are their ranks among themselves.  They are gathered in
            // lanes 0.. (through LDS), ranked by counting, and stored where they belong.
            const bool has_self = read_lane_i(ri, 0) >= 0;
            int n_left = has_self ? 1 : 0;
#pragma unroll
            for (int t = 0; t < NT; ++t) n_left += __popcll(ballot64(ok[t] && row.enters(cid[t], acc[t])));
            if (n_left <= 64) {
                float* cd = reinterpret_cast<float*>(hist + 64);
                int* ci = hist + 128;
                wave_lds_sync();
                int at = 0;
                if (has_self) {
                    if (lane == 0) { cd[0] = rd; ci[0] = ri; }
                    at = 1;
                }
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const bool in = ok[t] && row.enters(cid[t], acc[t]);
                    const uint64_t mk = ballot64(in);
                    if (in) {
                        const int p = at + mask_prefix(mk);
                        cd[p] = acc[t];
                        ci[p] = cid[t];
                    }
                    at += __popcll(mk);
                }
                wave_lds_sync();
                const float d = lane < n_left ? cd[lane] : INFINITY;
                const int c = lane < n_left ? ci[lane] : -1;
                float place[1] = {d};
                if (small_bucket::place_by_rank<1>(place, n_left)) {          // (not with equal distances: those take the usual way)
                    const int slot = __float_as_int(place[0]);
                    if (slot >= 0 && slot < K) {
                        const size_t to = (size_t)lids[m] * (size_t)K + slot;
                        knn_idx[to] = c;
                        knn_dist[to] = d;
                    }
                    return;
                }
            }
        }
        // tile after tile: the last slot a tile leaves behind already turns away candidates of the next
#pragma unroll
        for (int t = 0; t < NT; ++t)
            if (t < nt) row.merge(ok[t], cid[t], acc[t]);
        if (row.changed) {
            const size_t at = (size_t)lids[m] * (size_t)K;
            row.store(knn_idx + at, knn_dist + at);
        }
    };

    // members wave, wave + 4 (a pair), wave + 8, wave + 12 (the next pair), ...
    int ri0, ri1, nri0, nri1;
    float rd0, rd1, nrd0, nrd1;
    load_row(wave, ri0, rd0);
    load_row(wave + kRowsWaves, ri1, rd1);
    for (int m0 = wave; m0 < s; m0 += 2 * kRowsWaves) {
        const int m1 = m0 + kRowsWaves;
        load_row(m0 + 2 * kRowsWaves, nri0, nrd0);
        load_row(m1 + 2 * kRowsWaves, nri1, nrd1);
        const bool two = m1 < s;
        const float* r0 = rows + m0 * pitch;
        const float* r1 = rows + (two ? m1 : m0) * pitch;
        float acc0[NT], acc1[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) { acc0[t] = 0.0f; acc1[t] = 0.0f; }
        for (int d0 = 0; d0 < 4 * np; d0 += kRowsStep) {
            const int nq = min(kRowsStep / 4, np - (d0 >> 2));
            float4 x0[kRowsStep / 4], x1[kRowsStep / 4];
#pragma unroll
            for (int q = 0; q < kRowsStep / 4; ++q) {
                if (q < nq) {
                    x0[q] = *reinterpret_cast<const float4*>(r0 + d0 + 4 * q);
                    x1[q] = *reinterpret_cast<const float4*>(r1 + d0 + 4 * q);
                }
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (t < nt) {
                    const float* rc = rows + (64 * t + lane) * pitch + d0;
                    float a0 = acc0[t], a1 = acc1[t];
#pragma unroll
                    for (int q = 0; q < kRowsStep / 4; ++q) {
                        if (q < nq) {
                            const float4 v = *reinterpret_cast<const float4*>(rc + 4 * q);
                            float df;
                            df = x0[q].x - v.x; a0 = __builtin_fmaf(df, df, a0);
                            df = x0[q].y - v.y; a0 = __builtin_fmaf(df, df, a0);
                            df = x0[q].z - v.z; a0 = __builtin_fmaf(df, df, a0);
                            df = x0[q].w - v.w; a0 = __builtin_fmaf(df, df, a0);
                            df = x1[q].x - v.x; a1 = __builtin_fmaf(df, df, a1);
                            df = x1[q].y - v.y; a1 = __builtin_fmaf(df, df, a1);
                            df = x1[q].z - v.z; a1 = __builtin_fmaf(df, df, a1);
                            df = x1[q].w - v.w; a1 = __builtin_fmaf(df, df, a1);
                        }
                    }
                    acc0[t] = a0;
                    acc1[t] = a1;
                }
            }
        }
        finish(m0, ri0, rd0, acc0);
        if (two) finish(m1, ri1, rd1, acc1);
        ri0 = nri0; rd0 = nrd0;
        ri1 = nri1; rd1 = nrd1;
    }
}

template <int NT, bool DENSE>
int launch_rows_cfg(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes, int n_buckets,
                    int stride, int min_size, int max_size, int* knn_idx, float* knn_dist, int pitch, bool rows_sorted,
                    hipStream_t stream)
{
    const size_t lds = (size_t)64 * NT * pitch * sizeof(float) + (size_t)64 * (NT + 3 * kRowsWaves) * sizeof(int);
    auto kern = k_bucket_knn_rows<NT, DENSE>;
    RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3((unsigned)n_buckets), dim3(kRowsThreads), lds, stream, points, D, K, ids, starts, sizes, stride,
                       min_size, max_size, knn_idx, knn_dist, pitch, rows_sorted ? 1 : 0);
    RSFK_HIP(hipGetLastError());
    return 0;
}

int rows_pitch(int D)
{
    int pitch = (D + 3) & ~3;
    if (((pitch >> 2) & 1) == 0) pitch += 4;              // odd number of 16-byte units: rows start in different banks
    return pitch;
}

}  // namespace

// Largest bucket the kernel takes for points of D dimensions and rows of K neighbours (0: none).
int bucket_rows_cap(int D, int K)
{
    if (K > 64) return 0;
    const int per_point = rows_pitch(D) * (int)sizeof(float) + (int)sizeof(int);
    const int tiles = std::min(4, (kRowsLdsBytes - 3 * 64 * kRowsWaves * (int)sizeof(int)) / (64 * per_point));
    return 64 * tiles;
}

// Buckets of min_size..max_size points (others are skipped); max_size <= bucket_rows_cap(D, K).  young_rows: the rows
// may be new or far from done (the first trees of a build, or unknown).
int launch_bucket_knn_rows(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes, int n_buckets,
                           int stride, int min_size, int max_size, bool rows_sorted, bool young_rows, int* knn_idx,
                           float* knn_dist, hipStream_t stream)
{
    if (n_buckets <= 0 || max_size < 2) return 0;
    RSFK_CHECK(K >= 1 && K <= 64 && D >= 1, "bucket kernel with resident rows: K must be in 1..64 and D positive");
    RSFK_CHECK(max_size <= bucket_rows_cap(D, K), "bucket kernel with resident rows: buckets too large for the LDS");
    const int pitch = rows_pitch(D);
    const int tiles = (max_size + 63) / 64;
#define RSFK_ROWS_CASE(NTV, DV)                                                                                             \
    return launch_rows_cfg<NTV, DV>(points, D, K, ids, starts, sizes, n_buckets, stride, min_size, max_size, knn_idx, knn_dist, \
                                    pitch, rows_sorted, stream)
    if (young_rows) {
        if (tiles <= 2) RSFK_ROWS_CASE(2, true);
        if (tiles == 3) RSFK_ROWS_CASE(3, true);
        RSFK_ROWS_CASE(4, true);
    }
    if (tiles <= 2) RSFK_ROWS_CASE(2, false);
    if (tiles == 3) RSFK_ROWS_CASE(3, false);
    RSFK_ROWS_CASE(4, false);
#undef RSFK_ROWS_CASE
}

}  // namespace rsfk
