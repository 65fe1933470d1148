// Bucket K-NN with the pair matrix screened on the matrix cores: any bucket size,
// any K <= 256, same function and same results as the kernels in bucket_knn.hip /
// bucket_knn_small.hip (see bucket_knn.hip for the reference kernels all of them
// replace; the tile structure -- distances of a tile of the pair matrix into LDS,
// then its rows -- is that of compute_knn_from_buckets_pertile,
// src/kernels/compute_knn_from_buckets.cu:1382-1787).
//
// A pair (i, j) of a bucket changes row i only if its distance is at most the last
// slot of row i.  Once the rows are good that holds for a few per cent of the
// pairs, and the sequential fp32 chains of all the others -- the bulk of the
// arithmetic of the direct kernels -- are wasted.
//
// Decomposition.  A workgroup owns 64 members of a bucket (a "tile" of rows) and
// nothing else writes their K-NN rows: it walks over all tiles J of the bucket and
// offers their members to its own rows.  A bucket of s points is therefore worked on
// by ceil(s / 64) independent workgroups (no ordering between them, no row touched
// by two of them); every pair is looked at from both sides, which the screen makes
// cheap.  Per tile J:
//
//   1. Gram tile on the matrix cores.  The fp32 rows of both tiles are staged into
//      LDS (coalesced, up to 128 dimensions at a time, the next chunk travelling
//      while this one is used); each wavefront owns a 32 x 32 quadrant, reads its
//      operands from LDS and splits every value into two bfloat16 numbers,
//      x = hi + lo + r, |r| <= 2^-16 |x| (round to nearest twice), and accumulates
//      G = hi hi' + hi lo' + lo hi' with three v_mfma_f32_32x32x16_bf16 per 16
//      dimensions; the squared norms n of the rows are summed on the way.
//      d~ = n_i + n_j - 2 G_ij then differs from the real-number distance by at most
//      E = c S, S = n_i + n_j,
//          c = 3.1 * 2^-16 + (3.1 D' + 8) * 2^-23 + (D' + 2) * 2^-24
//      (dropped products <= 3 * 2^-16 |x||y| <= 1.5 * 2^-16 S; 3 D' exact products
//      per entry accumulated in fp32, every addition within 2^-23 of the sum of
//      absolute values whatever the order or rounding mode; norms; the two roundings
//      of the final expression), and the fp32 chain of the exact path returns at
//      least (1 - gamma) times the real-number distance, gamma = (D + 8) 2^-22.
//      A pair is dropped iff (d~ - E)(1 - gamma) > last slot of row i: its exact
//      distance is then above it, so it could not have entered the row.  NaN or
//      infinite intermediate values never drop a pair;
//   2. the pairs that are left go to a list in LDS and get the exact distance:
//      one pair per lane, sequential fused multiply-add chain over the rows in LDS
//      (the arithmetic of euclidean_distance_sqr, compute_knn_from_buckets.cu:40-54,
//      so a pair has the same distance value as in every other kernel);
//   3. the exact distances go into the tile's distance matrix in LDS (+inf elsewhere)
//      and the rows that got a candidate are merged (several K-NN rows in flight per
//      wavefront).
//
// Requires every K-NN row to be sorted on entry (the last slot is its maximum).
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"
#include "mfma_split.hpp"
#include <algorithm>

namespace rsfk {

namespace {

constexpr int kGT = 64;                       // points per tile side
constexpr int kGThreads = 256;
constexpr int kGDistPitch = kGT + 1;
constexpr int kGMaxChunk = 128;               // dimensions staged at once (a multiple of 16)
constexpr int kGBatch = 4;                    // pairs per thread between two passes over the chunks (long rows only)
constexpr int kGMeta = 6 * kGT + 4;           // ints of LDS for ids, last slots, norms, flags and the pair counter
constexpr int kGAhead = 4;                    // K-NN rows a wavefront requests together

// The rows of one tile on their way from HBM to LDS: PASSES 16-byte pieces per thread.  1 << lpr_shift lanes work on
// a row (8..32, at least the pieces of a chunk); zeros beyond D and for the rows beyond `rows`.
template <int PASSES>
struct TileLoads {
    float4 v[PASSES];

    __device__ __forceinline__ void request(const int* __restrict__ ids, int rows, const float* __restrict__ points, int D,
                                            int d0, int np4, int lpr_shift, bool vec_ok)
    {
        const int tid = threadIdx.x;
        const int piece = tid & ((1 << lpr_shift) - 1);
        const int r0 = tid >> lpr_shift;
        const int rows_per_pass = kGThreads >> lpr_shift;
        const int d = d0 + 4 * piece;
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            const int m = r0 + i * rows_per_pass;
            v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < rows && piece < np4 && d < D) {
                const float* src = points + (size_t)ids[m] * (size_t)D + d;
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

    __device__ __forceinline__ void commit(float* __restrict__ dst, int np4, int pitch, int lpr_shift) const
    {
        const int tid = threadIdx.x;
        const int piece = tid & ((1 << lpr_shift) - 1);
        const int r0 = tid >> lpr_shift;
        const int rows_per_pass = kGThreads >> lpr_shift;
        if (piece < np4) {
#pragma unroll
            for (int i = 0; i < PASSES; ++i) *reinterpret_cast<float4*>(&dst[(r0 + i * rows_per_pass) * pitch + 4 * piece]) = v[i];
        }
    }
};

// PASSES = 64 rows / (256 threads / lanes per row).  Workgroup w works on tile w % max_tiles of bucket w / max_tiles.
template <int SL, int PASSES>
__global__ __launch_bounds__(kGThreads, 2) void k_bucket_knn_gram(const float* __restrict__ points, int D, int K,
                                                                   const int* __restrict__ ids, const int* __restrict__ starts,
                                                                   const int* __restrict__ sizes, int stride, int min_size,
                                                                   int max_size, int max_tiles, int* __restrict__ knn_idx,
                                                                   float* __restrict__ knn_dist, int chunk, int pitch,
                                                                   int lpr_shift, float c_err, float one_minus_gamma)
{
    // dynamic LDS: rows of my tile | rows of tile J (launches with buckets above 64 points) | distance matrix | ids, last slots, norms of both tiles, flags |
    // pair counter | list of pairs
    extern __shared__ __align__(16) float lds_g[];
    float* rowsA = lds_g;
    float* rowsB = max_tiles > 1 ? lds_g + kGT * pitch : lds_g;      // a bucket of one tile only meets itself
    float* dist = rowsB + kGT * pitch;
    int* meta = reinterpret_cast<int*>(dist + kGT * kGDistPitch);
    int* ida = meta;
    int* idb = meta + kGT;
    float* tau_a = reinterpret_cast<float*>(meta + 2 * kGT);
    float* nrm_a = reinterpret_cast<float*>(meta + 3 * kGT);
    float* nrm_b = reinterpret_cast<float*>(meta + 4 * kGT);
    int* flag_a = meta + 5 * kGT;
    int* n_pairs = meta + 6 * kGT;
    uint16_t* list = reinterpret_cast<uint16_t*>(meta + kGMeta);

    const int bkt = blockIdx.x / max_tiles;
    const int I = blockIdx.x - bkt * max_tiles;
    const int s = sizes[bkt];
    if (s < min_size || s > max_size || I * kGT >= s) return;
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qi = wave >> 1, qj = wave & 1;             // quadrant of the tile this wavefront bounds
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int nt = (s + kGT - 1) / kGT;
    const int np4 = chunk >> 2;
    const int n_chunks = (D + chunk - 1) / chunk;
    const int rows = min(kGT, s - I * kGT);

    if (tid < kGT) {
        const int p = tid < rows ? bid[I * kGT + tid] : -1;
        ida[tid] = p;
        tau_a[tid] = p >= 0 ? knn_dist[(size_t)p * (size_t)K + (K - 1)] : 0.0f;
    }
    __syncthreads();

    TileLoads<PASSES> la, lb;
    for (int J = 0; J < nt; ++J) {
        const int cols = min(kGT, s - J * kGT);
        const bool diag = (I == J);
        if (tid < kGT) {
            idb[tid] = tid < cols ? bid[J * kGT + tid] : -1;
            flag_a[tid] = 0;
        }
        if (tid == kGT) n_pairs[0] = 0;
        __syncthreads();

        // ---- 1. Gram quadrants and norms; the next chunk travels while this one is used
        const bool active = 32 * qi < rows && 32 * qj < cols;
        f32x16 g;
#pragma unroll
        for (int i = 0; i < 16; ++i) g[i] = 0.0f;
        float na = 0.0f, nb = 0.0f;
        la.request(ida, rows, points, D, 0, np4, lpr_shift, vec_ok);
        lb.request(idb, cols, points, D, 0, np4, lpr_shift, vec_ok);
        for (int c = 0; c < n_chunks; ++c) {
            if (c > 0) __syncthreads();                  // the previous chunk has been consumed
            la.commit(rowsA, np4, pitch, lpr_shift);
            lb.commit(rowsB, np4, pitch, lpr_shift);
            __syncthreads();
            if (c + 1 < n_chunks) {
                la.request(ida, rows, points, D, (c + 1) * chunk, np4, lpr_shift, vec_ok);
                lb.request(idb, cols, points, D, (c + 1) * chunk, np4, lpr_shift, vec_ok);
            }
            if (active) {
                const float* pa = rowsA + (32 * qi + (lane & 31)) * pitch + 8 * (lane >> 5);
                const float* pb = rowsB + (32 * qj + (lane & 31)) * pitch + 8 * (lane >> 5);
                const int ksteps = min(chunk, (D - c * chunk + 15) & ~15) >> 4;
                for (int k = 0; k < ksteps; ++k) {
                    bf16x8 ah, al, bh, bl;
                    load_split(pa + 16 * k, ah, al, na);
                    load_split(pb + 16 * k, bh, bl, nb);
                    g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh, g, 0, 0, 0);
                    g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl, g, 0, 0, 0);
                    g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh, g, 0, 0, 0);
                }
            }
        }
        // a lane holds the squares of half of the dimensions of its row: add the two halves
        na += __shfl_xor(na, 32, 64);
        nb += __shfl_xor(nb, 32, 64);
        if (active && lane < 32) {                    // wavefronts that share a block write the same values
            nrm_a[32 * qi + lane] = na;
            nrm_b[32 * qj + lane] = nb;
        }
        wave_lds_sync();                              // a wavefront only reads back what it wrote itself

        // ---- 2. screen: accumulator i of lane l is pair (m, n), m = 32 qi + 8 (i / 4) + i % 4 + 4 (l / 32), n = 32 qj + l % 32
        if (active) {
            const int n = 32 * qj + (lane & 31);
            const float nn = nrm_b[n];
            const int mbase = 32 * qi + 4 * (lane >> 5);
            uint32_t bits = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int m = mbase + 8 * (i >> 2) + (i & 3);
                const float S = nrm_a[m] + nn;
                const float dt = __builtin_fmaf(-2.0f, g[i], S);
                const float lower = (dt - __builtin_fmaf(c_err, S, 1e-35f)) * one_minus_gamma;
                const bool drop = lower > tau_a[m];                           // false if anything is NaN
                const bool valid = m < rows && n < cols && !(diag && m == n);
                if (valid && !drop) bits |= 1u << i;
            }
            const int cnt = __popc(bits);
            int at = cnt ? atomicAdd(n_pairs, cnt) : 0;
            while (bits) {
                const int i = __ffs(bits) - 1;
                bits &= bits - 1;
                const int m = mbase + 8 * (i >> 2) + (i & 3);
                list[at++] = (uint16_t)(m | (n << 6));
            }
        }
        __syncthreads();
        const int n_list = n_pairs[0];
        if (n_list == 0) continue;                    // nothing in this tile can change a row of mine

        // ---- 3. exact distances of the listed pairs, straight into the tile's distance matrix (+inf elsewhere)
        for (int i = tid; i < kGT * kGDistPitch; i += kGThreads) dist[i] = INFINITY;
        auto put = [&](uint32_t e, float d) {
            const int m = (int)(e & 63u), n = (int)(e >> 6);
            dist[m * kGDistPitch + n] = d;
            if (d <= tau_a[m]) flag_a[m] = 1;            // plain stores of the same value: no ordering needed
        };
        auto chain = [&](uint32_t e, int np, float a) {
            const float* ra = rowsA + (e & 63u) * (uint32_t)pitch;
            const float* rb = rowsB + (e >> 6) * (uint32_t)pitch;
            for (int q = 0; q < np; ++q) {
                const float4 x = *reinterpret_cast<const float4*>(ra + 4 * q);
                const float4 y = *reinterpret_cast<const float4*>(rb + 4 * q);
                float df;
                df = x.x - y.x; a = __builtin_fmaf(df, df, a);
                df = x.y - y.y; a = __builtin_fmaf(df, df, a);
                df = x.z - y.z; a = __builtin_fmaf(df, df, a);
                df = x.w - y.w; a = __builtin_fmaf(df, df, a);
            }
            return a;
        };
        if (n_chunks == 1) {
            __syncthreads();                          // the matrix is cleared; the rows are still in LDS
            const int np = (D + 3) >> 2;
            for (int p = tid; p < n_list; p += kGThreads) {
                const uint32_t e = list[p];
                put(e, chain(e, np, 0.0f));
            }
        } else {
            // the rows of the first chunks are gone: they pass through LDS again, for kGBatch pairs per thread at a time
            for (int base = 0; base < n_list; base += kGBatch * kGThreads) {
                float acc[kGBatch];
                uint32_t ev[kGBatch];
#pragma unroll
                for (int k = 0; k < kGBatch; ++k) {
                    const int p = base + tid + k * kGThreads;
                    acc[k] = 0.0f;
                    ev[k] = p < n_list ? list[p] : 0u;                   // idle threads compute pair (0, 0)
                }
                la.request(ida, rows, points, D, 0, np4, lpr_shift, vec_ok);
                lb.request(idb, cols, points, D, 0, np4, lpr_shift, vec_ok);
                for (int c = 0; c < n_chunks; ++c) {
                    __syncthreads();
                    la.commit(rowsA, np4, pitch, lpr_shift);
                    lb.commit(rowsB, np4, pitch, lpr_shift);
                    __syncthreads();
                    if (c + 1 < n_chunks) {
                        la.request(ida, rows, points, D, (c + 1) * chunk, np4, lpr_shift, vec_ok);
                        lb.request(idb, cols, points, D, (c + 1) * chunk, np4, lpr_shift, vec_ok);
                    }
                    const int np = min(chunk, (D - c * chunk + 3) & ~3) >> 2;
#pragma unroll
                    for (int k = 0; k < kGBatch; ++k)
                        if (base + k * kGThreads < n_list) acc[k] = chain(ev[k], np, acc[k]);
                }
#pragma unroll
                for (int k = 0; k < kGBatch; ++k)
                    if (base + tid + k * kGThreads < n_list) put(ev[k], acc[k]);
            }
        }
        __syncthreads();

        // ---- 4. my rows take the members of tile J as candidates: a wavefront walks its members that have a candidate,
        //         the K-NN rows of up to kGAhead of them in flight
        {
            const int fm = wave + 4 * lane;                       // bit u of the mask: member wave + 4 u
            uint32_t todo = (uint32_t)ballot64(lane < 16 && fm < rows && flag_a[fm < kGT ? fm : 0] != 0);
            const int cand_id = idb[lane];
            while (todo != 0) {
                int mem[kGAhead];
                int ri[kGAhead][SL];
                float rd[kGAhead][SL];
#pragma unroll
                for (int u = 0; u < kGAhead; ++u) {
                    mem[u] = -1;
                    if (todo != 0) {
                        mem[u] = wave + 4 * (__ffs(todo) - 1);
                        todo &= todo - 1;
                    }
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) {
                        const int k = lane + 64 * sl;
                        ri[u][sl] = -2;
                        rd[u][sl] = INFINITY;
                        if (mem[u] >= 0 && k < K) {
                            const size_t at = (size_t)ida[mem[u]] * (size_t)K + k;
                            ri[u][sl] = knn_idx[at];
                            rd[u][sl] = knn_dist[at];
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < kGAhead; ++u) {
                    const int ci = mem[u];
                    if (ci < 0) break;
                    KnnRow<SL> row;
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) { row.idx[sl] = ri[u][sl]; row.dist[sl] = rd[u][sl]; }
                    row.init_sorted(K);
                    const bool ok = lane < cols && !(diag && lane == ci);
                    row.merge(ok, cand_id, dist[ci * kGDistPitch + lane]);
                    if (row.changed) {
                        const size_t at = (size_t)ida[ci] * (size_t)K;
                        row.store(knn_idx + at, knn_dist + at);
                        if (lane == 0) tau_a[ci] = row.tau;           // only this wavefront reads it again (next tile)
                    }
                }
            }
        }
        __syncthreads();                              // the next tile reuses the LDS
    }
}

template <int SL, int PASSES>
int launch_gram_cfg(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes, int n_buckets,
                    int stride, int min_size, int max_size, int max_tiles, int* knn_idx, float* knn_dist, int chunk, int pitch,
                    int lpr_shift, float c_err, float one_minus_gamma, size_t lds, hipStream_t stream)
{
    auto kern = k_bucket_knn_gram<SL, PASSES>;
    RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3((unsigned)n_buckets * (unsigned)max_tiles), dim3(kGThreads), lds, stream, points, D, K, ids,
                       starts, sizes, stride, min_size, max_size, max_tiles, knn_idx, knn_dist, chunk, pitch, lpr_shift, c_err,
                       one_minus_gamma);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace

// Buckets of min_size..max_size points (others are skipped); every K-NN row sorted on entry.  max_size bounds the
// grid (a workgroup per 64 members of the largest bucket, for every bucket), so it should be the real maximum.
int launch_bucket_knn_gram(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                           int n_buckets, int stride, int min_size, int max_size, int* knn_idx, float* knn_dist,
                           hipStream_t stream)
{
    if (n_buckets <= 0 || max_size < 2) return 0;
    const int max_tiles = (max_size + kGT - 1) / kGT;
    RSFK_CHECK((long long)n_buckets * max_tiles < (1ll << 31), "screened bucket kernel: too many workgroups");
    RSFK_CHECK(K >= 1 && K <= 256 && D >= 1, "screened bucket kernel: K must be in 1..256 and D positive");
    min_size = std::max(min_size, 2);
    const int d16 = (D + 15) & ~15;
    const int chunk = std::min(d16, kGMaxChunk);
    int pitch = chunk + 4;
    if (((pitch >> 2) & 1) == 0) pitch += 4;              // odd number of 16-byte units: rows start in different banks
    int lpr_shift = 3;
    while ((1 << lpr_shift) < (chunk >> 2)) ++lpr_shift;  // lanes per row while staging: 8, 16 or 32
    const size_t lds = (size_t)(max_tiles > 1 ? 2 : 1) * kGT * pitch * 4 + (size_t)kGT * kGDistPitch * 4 + (size_t)kGMeta * 4 +
                       (size_t)kGT * kGT * 2;
    const float c_err = split_gram_error_coefficient(d16);
    const float one_minus_gamma = 1.0f - (float)(D + 8) * (1.0f / 4194304.0f);
    RSFK_CHECK(one_minus_gamma > 0.5f, "screened bucket kernel: D too large");
#define RSFK_GRAM_CASE(SLV, PV)                                                                                            \
    return launch_gram_cfg<SLV, PV>(points, D, K, ids, starts, sizes, n_buckets, stride, min_size, max_size, max_tiles,   \
                                    knn_idx, knn_dist, chunk, pitch, lpr_shift, c_err, one_minus_gamma, lds, stream)
    const int passes = (kGT << lpr_shift) / kGThreads;    // 2, 4 or 8
    if (K <= 64) {
        if (passes == 2) RSFK_GRAM_CASE(1, 2);
        if (passes == 4) RSFK_GRAM_CASE(1, 4);
        RSFK_GRAM_CASE(1, 8);
    } else if (K <= 128) {
        if (passes == 2) RSFK_GRAM_CASE(2, 2);
        if (passes == 4) RSFK_GRAM_CASE(2, 4);
        RSFK_GRAM_CASE(2, 8);
    } else {
        if (passes == 2) RSFK_GRAM_CASE(4, 2);
        if (passes == 4) RSFK_GRAM_CASE(4, 4);
        RSFK_GRAM_CASE(4, 8);
    }
#undef RSFK_GRAM_CASE
}

}  // namespace rsfk
