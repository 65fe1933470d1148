// Bucket K-NN: for every leaf bucket, all-pairs squared distances and the
// per-point top-K update.
//
// Replaces the reference's bucket kernels (the function they all compute is
// the same): compute_knn_from_buckets_predist_nolock ("diagonal",
// src/kernels/compute_knn_from_buckets.cu:998-1378), ..._pertile (:1382-1787)
// and ..._perblock_coalesced_symmetric_dividek (:547-814).
//
// Common to both kernels here:
//   * every pair of a bucket is computed once (symmetric schedule);
//   * point rows are gathered from HBM with coalesced 128-byte segments into
//     LDS, 32 dimensions at a time;
//   * each thread accumulates a 4x4 block of pair distances in registers with a
//     sequential fused multiply-add chain per pair (the arithmetic of
//     euclidean_distance_sqr, compute_knn_from_buckets.cu:40-54);
//   * the distances go to LDS and one wavefront per point merges them into the
//     point's K-NN row, held in registers with K divided over the lanes.  A row
//     is owned by one wavefront at a time, so there are no locks.
//
// k_bucket_knn_small : buckets of at most 64 points, K <= 64 (the shape the
//     default parameters produce).  Two wavefronts per bucket; the 4x4 blocks
//     cover only the upper triangle; the K-NN rows of the bucket are loaded into
//     registers before the distance phase so that their latency is hidden; ids
//     already present in a row are found through a hash table of the bucket in
//     LDS instead of a scan per candidate.
// k_bucket_knn       : any bucket size, any K <= 256, 64x64 tiles of the pair
//     matrix, rows and columns of a tile updated in turn.
#include "rsfk_common.hpp"
#include "knn_list.hpp"

namespace rsfk {

constexpr int kTile = 64;          // points per tile side
constexpr int kDC = 32;            // dimensions staged per step
constexpr int kDCP = kDC + 4;      // LDS row pitch in floats: 9 x 16 B, odd => conflict-free b128 reads
constexpr int kDistPitch = kTile + 1;

// ---------------------------------------------------------------------------
// general kernel
// ---------------------------------------------------------------------------
struct BucketKnnLds {
    float a[kTile * kDCP];
    float b[kTile * kDCP];
    float dist[kTile * kDistPitch];
    int ida[kTile];
    int idb[kTile];
};

// Stage rows ids[0..rows) x dims [d0, d0+32) into dst (zero filled outside).
__device__ __forceinline__ void stage_rows(float* __restrict__ dst, const int* __restrict__ ids, int rows,
                                           const float* __restrict__ points, int D, int d0, bool vec_ok)
{
    const int t = threadIdx.x;
    const int r = t >> 2;            // 0..63
    const int seg = (t & 3) * 8;     // 0,8,16,24
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    if (r < rows) {
        const float* src = points + (size_t)ids[r] * (size_t)D + d0 + seg;
        const int left = D - d0 - seg;
        if (vec_ok && left >= 8) {
            const float4 q0 = *reinterpret_cast<const float4*>(src);
            const float4 q1 = *reinterpret_cast<const float4*>(src + 4);
            v[0] = q0.x; v[1] = q0.y; v[2] = q0.z; v[3] = q0.w;
            v[4] = q1.x; v[5] = q1.y; v[6] = q1.z; v[7] = q1.w;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) if (e < left) v[e] = src[e];
        }
    }
    float4* d4 = reinterpret_cast<float4*>(dst + r * kDCP + seg);
    d4[0] = make_float4(v[0], v[1], v[2], v[3]);
    d4[1] = make_float4(v[4], v[5], v[6], v[7]);
}

template <int SL>
__global__ __launch_bounds__(256) void k_bucket_knn(const float* __restrict__ points, int D, int K,
                                                     const int* __restrict__ ids, const int* __restrict__ starts,
                                                     const int* __restrict__ sizes, int stride, int skip_upto,
                                                     int* __restrict__ knn_idx, float* __restrict__ knn_dist)
{
    __shared__ BucketKnnLds L;
    const int bkt = blockIdx.x;
    const int s = sizes[bkt];
    if (s < 2 || s <= skip_upto) return;
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ty = tid >> 4, tx = tid & 15;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int nt = (s + kTile - 1) / kTile;

    for (int I = 0; I < nt; ++I) {
        const int rows = min(kTile, s - I * kTile);
        for (int J = I; J < nt; ++J) {
            const int cols = min(kTile, s - J * kTile);
            const bool diag = (I == J);
            __syncthreads();   // previous tile's LDS fully consumed
            if (tid < kTile) {
                L.ida[tid] = tid < rows ? bid[I * kTile + tid] : -1;
                L.idb[tid] = tid < cols ? bid[J * kTile + tid] : -1;
            }
            const int nrb = (rows + 15) >> 4, ncb = (cols + 15) >> 4;
            float acc[4][4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
            __syncthreads();
            for (int d0 = 0; d0 < D; d0 += kDC) {
                stage_rows(L.a, L.ida, rows, points, D, d0, vec_ok);
                if (!diag) stage_rows(L.b, L.idb, cols, points, D, d0, vec_ok);
                __syncthreads();
                const float* B = diag ? L.a : L.b;
#pragma unroll 2
                for (int dd = 0; dd < kDC; dd += 4) {
                    float4 av[4], bv[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) av[r] = *reinterpret_cast<const float4*>(&L.a[(ty + 16 * r) * kDCP + dd]);
#pragma unroll
                    for (int c = 0; c < 4; ++c) bv[c] = *reinterpret_cast<const float4*>(&B[(tx + 16 * c) * kDCP + dd]);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (r >= nrb) continue;
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            if (c >= ncb || (diag && c < r)) continue;
                            float df;
                            df = av[r].x - bv[c].x; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                            df = av[r].y - bv[c].y; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                            df = av[r].z - bv[c].z; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                            df = av[r].w - bv[c].w; acc[r][c] = __builtin_fmaf(df, df, acc[r][c]);
                        }
                    }
                }
                __syncthreads();
            }
            // distances of the tile -> LDS (mirror the strictly-upper blocks of a diagonal tile)
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (r >= nrb || c >= ncb || (diag && c < r)) continue;
                    const int i = ty + 16 * r, j = tx + 16 * c;
                    L.dist[i * kDistPitch + j] = acc[r][c];
                    if (diag && c > r) L.dist[j * kDistPitch + i] = acc[r][c];
                }
            __syncthreads();
            // rows of tile I take the columns of tile J as candidates
            for (int i = wave; i < rows; i += 4) {
                const int p = L.ida[i];
                KnnRow<SL> row;
                row.load(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
                const bool ok = lane < cols && !(diag && lane == i);
                const float d = L.dist[i * kDistPitch + lane];
                row.offer_lanes(ok, L.idb[lane], d);
                if (row.changed) row.store(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K);
            }
            if (!diag) {
                // columns of tile J take the rows of tile I as candidates
                for (int j = wave; j < cols; j += 4) {
                    const int p = L.idb[j];
                    KnnRow<SL> row;
                    row.load(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
                    const bool ok = lane < rows;
                    const float d = L.dist[lane * kDistPitch + j];
                    row.offer_lanes(ok, L.ida[lane], d);
                    if (row.changed) row.store(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// small-bucket kernel
// ---------------------------------------------------------------------------
constexpr int kSmallCap = 64;
constexpr int kSmallThreads = 128;
constexpr int kSmallWaves = kSmallThreads / 64;
constexpr int kSmallRowsPerWave = kSmallCap / kSmallWaves;
constexpr int kSmallHash = 128;

struct SmallLds {
    union {
        float rows[kSmallCap * kDCP];            // 32 dimensions of every point of the bucket
        float dist[kSmallCap * kDistPitch];      // pair distances (written after the last read of rows)
    } u;
    int ids[kSmallCap];
    int table[kSmallHash];                       // id -> position in the bucket (open addressing)
    unsigned char flags[kSmallWaves][kSmallCap];
};

__device__ __forceinline__ uint32_t bucket_hash(int id)
{
    uint32_t h = (uint32_t)id * 0x9E3779B1u;
    return (h ^ (h >> 15)) & (kSmallHash - 1);
}

// LDS row of bucket member m: members 4t..4t+3 sit 16 rows apart so that the
// 4x4 block of a thread reads rows t, t+16, t+32, t+48 (conflict-free b128).
__device__ __forceinline__ int small_phys(int m) { return (m >> 2) + 16 * (m & 3); }

__global__ __launch_bounds__(kSmallThreads, 3) void k_bucket_knn_small(const float* __restrict__ points, int D, int K,
                                                                    const int* __restrict__ ids,
                                                                    const int* __restrict__ starts,
                                                                    const int* __restrict__ sizes, int stride,
                                                                    int* __restrict__ knn_idx,
                                                                    float* __restrict__ knn_dist)
{
    __shared__ __align__(16) SmallLds L;
    const int bkt = blockIdx.x;
    const int s = sizes[bkt];
    if (s < 2 || s > kSmallCap) return;
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);

    L.table[tid] = -1;
    if (tid < kSmallCap) L.ids[tid] = tid < s ? bid[tid] : -1;
    __syncthreads();

    // K-NN rows of the members this wavefront owns (i = wave, wave+2, ...); loaded while the
    // last block of dimensions is being consumed, so their latency hides behind arithmetic
    int pidx[kSmallRowsPerWave];
    float pdist[kSmallRowsPerWave];
    // hash table of the bucket
    if (tid < s) {
        uint32_t h = bucket_hash(L.ids[tid]);
        for (int probe = 0; probe < kSmallHash; ++probe) {
            if (atomicCAS(&L.table[h], -1, tid) == -1) break;
            h = (h + 1) & (kSmallHash - 1);
        }
    }

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

    // staging: thread t loads piece (t&7) of members (t>>3) + 16*i, i = 0..3
    const int piece = tid & 7;
    const float* rp[4];
    bool live[4];
    int prow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = (tid >> 3) + 16 * i;
        live[i] = m < s;
        rp[i] = points + (size_t)(live[i] ? L.ids[m] : 0) * (size_t)D;
        prow[i] = small_phys(m) * kDCP + piece * 4;
    }
    auto load_piece = [&](int i, int d) -> float4 {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live[i] && d < D) {
            if (vec_ok) {
                v = *reinterpret_cast<const float4*>(rp[i] + d);
            } else {
                v.x = rp[i][d];
                if (d + 1 < D) v.y = rp[i][d + 1];
                if (d + 2 < D) v.z = rp[i][d + 2];
                if (d + 3 < D) v.w = rp[i][d + 3];
            }
        }
        return v;
    };
    float4 pre[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) pre[i] = load_piece(i, piece * 4);

    for (int d0 = 0; d0 < D; d0 += kDC) {
        __syncthreads();                       // previous step's reads of rows are done
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<float4*>(&L.u.rows[prow[i]]) = pre[i];
        if (d0 + kDC < D) {
#pragma unroll
            for (int i = 0; i < 4; ++i) pre[i] = load_piece(i, d0 + kDC + piece * 4);
        }
        __syncthreads();
        if (d0 + kDC >= D) {
#pragma unroll
            for (int u = 0; u < kSmallRowsPerWave; ++u) {
                const int i = wave + kSmallWaves * u;
                pidx[u] = -2;
                pdist[u] = INFINITY;
                if (i < s && lane < K) {
                    const size_t at = (size_t)L.ids[i] * (size_t)K + lane;
                    pidx[u] = knn_idx[at];
                    pdist[u] = knn_dist[at];
                }
            }
        }
        const int pieces = min(8, (D - d0 + 3) >> 2);
        if (has_tile) {
            for (int q = 0; q < pieces; ++q) {
                float4 av[4], bv[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) av[r] = *reinterpret_cast<const float4*>(&L.u.rows[(ti + 16 * r) * kDCP + 4 * q]);
#pragma unroll
                for (int c = 0; c < 4; ++c) bv[c] = *reinterpret_cast<const float4*>(&L.u.rows[(tj + 16 * c) * kDCP + 4 * q]);
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
            const float* ra = &L.u.rows[(dt + 16 * dr) * kDCP];
            const float* rb = &L.u.rows[(dt + 16 * dc) * kDCP];
            for (int q = 0; q < pieces; ++q) {
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
    __syncthreads();                           // rows no longer needed: the union becomes the distance matrix
    if (has_tile) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int i = 4 * ti + r, j = 4 * tj + c;
                if (i < s && j < s) {
                    L.u.dist[i * kDistPitch + j] = acc[r][c];
                    L.u.dist[j * kDistPitch + i] = acc[r][c];
                }
            }
    }
    if (has_diag) {
        const int i = 4 * dt + dr, j = 4 * dt + dc;
        if (j < s) {
            L.u.dist[i * kDistPitch + j] = dacc;
            L.u.dist[j * kDistPitch + i] = dacc;
        }
    }
    __syncthreads();

    // top-K update, one member at a time per wavefront
#pragma unroll
    for (int u = 0; u < kSmallRowsPerWave; ++u) {
        const int i = wave + kSmallWaves * u;
        if (i >= s) break;
        KnnRow<1> row;
        row.idx[0] = pidx[u];
        row.dist[0] = pdist[u];
        row.init_from_regs(K);
        // which members of the bucket does the row already hold?
        L.flags[wave][lane] = 0;
        const int mine = row.idx[0];
        if (mine >= 0) {
            uint32_t h = bucket_hash(mine);
            for (int probe = 0; probe < kSmallHash; ++probe) {
                const int e = L.table[h];
                if (e < 0) break;
                if (L.ids[e] == mine) { L.flags[wave][e] = 1; break; }
                h = (h + 1) & (kSmallHash - 1);
            }
        }
        wave_lds_sync();
        const bool ok = lane < s && lane != i && L.flags[wave][lane] == 0;
        const float d = L.u.dist[i * kDistPitch + lane];
        row.offer_lanes<false>(ok, L.ids[lane], d);
        wave_lds_sync();
        if (row.changed) {
            const size_t at = (size_t)L.ids[i] * (size_t)K;
            row.store(knn_idx + at, knn_dist + at);
        }
    }
}

// Host launcher.  All pointers are device pointers.  max_bucket: size of the
// largest bucket if known, otherwise -1.
int launch_bucket_knn(const float* points, int N, int D, int K, const int* ids, const int* starts,
                      const int* sizes, int n_buckets, int stride, int max_bucket, int* knn_idx, float* knn_dist,
                      hipStream_t stream)
{
    (void)N;
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 256, "bucket K-NN: K must be in 1..256");
    RSFK_CHECK(D >= 1, "bucket K-NN: D must be positive");
    dim3 grid((unsigned)n_buckets);
    int skip_upto = 0;
    if (K <= 64) {
        hipLaunchKernelGGL(k_bucket_knn_small, grid, dim3(kSmallThreads), 0, stream, points, D, K, ids, starts, sizes,
                           stride, knn_idx, knn_dist);
        if (max_bucket >= 0 && max_bucket <= kSmallCap) {
            RSFK_HIP(hipGetLastError());
            return 0;
        }
        skip_upto = kSmallCap;
    }
    dim3 block(256);
    if (K <= 64)
        hipLaunchKernelGGL(k_bucket_knn<1>, grid, block, 0, stream, points, D, K, ids, starts, sizes, stride, skip_upto, knn_idx, knn_dist);
    else if (K <= 128)
        hipLaunchKernelGGL(k_bucket_knn<2>, grid, block, 0, stream, points, D, K, ids, starts, sizes, stride, skip_upto, knn_idx, knn_dist);
    else
        hipLaunchKernelGGL(k_bucket_knn<4>, grid, block, 0, stream, points, D, K, ids, starts, sizes, stride, skip_upto, knn_idx, knn_dist);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
