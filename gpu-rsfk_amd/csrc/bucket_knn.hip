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
// k_bucket_knn_small (bucket_knn_small.hip): buckets of at most 64 points,
//     K <= 64 -- the shape the default parameters produce.
// k_bucket_knn (this file): any bucket size, any K <= 1024, 64x64 tiles of the
//     pair matrix, rows and columns of a tile updated in turn.
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"
#include <algorithm>
#include <cstdlib>

namespace rsfk {

constexpr int kTile = 64;          // points per tile side
constexpr int kDC = 32;            // dimensions staged per step
constexpr int kDCP = kDC + 4;      // LDS row pitch in floats: 9 x 16 B, odd => conflict-free b128 reads
constexpr int kDistPitch = kTile + 1;
constexpr int kStripBuckets = 4096;  // launches over at most this many buckets split them into strips of 64 members

// ---------------------------------------------------------------------------
// general kernel
// ---------------------------------------------------------------------------
struct alignas(16) BucketKnnLds {
    float a[kTile * kDCP];
    float b[kTile * kDCP];
    float dist[kTile * kDistPitch];
    int ida[kTile];
    int idb[kTile];
    // last slot of the rows of the two tiles when the rows are known to be sorted (else +inf), and whether a row got a
    // candidate below it: a row without one is neither read nor written
    float tau_a[kTile];
    float tau_b[kTile];
    int flag_a[kTile];
    int flag_b[kTile];
};

// A thread's share (8 values of one row) of the rows ids[0..rows) x dims [d0, d0+32) on its way from memory to LDS:
// requested into registers first, so that the next 32 dimensions travel while these are being used.
struct StagedRows {
    float v[8];

    __device__ __forceinline__ void request(const int* __restrict__ ids, int rows, const float* __restrict__ points, int D,
                                            int d0, bool vec_ok)
    {
        const int t = threadIdx.x;
        const int r = t >> 2;            // 0..63
        const int seg = (t & 3) * 8;     // 0,8,16,24
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.0f;
        if (r < rows && d0 + seg < D) {
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
    }

    // (zero filled outside the rows and beyond D)
    __device__ __forceinline__ void commit(float* __restrict__ dst) const
    {
        const int t = threadIdx.x;
        float4* d4 = reinterpret_cast<float4*>(dst + (t >> 2) * kDCP + (t & 3) * 8);
        d4[0] = make_float4(v[0], v[1], v[2], v[3]);
        d4[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
};

// STRIP = false: a workgroup per bucket walks the tiles (I, J >= I) of the upper triangle and updates the rows of
// both tiles.  STRIP = true: a workgroup per 64 members of a bucket (workgroup w: tile w % max_tiles of bucket
// w / max_tiles) walks all tiles J and updates only its own rows -- every pair is computed from both ends, but a launch
// over few buckets has max_tiles times as many workgroups, each with half the merges: for grids that would
// otherwise leave most of the device idle.
template <int SL, bool STRIP>
__global__ __launch_bounds__(256) void k_bucket_knn(const float* __restrict__ points, int D, int K,
                                                     const int* __restrict__ ids, const int* __restrict__ starts,
                                                     const int* __restrict__ sizes, int stride, int skip_upto,
                                                     int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                     int rows_sorted, int max_tiles)
{
    __shared__ BucketKnnLds L;
    const int bkt = STRIP ? blockIdx.x / max_tiles : blockIdx.x;
    const int s = sizes[bkt];
    if (s < 2 || s <= skip_upto) return;
    const int I_first = STRIP ? (int)blockIdx.x - bkt * max_tiles : 0;
    if (I_first * kTile >= s) return;
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ty = tid >> 4, tx = tid & 15;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int nt = (s + kTile - 1) / kTile;

    for (int I = I_first; I < (STRIP ? I_first + 1 : nt); ++I) {
        const int rows = min(kTile, s - I * kTile);
        for (int J = STRIP ? 0 : I; J < nt; ++J) {
            const int cols = min(kTile, s - J * kTile);
            const bool diag = (I == J);
            __syncthreads();   // previous tile's LDS fully consumed
            if (tid < kTile) {
                const int p = tid < rows ? bid[I * kTile + tid] : -1;
                L.ida[tid] = p;
                L.tau_a[tid] = (rows_sorted && p >= 0) ? knn_dist[(size_t)p * (size_t)K + (K - 1)] : INFINITY;
                L.flag_a[tid] = 0;
            } else if (tid < 2 * kTile) {
                const int u = tid - kTile;
                const int p = u < cols ? bid[J * kTile + u] : -1;
                L.idb[u] = p;
                L.tau_b[u] = (rows_sorted && p >= 0) ? knn_dist[(size_t)p * (size_t)K + (K - 1)] : INFINITY;
                L.flag_b[u] = 0;
            }
            const int nrb = (rows + 15) >> 4, ncb = (cols + 15) >> 4;
            float acc[4][4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
            __syncthreads();
            StagedRows sa, sb;
            sa.request(L.ida, rows, points, D, 0, vec_ok);
            if (!diag) sb.request(L.idb, cols, points, D, 0, vec_ok);
            for (int d0 = 0; d0 < D; d0 += kDC) {
                sa.commit(L.a);
                if (!diag) sb.commit(L.b);
                __syncthreads();
                if (d0 + kDC < D) {
                    sa.request(L.ida, rows, points, D, d0 + kDC, vec_ok);
                    if (!diag) sb.request(L.idb, cols, points, D, d0 + kDC, vec_ok);
                }
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
                    const float d = acc[r][c];
                    L.dist[i * kDistPitch + j] = d;
                    if (diag && c > r) L.dist[j * kDistPitch + i] = d;
                    if (i < rows && j < cols && !(diag && i == j)) {       // plain stores of the same value: no ordering needed
                        if (d <= L.tau_a[i]) L.flag_a[i] = 1;
                        if (diag) { if (d <= L.tau_a[j]) L.flag_a[j] = 1; }
                        else if (d <= L.tau_b[j]) L.flag_b[j] = 1;
                    }
                }
            __syncthreads();
            // Rows of tile I take the columns of tile J as candidates, then (off the diagonal) the columns of tile J
            // the rows of tile I.  A wavefront walks its rows that have a candidate, the next one's row in flight.
            for (int side = 0; side < ((diag || STRIP) ? 1 : 2); ++side) {
                const int n_mine = side == 0 ? rows : cols, n_other = side == 0 ? cols : rows;
                const int* id_mine = side == 0 ? L.ida : L.idb;
                const int* id_other = side == 0 ? L.idb : L.ida;
                const int* flag = side == 0 ? L.flag_a : L.flag_b;
                const int fm = wave + 4 * lane;                       // bit u of the mask: member wave + 4 u
                uint32_t active = (uint32_t)ballot64(lane < 16 && fm < n_mine && flag[fm < kTile ? fm : 0] != 0);
                auto next_member = [&]() {
                    if (active == 0) return -1;
                    const int u = __ffs(active) - 1;
                    active &= active - 1;
                    return wave + 4 * u;
                };
                int ci = next_member();
                int ri[SL];
                float rd[SL];
                auto fetch = [&](int i, int (&oi)[SL], float (&od)[SL]) {
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) {
                        const int k = lane + 64 * sl;
                        oi[sl] = -2;
                        od[sl] = INFINITY;
                        if (i >= 0 && k < K) {
                            const size_t at = (size_t)id_mine[i] * (size_t)K + k;
                            oi[sl] = knn_idx[at];
                            od[sl] = knn_dist[at];
                        }
                    }
                };
                fetch(ci, ri, rd);
                while (ci >= 0) {
                    const int ni = next_member();
                    int nri[SL];
                    float nrd[SL];
                    fetch(ni, nri, nrd);
                    KnnRow<SL> row;
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) { row.idx[sl] = ri[sl]; row.dist[sl] = rd[sl]; }
                    row.init_from_regs(K);                            // rows that arrive unsorted are rebuilt here
                    const bool ok = lane < n_other && !(diag && lane == ci);
                    const float d = side == 0 ? L.dist[ci * kDistPitch + lane] : L.dist[lane * kDistPitch + ci];
                    row.merge(ok, id_other[lane], d);
                    if (row.changed) {
                        const size_t at = (size_t)id_mine[ci] * (size_t)K;
                        row.store(knn_idx + at, knn_dist + at);
                    }
                    ci = ni;
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) { ri[sl] = nri[sl]; rd[sl] = nrd[sl]; }
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------
// every pair once: the distances of a launch's buckets go through memory
// ---------------------------------------------------------------------------
// The chains of one tile: NRB x NCB blocks of 16 x 16 pairs (a thread has one pair of each block), DIAG: a tile on the
// diagonal, only the blocks on and above the diagonal.  Rows of the two tiles come through LDS 32 dimensions at a time,
// the next 32 on their way while these are used.
template <int NRB, int NCB, bool DIAG>
__device__ __forceinline__ void pair_tile_chains(BucketKnnLds& L, const float* __restrict__ points, int D, int rows, int cols,
                                                 bool vec_ok, float (&acc)[4][4])
{
    const int tid = threadIdx.x;
    const int ty = tid >> 4, tx = tid & 15;
    StagedRows sa, sb;
    sa.request(L.ida, rows, points, D, 0, vec_ok);
    if (!DIAG) sb.request(L.idb, cols, points, D, 0, vec_ok);
    const float* B = DIAG ? L.a : L.b;
    for (int d0 = 0; d0 < D; d0 += kDC) {
        sa.commit(L.a);
        if (!DIAG) sb.commit(L.b);
        __syncthreads();
        if (d0 + kDC < D) {
            sa.request(L.ida, rows, points, D, d0 + kDC, vec_ok);
            if (!DIAG) sb.request(L.idb, cols, points, D, d0 + kDC, vec_ok);
        }
#pragma unroll 2
        for (int dd = 0; dd < kDC; dd += 4) {
            float4 av[NRB], bv[NCB];
#pragma unroll
            for (int r = 0; r < NRB; ++r) av[r] = *reinterpret_cast<const float4*>(&L.a[(ty + 16 * r) * kDCP + dd]);
#pragma unroll
            for (int c = 0; c < NCB; ++c) bv[c] = *reinterpret_cast<const float4*>(&B[(tx + 16 * c) * kDCP + dd]);
#pragma unroll
            for (int r = 0; r < NRB; ++r) {
#pragma unroll
                for (int c = 0; c < NCB; ++c) {
                    if (DIAG && c < r) continue;
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
}

// k_bucket_pairs: workgroup (bucket, I, J >= I) evaluates the 64 x 64 tile (I, J) of the bucket's pair matrix -- the
// chains of k_bucket_knn, one pair per accumulator -- and stores it, and its mirror image (J, I), into the bucket's
// matrix of `pitch` x `pitch` floats (pitch = 64 x the largest number of tiles of a bucket of the launch).  No row is
// touched: every tile of every bucket is a workgroup of its own, whatever the number of buckets, and no pair is
// evaluated from both ends.  k_bucket_merge_pairs (below) then gives every member its row of that matrix.
// tri = max_tiles (max_tiles + 1) / 2 workgroups per bucket; those beyond a bucket's own tiles leave at once.
__global__ __launch_bounds__(256) void k_bucket_pairs(const float* __restrict__ points, int D, const int* __restrict__ ids,
                                                       const int* __restrict__ starts, const int* __restrict__ sizes, int stride,
                                                       int skip_upto, int max_tiles, int tri, int pitch,
                                                       float* __restrict__ pair_dist)
{
    __shared__ BucketKnnLds L;
    const int bkt = blockIdx.x / tri;
    const int s = sizes[bkt];
    if (s < 2 || s <= skip_upto) return;
    // tile (I, J) of place t in the order (0,0) (0,1) .. (0,T-1) (1,1) ..
    int t = (int)blockIdx.x - bkt * tri, I = 0;
    while (t >= max_tiles - I) { t -= max_tiles - I; ++I; }
    const int J = I + t;
    if (J * kTile >= s) return;
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int tid = threadIdx.x;
    const int ty = tid >> 4, tx = tid & 15;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int rows = min(kTile, s - I * kTile), cols = min(kTile, s - J * kTile);
    const bool diag = I == J;
    if (tid < kTile) L.ida[tid] = tid < rows ? bid[I * kTile + tid] : -1;
    else if (tid < 2 * kTile) L.idb[tid - kTile] = tid - kTile < cols ? bid[J * kTile + tid - kTile] : -1;
    const int nrb = (rows + 15) >> 4, ncb = (cols + 15) >> 4;
    float acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
    __syncthreads();
    // (off the diagonal tile I is full: J > I; on it rows == cols)
    if (diag) {
        switch (nrb) {
        case 1: pair_tile_chains<1, 1, true>(L, points, D, rows, cols, vec_ok, acc); break;
        case 2: pair_tile_chains<2, 2, true>(L, points, D, rows, cols, vec_ok, acc); break;
        case 3: pair_tile_chains<3, 3, true>(L, points, D, rows, cols, vec_ok, acc); break;
        default: pair_tile_chains<4, 4, true>(L, points, D, rows, cols, vec_ok, acc); break;
        }
    } else {
        switch (ncb) {
        case 1: pair_tile_chains<4, 1, false>(L, points, D, rows, cols, vec_ok, acc); break;
        case 2: pair_tile_chains<4, 2, false>(L, points, D, rows, cols, vec_ok, acc); break;
        case 3: pair_tile_chains<4, 3, false>(L, points, D, rows, cols, vec_ok, acc); break;
        default: pair_tile_chains<4, 4, false>(L, points, D, rows, cols, vec_ok, acc); break;
        }
    }
    // the tile -> LDS (the blocks below the diagonal of a diagonal tile are the mirror image of those above)
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
    // ... -> the bucket's matrix: rows of tile I (a wavefront stores 64 consecutive floats of a row), then, off the
    // diagonal, the rows of tile J (the columns of the tile in LDS: pitch 65, no bank conflicts)
    float* M = pair_dist + (size_t)bkt * (size_t)pitch * (size_t)pitch;
    const int lane = tid & 63, wave = tid >> 6;
    for (int i = wave; i < rows; i += 4)
        if (lane < cols) M[(size_t)(I * kTile + i) * pitch + J * kTile + lane] = L.dist[i * kDistPitch + lane];
    if (!diag)
        for (int j = wave; j < cols; j += 4)
            if (lane < rows) M[(size_t)(J * kTile + j) * pitch + I * kTile + lane] = L.dist[lane * kDistPitch + j];
}

// One wavefront per member of a bucket: the member's row of the bucket's pair matrix (k_bucket_pairs), 64 distances
// at a time; the K-NN row is read when the first distance at or below its last slot turns up (rows_sorted; else at
// once), takes the candidates of every such batch, and is written back if it changed.
template <int SL>
__global__ __launch_bounds__(256) void k_bucket_merge_pairs(int K, const int* __restrict__ ids, const int* __restrict__ starts,
                                                             const int* __restrict__ sizes, int stride, int skip_upto,
                                                             int pitch, const float* __restrict__ pair_dist,
                                                             int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                             int rows_sorted)
{
    const int per = pitch >> 2;                            // workgroups per bucket: four members each
    const int bkt = blockIdx.x / per;
    const int lane = threadIdx.x & 63;
    const int m = (((int)blockIdx.x - bkt * per) << 2) + (threadIdx.x >> 6);
    const int s = sizes[bkt];
    if (s < 2 || s <= skip_upto || m >= s) return;         // (a whole wavefront leaves)
    const int* bid = ids + (starts ? (size_t)starts[bkt] : (size_t)bkt * (size_t)stride);
    const int p = bid[m];
    const size_t at = (size_t)p * (size_t)K;
    const float* drow = pair_dist + ((size_t)bkt * (size_t)pitch + (size_t)m) * (size_t)pitch;
    const float tau0 = rows_sorted ? knn_dist[at + (K - 1)] : INFINITY;
    KnnRow<SL> row;
    bool loaded = false;
    for (int j0 = 0; j0 < s; j0 += 64) {
        const int j = j0 + lane;
        const bool in = j < s && j != m;
        const float d = in ? drow[j] : INFINITY;
        const int c = in ? bid[j] : -1;
        const bool ok = in && d <= tau0;
        if (ballot64(ok) == 0) continue;
        if (!loaded) {
            row.load(knn_idx + at, knn_dist + at, K);         // rows that arrive unsorted are rebuilt here
            loaded = true;
        }
        row.merge(ok, c, d);
    }
    if (loaded && row.changed) row.store(knn_idx + at, knn_dist + at);
}

namespace {

// Is the form that evaluates every pair once wanted?  RSFK_BUCKET_PAIRS=0 / 1 overrides the choice (the results are
// the same).
bool pairs_form_wanted()
{
    const char* env = std::getenv("RSFK_BUCKET_PAIRS");
    return !(env && env[0] == '0');
}

// The buckets of a launch through k_bucket_pairs + k_bucket_merge_pairs, as many at a time as the working memory holds.
int launch_pairs_form(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes, int n_buckets,
                      int stride, int skip_upto, int* knn_idx, float* knn_dist, hipStream_t stream, bool rows_sorted,
                      int max_tiles, const PairScratch& ps)
{
    const int pitch = max_tiles * kTile, tri = max_tiles * (max_tiles + 1) / 2;
    const size_t per_bucket = (size_t)pitch * (size_t)pitch;
    // (grids stay below 2^31 workgroups)
    const size_t most = std::min(ps.floats / per_bucket, (size_t)0x7fffffff / (size_t)std::max(tri, pitch / 4));
    const int rs = rows_sorted ? 1 : 0;
    for (int b0 = 0; b0 < n_buckets; b0 += (int)most) {
        const int nb = (int)std::min<size_t>(most, (size_t)(n_buckets - b0));
        const int* ids_c = starts ? ids : ids + (size_t)b0 * (size_t)stride;
        const int* starts_c = starts ? starts + b0 : nullptr;
        hipLaunchKernelGGL(k_bucket_pairs, dim3((unsigned)nb * (unsigned)tri), dim3(256), 0, stream, points, D, ids_c, starts_c,
                           sizes + b0, stride, skip_upto, max_tiles, tri, pitch, ps.p);
        const dim3 grid((unsigned)nb * (unsigned)(pitch / 4)), block(256);
#define RSFK_PAIRS_CASE(SLV)                                                                                                \
        hipLaunchKernelGGL(k_bucket_merge_pairs<SLV>, grid, block, 0, stream, K, ids_c, starts_c, sizes + b0, stride, skip_upto, \
                           pitch, ps.p, knn_idx, knn_dist, rs)
        if (K <= 64) RSFK_PAIRS_CASE(1);
        else if (K <= 128) RSFK_PAIRS_CASE(2);
        else if (K <= 256) RSFK_PAIRS_CASE(4);
        else if (K <= 512) RSFK_PAIRS_CASE(8);
        else RSFK_PAIRS_CASE(16);
#undef RSFK_PAIRS_CASE
    }
    RSFK_HIP(hipGetLastError());
    return 0;
}

// pairs: working memory for the form that evaluates every pair once (null, or too small for one bucket of the
// launch: the forms that need none)
int launch_general(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes, int n_buckets,
                   int stride, int skip_upto, int* knn_idx, float* knn_dist, hipStream_t stream, bool rows_sorted = false,
                   int max_bucket = -1, int* launched = nullptr, const PairScratch* pairs = nullptr)
{
    if (n_buckets <= 0) return 0;
    const int rs = rows_sorted ? 1 : 0;
    if (pairs && pairs->p && max_bucket > 0 && pairs_form_wanted()) {
        const int mt = (max_bucket + kTile - 1) / kTile;
        if ((size_t)mt * kTile * (size_t)mt * kTile <= pairs->floats) {
            if (launched) *launched |= kBucketKernelPairs;
            return launch_pairs_form(points, D, K, ids, starts, sizes, n_buckets, stride, skip_upto, knn_idx, knn_dist, stream,
                                     rows_sorted, mt, *pairs);
        }
    }
    // few buckets (and their largest size known): a workgroup per 64 members instead of one per bucket
    const int max_tiles = max_bucket > 0 ? (max_bucket + kTile - 1) / kTile : 0;
    const char* env = std::getenv("RSFK_BUCKET_STRIP");        // 0 / 1 overrides the choice (the results are the same)
    const bool strip = max_tiles > 1 && (env && *env ? env[0] == '1' : n_buckets <= kStripBuckets);
    dim3 grid((unsigned)n_buckets * (unsigned)(strip ? max_tiles : 1)), block(256);
    if (launched) *launched |= strip ? kBucketKernelStrip : kBucketKernelTiled;
#define RSFK_GENERAL_CASE(SLV)                                                                                              \
    do {                                                                                                                    \
        if (strip)                                                                                                          \
            hipLaunchKernelGGL((k_bucket_knn<SLV, true>), grid, block, 0, stream, points, D, K, ids, starts, sizes, stride,  \
                               skip_upto, knn_idx, knn_dist, rs, max_tiles);                                                \
        else                                                                                                                \
            hipLaunchKernelGGL((k_bucket_knn<SLV, false>), grid, block, 0, stream, points, D, K, ids, starts, sizes, stride, \
                               skip_upto, knn_idx, knn_dist, rs, 1);                                                        \
    } while (0)
    if (K <= 64) RSFK_GENERAL_CASE(1);
    else if (K <= 128) RSFK_GENERAL_CASE(2);
    else if (K <= 256) RSFK_GENERAL_CASE(4);
    else if (K <= 512) RSFK_GENERAL_CASE(8);
    else RSFK_GENERAL_CASE(16);
#undef RSFK_GENERAL_CASE
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace

namespace {

__global__ __launch_bounds__(256) void k_max_size(const int* __restrict__ sizes, int n, int* __restrict__ out)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    int v = i < n ? sizes[i] : 0;
    v = max(v, __shfl_xor(v, 32, 64));
    v = max(v, __shfl_xor(v, 16, 64));
    v = max(v, __shfl_xor(v, 8, 64));
    v = max(v, __shfl_xor(v, 4, 64));
    v = max(v, __shfl_xor(v, 2, 64));
    v = max(v, __shfl_xor(v, 1, 64));
    if ((threadIdx.x & 63) == 0 && v > 0) atomicMax(out, v);
}

// size of the largest bucket of a table in device memory (one trip to the host)
int largest_bucket(const int* sizes, int n, hipStream_t stream, int* out)
{
    void* d = nullptr;
    if (ws_alloc(&d, sizeof(int))) return 1;
    int v = 0;
    hipError_t e = hipMemcpyAsync(d, &v, sizeof(int), hipMemcpyHostToDevice, stream);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(k_max_size, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, sizes, n, static_cast<int*>(d));
        e = hipMemcpyAsync(&v, d, sizeof(int), hipMemcpyDeviceToHost, stream);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    ws_free(d);
    if (e != hipSuccess) { set_last_error(std::string("largest bucket: ") + hipGetErrorString(e)); return 1; }
    *out = v;
    return 0;
}

}  // namespace

// Largest bucket that goes to the kernel that keeps a bucket's points in LDS (0: none); RSFK_BUCKET_ROWS=0 switches
// it off.
static int resident_rows_cap(int D, int K)
{
    const char* e = std::getenv("RSFK_BUCKET_ROWS");
    if (e && e[0] == '0') return 0;
    return bucket_rows_cap(D, K);
}

int bucket_gram_from()
{
    // Off unless asked for: on the shapes measured so far (bucket sizes 33..256, D 32..784, K 32 and 90) the direct
    // kernels are faster -- their time goes into the merges and the waits between phases, not into the fp32 chains
    // the screen saves.
    const char* e = std::getenv("RSFK_GRAM_FROM");
    if (e && *e) return std::max(0, std::atoi(e));
    return 0x7fffffff;
}

size_t pair_scratch_max()
{
    const char* e = std::getenv("RSFK_BUCKET_PAIRS_MB");
    const long long mb = e && *e ? std::atoll(e) : 512;
    return (size_t)std::max(1ll, std::min(mb, 16384ll)) << 18;          // floats
}

size_t bucket_pairs_scratch_floats(int D, int K, int n_buckets, int max_bucket)
{
    if (n_buckets <= 0 || max_bucket < 2 || !pairs_form_wanted()) return 0;
    // (buckets the specialised kernels take never reach the general one)
    if (K <= 64 && max_bucket <= std::max(medium_bucket_cap(), resident_rows_cap(D, K))) return 0;
    const size_t pitch = (size_t)((max_bucket + kTile - 1) / kTile) * kTile;
    if (pitch * pitch > pair_scratch_max()) return 0;
    return std::min(pair_scratch_max(), (size_t)n_buckets * pitch * pitch);
}

// Host launcher for an arbitrary list of buckets.  All pointers are device pointers.  max_bucket: size of
// the largest bucket if known, otherwise -1.
int launch_bucket_knn(const float* points, int N, int D, int K, const int* ids, const int* starts,
                      const int* sizes, int n_buckets, int stride, int max_bucket, int* knn_idx, float* knn_dist,
                      hipStream_t stream)
{
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= kMaxK, "bucket K-NN: K must be in 1..1024");
    RSFK_CHECK(D >= 1, "bucket K-NN: D must be positive");
    if (bucket_gram_from() == 0 && K <= kMaxKJoin) {
        // RSFK_GRAM_FROM=0: the screened kernel for every call; it needs sorted rows and the size of the largest bucket
        if (launch_sort_rows(knn_idx, knn_dist, N, K, stream)) return 1;
        if (max_bucket < 0 && largest_bucket(sizes, n_buckets, stream, &max_bucket)) return 1;
        return launch_bucket_knn_gram(points, D, K, ids, starts, sizes, n_buckets, stride, 2, max_bucket, knn_idx, knn_dist, stream);
    }
    int skip_upto = 0;
    if (K <= 64) {
        // buckets of up to 72 points go to the specialised kernels; the general one skips them
        if (bucket_screen_share_q16() == kScreenAlways) {
            // RSFK_BUCKET_SCREEN=always: the screened kernel for every call; it needs sorted rows
            if (launch_sort_rows(knn_idx, knn_dist, N, K, stream)) return 1;
            if (launch_bucket_knn_screen(points, D, K, ids, starts, sizes, n_buckets, stride, knn_idx, knn_dist, stream)) return 1;
        } else if (launch_bucket_knn_small(points, D, K, ids, starts, sizes, n_buckets, stride, false, knn_idx, knn_dist, stream))
            return 1;
        if (max_bucket >= 0 && max_bucket <= small_bucket_cap()) return 0;
        if (launch_bucket_knn_medium(points, D, K, ids, starts, sizes, n_buckets, stride, false, knn_idx, knn_dist, stream))
            return 1;
        if (max_bucket >= 0 && max_bucket <= medium_bucket_cap()) return 0;
        skip_upto = medium_bucket_cap();
        const int rows_cap = resident_rows_cap(D, K);
        if (rows_cap > skip_upto) {
            // buckets whose points fit into LDS whole: every K-NN row is touched once
            if (launch_bucket_knn_rows(points, D, K, ids, starts, sizes, n_buckets, stride, skip_upto + 1,
                                       max_bucket >= 0 ? std::min(max_bucket, rows_cap) : rows_cap, false, true, knn_idx, knn_dist, stream))
                return 1;
            if (max_bucket >= 0 && max_bucket <= rows_cap) return 0;
            skip_upto = rows_cap;
        }
    }
    // the rest: every pair once, with working memory for the pair matrices, when there is room for it
    PairScratch ps;
    if (pairs_form_wanted()) {
        if (max_bucket < 0 && largest_bucket(sizes, n_buckets, stream, &max_bucket)) return 1;
        if (max_bucket <= skip_upto) return 0;            // (the kernels above have taken every bucket)
        const size_t want = bucket_pairs_scratch_floats(D, K, n_buckets, max_bucket);
        void* mem = nullptr;
        if (want > 0 && ws_try_alloc(&mem, want * sizeof(float)) == 0) {
            ps.p = static_cast<float*>(mem);
            ps.floats = want;
        }
    }
    const int rc = launch_general(points, D, K, ids, starts, sizes, n_buckets, stride, skip_upto, knn_idx, knn_dist, stream, false,
                                  max_bucket, nullptr, &ps);
    if (ps.p) {
        // (the block goes back to the pool only when nothing uses it any more)
        const hipError_t e = hipStreamSynchronize(stream);
        ws_free(ps.p);
        if (rc == 0 && e != hipSuccess) { set_last_error(std::string("bucket K-NN: ") + hipGetErrorString(e)); return 1; }
    }
    return rc;
}

// Host launcher for the leaf table of one tree: n_small buckets of at most kBucketSplit points at the front of
// (starts, sizes), n_big larger ones at the back of the table of leaf_cap entries.  rows_sorted: every K-NN row is
// known to be sorted by distance.  stats (8 zeroed words; with K <= 64 and sorted rows): the small buckets go to the
// kernel that chooses between the direct and the screened form from the pairs of the tree before (prev_stats, null for
// the first tree) and leaves its own numbers in stats.  part: 0 = all buckets, 1 = only the small ones, 2 = only the larger ones (the two
// kinds touch different rows, so the two parts of one tree may run side by side).  young_rows: the rows may be new or
// far from done (first trees of a build).  pairs: working memory for the buckets that reach the general kernel (null:
// its forms that need none); launches that may run side by side need one each.
int launch_bucket_knn_tree(const float* points, const unsigned long long* prev_stats, unsigned long long* stats,
                           bool rows_sorted, bool gram, int D, int K, const int* ids, const int* starts, const int* sizes,
                           int leaf_cap, int n_small, int n_big, int max_bucket, int* knn_idx, float* knn_dist,
                           hipStream_t stream, int part, bool young_rows, int* launched, const PairScratch* pairs)
{
    RSFK_CHECK(K >= 1 && K <= kMaxK, "bucket K-NN: K must be in 1..1024");
    RSFK_CHECK(D >= 1, "bucket K-NN: D must be positive");
    int none = 0;
    int& used = launched ? *launched : none;              // which kernels this tree's buckets went to (kBucketKernel...)
    if (gram && rows_sorted && K <= kMaxKJoin) {
        used |= kBucketKernelGram;
        // pair matrix screened on the matrix cores; buckets of 65..72 points (K <= 64) keep their own kernel
        if (n_small > 0 && part != 2 &&
            launch_bucket_knn_gram(points, D, K, ids, starts, sizes, n_small, 0, 2, kBucketSplit, knn_idx, knn_dist, stream))
            return 1;
        if (n_big <= 0 || part == 1) return 0;
        const int off = leaf_cap - n_big;
        int from = kBucketSplit + 1;
        if (K <= 64) {
            used |= kBucketKernelMedium;
            if (launch_bucket_knn_medium(points, D, K, ids, starts + off, sizes + off, n_big, 0, rows_sorted, knn_idx, knn_dist, stream))
                return 1;
            if (max_bucket >= 0 && max_bucket <= medium_bucket_cap()) return 0;
            from = medium_bucket_cap() + 1;
        }
        if (max_bucket < 0 && largest_bucket(sizes + off, n_big, stream, &max_bucket)) return 1;
        return launch_bucket_knn_gram(points, D, K, ids, starts + off, sizes + off, n_big, 0, from, max_bucket, knn_idx, knn_dist,
                                      stream);
    }
    if (n_small > 0 && part != 2) {
        if (K <= 64 && stats && rows_sorted) {
            used |= kBucketKernelAuto;
            if (launch_bucket_knn_auto(points, D, K, ids, starts, sizes, n_small, knn_idx, knn_dist, prev_stats, stats, stream))
                return 1;
        } else if (K <= 64) {
            used |= kBucketKernelSmall;
            if (launch_bucket_knn_small(points, D, K, ids, starts, sizes, n_small, 0, rows_sorted, knn_idx, knn_dist, stream)) return 1;
        } else if (launch_general(points, D, K, ids, starts, sizes, n_small, 0, 0, knn_idx, knn_dist, stream, rows_sorted,
                                  kBucketSplit, &used, pairs)) {
            return 1;
        }
    }
    // the large ones: 65..72 points to the three-wavefront variant of the small kernel, the rest to the general one
    if (n_big <= 0 || part == 1) return 0;
    const int off = leaf_cap - n_big;
    int skip_upto = 0;
    if (K <= 64) {
        used |= kBucketKernelMedium;
        if (launch_bucket_knn_medium(points, D, K, ids, starts + off, sizes + off, n_big, 0, rows_sorted, knn_idx, knn_dist, stream))
            return 1;
        if (max_bucket >= 0 && max_bucket <= medium_bucket_cap()) return 0;
        skip_upto = medium_bucket_cap();
        const int rows_cap = resident_rows_cap(D, K);
        if (rows_cap > skip_upto) {
            used |= kBucketKernelRows;
            if (launch_bucket_knn_rows(points, D, K, ids, starts + off, sizes + off, n_big, 0, skip_upto + 1,
                                       max_bucket >= 0 ? std::min(max_bucket, rows_cap) : rows_cap, rows_sorted, young_rows, knn_idx,
                                       knn_dist, stream))
                return 1;
            if (max_bucket >= 0 && max_bucket <= rows_cap) return 0;
            skip_upto = rows_cap;
        }
    }
    return launch_general(points, D, K, ids, starts + off, sizes + off, n_big, 0, skip_upto, knn_idx, knn_dist, stream,
                          rows_sorted, max_bucket, &used, pairs);
}

}  // namespace rsfk
