// Neighbourhood exploration: every point looks at the neighbours of its
// neighbours (taken from a snapshot of the index array) and merges the closer
// ones into its own row.  Replaces nearest_neighbors_exploring
// (src/kernels/nearest_neighbors_exploring.cu:41-146) and its host loop
// (src/rsfk.cu:2100-2135).
//
// One wavefront per point:
//   * the K*K candidate ids are read with coalesced row reads of the snapshot,
//     up to 16 rows of 64 ids in flight at a time;
//   * a per-wavefront hash set in LDS drops ids that were already seen (the
//     point itself, its current row, earlier candidates), so each distinct
//     candidate costs one distance.  The reference re-evaluates repeats; the
//     result is the same because a rejected candidate stays rejected (the row
//     maximum only decreases) and an accepted one is found in the row later;
//   * surviving ids are compacted (ballot + mbcnt ranks) into a queue; whenever
//     64 are queued their rows are gathered with coalesced 128-byte segments
//     (8 lanes per row, 32 dimensions per step), transposed through LDS, and
//     each lane accumulates the distance of "its" candidate with the same
//     sequential fused multiply-add chain as the bucket kernel
//     (compute_knn_from_buckets.cu:40-54), so a pair has one distance value
//     everywhere.  The next 32 dimensions are in flight while the current ones
//     are consumed; a batch stops early once every partial sum has reached the
//     row maximum (such candidates cannot enter the row).
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include <algorithm>

namespace rsfk {

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kChunk = 32;              // dimensions per staging step
constexpr int kPitch = kChunk + 4;      // 9 x 16 B: conflict-free b128 reads down a column of rows
constexpr int kQueue = 128;             // candidate queue entries per wavefront
constexpr int kIdRows = 16;             // batches of 64 candidate ids loaded back to back

__device__ __forceinline__ uint32_t hash_id(int c)
{
    uint32_t h = (uint32_t)c * 0x9E3779B1u;
    return h ^ (h >> 15);
}

// returns true when c was not in the set (and is now, if there was room)
__device__ __forceinline__ bool set_insert(int* table, int mask, int c, int max_probe)
{
    uint32_t h = hash_id(c) & (uint32_t)mask;
    for (int i = 0; i < max_probe; ++i) {
        const int old = atomicCAS(&table[h], -1, c);
        if (old == -1) return true;
        if (old == c) return false;
        h = (h + 1) & (uint32_t)mask;
    }
    return true;     // set is crowded: treat as new, the row itself is still checked on insertion
}

struct ExploreLds {          // per wavefront; sizes fixed at launch
    int* table;              // hash set, table_size ints
    int* srow;               // snapshot of the point's own row, K ints
    int* queue;              // kQueue ints
    float* xrow;             // the point's coordinates, Dpad floats
    float* tile;             // 64 x kPitch floats
};

// Load one 16-byte piece (4 dimensions) of a candidate row, zero beyond D.
__device__ __forceinline__ float4 load_piece(const float* __restrict__ row, int d, int D, bool vec_ok, bool live)
{
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live && d < D) {
        if (vec_ok) {
            v = *reinterpret_cast<const float4*>(row + d);
        } else {
            v.x = row[d];
            if (d + 1 < D) v.y = row[d + 1];
            if (d + 2 < D) v.z = row[d + 2];
            if (d + 3 < D) v.w = row[d + 3];
        }
    }
    return v;
}

// Distances of the first n queued candidates to the point, then offer them.
template <int SL>
__device__ __forceinline__ void process_batch(const ExploreLds& L, int n, const float* __restrict__ points, int D,
                                              bool vec_ok, KnnRow<SL>& row)
{
    const int lane = lane_id();
    const int sub = lane >> 3;          // which of 8 rows of a load step
    const int piece = lane & 7;         // which 16-byte piece of the 128-byte segment
    const int my_c = lane < n ? L.queue[lane] : -1;
    // row pointers of the 8 rows this lane helps to load
    const float* rp[8];
    bool live[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = i * 8 + sub;
        live[i] = r < n;
        const int c = live[i] ? L.queue[r] : 0;
        rp[i] = points + (size_t)c * (size_t)D;
    }
    float4 pre[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) pre[i] = load_piece(rp[i], piece * 4, D, vec_ok, live[i]);
    float acc = 0.0f;
    const float tau0 = row.tau;
    for (int d0 = 0; d0 < D; d0 += kChunk) {
        wave_lds_sync();                 // previous step's tile reads are done
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *reinterpret_cast<float4*>(&L.tile[(i * 8 + sub) * kPitch + piece * 4]) = pre[i];
        if (d0 + kChunk < D) {
#pragma unroll
            for (int i = 0; i < 8; ++i) pre[i] = load_piece(rp[i], d0 + kChunk + piece * 4, D, vec_ok, live[i]);
        }
        wave_lds_sync();
        const int pieces = min(8, (D - d0 + 3) >> 2);
        const float* mine = &L.tile[lane * kPitch];
        const float* xs = &L.xrow[d0];
        for (int q = 0; q < pieces; ++q) {
            const float4 a = *reinterpret_cast<const float4*>(mine + 4 * q);
            const float4 x = *reinterpret_cast<const float4*>(xs + 4 * q);
            float df;
            df = a.x - x.x; acc = __builtin_fmaf(df, df, acc);
            df = a.y - x.y; acc = __builtin_fmaf(df, df, acc);
            df = a.z - x.z; acc = __builtin_fmaf(df, df, acc);
            df = a.w - x.w; acc = __builtin_fmaf(df, df, acc);
        }
        // partial sums only grow: once all of them reached the row maximum nothing can enter
        if (ballot64(lane < n && acc < tau0) == 0) break;
    }
    row.offer_lanes(lane < n, my_c, acc);
}

template <int SL>
__global__ __launch_bounds__(64 * kWavesPerBlock) void k_explore(const float* __restrict__ points, int N, int D, int K,
                                                                  const int* __restrict__ old_idx,
                                                                  int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                                  int table_size, int wave_lds_ints, int dpad)
{
    extern __shared__ __align__(16) int lds_i[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int p = blockIdx.x * kWavesPerBlock + wave;
    if (p >= N) return;                                   // whole wavefront leaves together
    int* base = lds_i + (size_t)wave * (size_t)wave_lds_ints;
    ExploreLds L;
    L.tile = reinterpret_cast<float*>(base);                        // 64*kPitch floats, 16-byte aligned
    L.xrow = reinterpret_cast<float*>(base + 64 * kPitch);          // dpad floats (multiple of 4)
    L.queue = base + 64 * kPitch + dpad;
    L.table = L.queue + kQueue;
    L.srow = L.table + table_size;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int mask = table_size - 1;

    for (int i = lane; i < table_size; i += 64) L.table[i] = -1;
    KnnRow<SL> row;
    row.load(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
    for (int k = lane; k < K; k += 64) L.srow[k] = old_idx[(size_t)p * K + k];
    const float* xp = points + (size_t)p * D;
    for (int d = lane; d < dpad; d += 64) L.xrow[d] = d < D ? xp[d] : 0.0f;
    wave_lds_sync();
    // seed the set with the point itself and its current row
    if (lane == 0) set_insert(L.table, mask, p, table_size);
#pragma unroll
    for (int s = 0; s < SL; ++s)
        if (row.idx[s] >= 0) set_insert(L.table, mask, row.idx[s], table_size);

    const int total = K * K;
    int queued = 0;                                        // wave-uniform
    for (int g0 = 0; g0 < total; g0 += 64 * kIdRows) {
        int cand[kIdRows];
#pragma unroll
        for (int b = 0; b < kIdRows; ++b) {
            const int e = g0 + b * 64 + lane;
            int c = -1;
            if (e < total) {
                const int i = e / K, k = e - i * K;
                const int q = L.srow[i];
                if (q >= 0 && q < N) c = old_idx[(size_t)q * K + k];
            }
            cand[b] = c;
        }
#pragma unroll
        for (int b = 0; b < kIdRows; ++b) {
            if (g0 + b * 64 >= total) break;
            const int c = cand[b];
            bool fresh = c >= 0 && c < N && c != p;
            if (fresh) fresh = set_insert(L.table, mask, c, 64);
            const uint64_t m = ballot64(fresh);
            if (fresh) L.queue[queued + mask_prefix(m)] = c;
            queued += __popcll(m);
            if (queued >= 64) {
                wave_lds_sync();
                process_batch<SL>(L, 64, points, D, vec_ok, row);
                wave_lds_sync();
                // move the overflow to the front
                const int rest = queued - 64;
                const int mv = lane < rest ? L.queue[64 + lane] : 0;
                wave_lds_sync();
                if (lane < rest) L.queue[lane] = mv;
                queued = rest;
            }
        }
    }
    if (queued > 0) {
        wave_lds_sync();
        process_batch<SL>(L, queued, points, D, vec_ok, row);
    }
    if (row.changed) row.store(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K);
}

int next_pow2(int v)
{
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

}  // namespace

// One exploration pass.  old_idx is scratch of N*K ints (receives the snapshot).
int launch_explore(const float* points, int N, int D, int K, int* knn_idx, float* knn_dist, int* old_idx,
                   hipStream_t stream)
{
    if (N <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 256, "exploration: K must be in 1..256");
    RSFK_HIP(hipMemcpyAsync(old_idx, knn_idx, sizeof(int) * (size_t)N * (size_t)K, hipMemcpyDeviceToDevice, stream));
    const int dpad = (D + 3) / 4 * 4;
    const int fixed = 64 * kPitch + dpad + kQueue + K;                 // ints per wavefront besides the set
    RSFK_CHECK((fixed + 64) * 4 * kWavesPerBlock <= 150 * 1024, "exploration: D too large for the LDS budget");
    // set size: at least the number of distinct ids a point can meet, capped by LDS
    int table = std::max(64, next_pow2(K * K + K + 1));
    // two workgroups per CU when possible (160 KB of LDS per CU)
    const int pref_budget = 76 * 1024 / kWavesPerBlock / 4 - fixed;
    const int max_budget = 150 * 1024 / kWavesPerBlock / 4 - fixed;
    if (table > pref_budget && (table >> 1) >= K * K / 2 && (table >> 1) <= pref_budget) table >>= 1;
    while (table > max_budget && table > 64) table >>= 1;
    const int wave_ints = (fixed + table + 3) / 4 * 4;
    const size_t lds = (size_t)kWavesPerBlock * (size_t)wave_ints * sizeof(int);
    dim3 grid((unsigned)((N + kWavesPerBlock - 1) / kWavesPerBlock)), block(64 * kWavesPerBlock);
#define RSFK_EXPLORE_LAUNCH(SLV)                                                                                   \
    do {                                                                                                           \
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore<SLV>),                                \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                       \
        hipLaunchKernelGGL(k_explore<SLV>, grid, block, lds, stream, points, N, D, K, old_idx, knn_idx, knn_dist,  \
                           table, wave_ints, dpad);                                                                \
    } while (0)
    if (K <= 64) RSFK_EXPLORE_LAUNCH(1);
    else if (K <= 128) RSFK_EXPLORE_LAUNCH(2);
    else RSFK_EXPLORE_LAUNCH(4);
#undef RSFK_EXPLORE_LAUNCH
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
