// Neighbourhood exploration: every point looks at the neighbours of its
// neighbours (taken from a snapshot of the index array) and merges the closer
// ones into its own row.  Replaces nearest_neighbors_exploring
// (src/kernels/nearest_neighbors_exploring.cu:41-146) and its host loop
// (src/rsfk.cu:2100-2135).
//
// One wavefront per point.  The K*K candidate ids are read 64 at a time with
// coalesced row reads of the snapshot; a per-wavefront hash set in LDS drops
// candidates that were already seen (the point itself, its current row, and
// earlier candidates), so each distinct candidate costs one distance.  The
// reference re-evaluates repeated candidates; the result is the same because a
// rejected candidate stays rejected (the row maximum only decreases) and an
// accepted one is found in the row afterwards.
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include <algorithm>

namespace rsfk {

namespace {

constexpr int kWavesPerBlock = 4;

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

// sequential fused multiply-add chain, same arithmetic as the bucket kernel
__device__ __forceinline__ float sqdist_seq(const float* __restrict__ a, const float* __restrict__ b, int D, bool vec_ok)
{
    float acc = 0.0f;
    if (vec_ok) {
        for (int d = 0; d < D; d += 4) {
            const float4 x = *reinterpret_cast<const float4*>(a + d);
            const float4 y = *reinterpret_cast<const float4*>(b + d);
            float df;
            df = x.x - y.x; acc = __builtin_fmaf(df, df, acc);
            df = x.y - y.y; acc = __builtin_fmaf(df, df, acc);
            df = x.z - y.z; acc = __builtin_fmaf(df, df, acc);
            df = x.w - y.w; acc = __builtin_fmaf(df, df, acc);
        }
    } else {
        for (int d = 0; d < D; ++d) {
            const float df = a[d] - b[d];
            acc = __builtin_fmaf(df, df, acc);
        }
    }
    return acc;
}

template <int SL>
__global__ __launch_bounds__(64 * kWavesPerBlock) void k_explore(const float* __restrict__ points, int N, int D, int K,
                                                                  const int* __restrict__ old_idx,
                                                                  int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                                  int table_size)
{
    // dynamic LDS per wavefront: table[table_size] | snapshot row[K]
    extern __shared__ int lds_i[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int* table = lds_i + (size_t)wave * (size_t)(table_size + K);
    int* srow = table + table_size;
    const int p = blockIdx.x * kWavesPerBlock + wave;
    if (p >= N) return;                                   // whole wavefront leaves together
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const int mask = table_size - 1;

    for (int i = lane; i < table_size; i += 64) table[i] = -1;
    KnnRow<SL> row;
    row.load(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
    for (int k = lane; k < K; k += 64) srow[k] = old_idx[(size_t)p * K + k];
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    // seed the set with the point itself and its current row
    if (lane == 0) set_insert(table, mask, p, table_size);
#pragma unroll
    for (int s = 0; s < SL; ++s)
        if (row.idx[s] >= 0) set_insert(table, mask, row.idx[s], table_size);

    const float* xp = points + (size_t)p * D;
    const int total = K * K;
    for (int e0 = 0; e0 < total; e0 += 64) {
        const int e = e0 + lane;
        int c = -1;
        if (e < total) {
            const int i = e / K, k = e - i * K;
            const int q = srow[i];
            if (q >= 0 && q < N) c = old_idx[(size_t)q * K + k];
        }
        bool fresh = c >= 0 && c < N && c != p;
        if (fresh) fresh = set_insert(table, mask, c, 64);
        float d = INFINITY;
        if (fresh) d = sqdist_seq(points + (size_t)c * D, xp, D, vec_ok);
        row.offer_lanes(fresh, c, d);
    }
    if (row.changed) row.store(knn_idx + (size_t)p * K, knn_dist + (size_t)p * K, K);
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
    // set size: at least the number of distinct ids a point can meet, capped by LDS
    int table = std::max(64, next_pow2(K * K + K + 1));
    const int lds_budget = 144 * 1024 / kWavesPerBlock - K * 4;
    while (table * 4 > lds_budget) table >>= 1;
    const size_t lds = (size_t)kWavesPerBlock * (size_t)(table + K) * sizeof(int);
    dim3 grid((unsigned)((N + kWavesPerBlock - 1) / kWavesPerBlock)), block(64 * kWavesPerBlock);
#define RSFK_EXPLORE_LAUNCH(SLV)                                                                                   \
    do {                                                                                                           \
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore<SLV>),                                \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                       \
        hipLaunchKernelGGL(k_explore<SLV>, grid, block, lds, stream, points, N, D, K, old_idx, knn_idx, knn_dist,  \
                           table);                                                                                 \
    } while (0)
    if (K <= 64) RSFK_EXPLORE_LAUNCH(1);
    else if (K <= 128) RSFK_EXPLORE_LAUNCH(2);
    else RSFK_EXPLORE_LAUNCH(4);
#undef RSFK_EXPLORE_LAUNCH
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
