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
//     candidate is looked at once.  The reference re-evaluates repeats; the
//     result is the same because a rejected candidate stays rejected (the row
//     maximum only decreases) and an accepted one is found in the row later;
//   * surviving ids are compacted (ballot + mbcnt ranks) into a queue.  Whenever
//     64 are queued they are screened on the bfloat16 copy of the points: the
//     rows are gathered with coalesced 128-byte segments (8 lanes per row, 64
//     dimensions per step), transposed through LDS, and each lane accumulates for
//     "its" candidate the approximate squared distance d~ and a bound E on
//     |d~ - d|; a candidate with d~ - E >= row maximum cannot enter the row and is
//     dropped without ever touching its fp32 row (most candidates);
//   * the few that pass go to a second queue and get the exact distance from the
//     fp32 rows: same gather/transposition, 32 dimensions per step, sequential
//     fused multiply-add chain per candidate -- the arithmetic of the bucket
//     kernel (compute_knn_from_buckets.cu:40-54), so a pair has one distance
//     value everywhere -- and are then offered to the sorted row.
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
#include <algorithm>

namespace rsfk {

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kChunk = 32;              // fp32 dimensions per staging step (exact path)
constexpr int kChunkB = 64;             // bfloat16 dimensions per staging step (screen)
constexpr int kPitch = kChunk + 4;      // 36 words = 9 x 16 B: conflict-free b128 reads down a column of rows
constexpr int kQueue = 128;             // entries of each candidate queue per wavefront
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
    int* queue;              // fresh candidates waiting for the screen
    int* queue2;             // candidates that passed the screen, waiting for the exact distance
    float* xrow;             // the point's coordinates, zero padded to bf16_pitch(D)
    float* tile;             // 64 x kPitch words
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

// Exact distances of the first n candidates of `queue` to the point, then offer them.
template <int SL>
__device__ __forceinline__ void exact_batch(const ExploreLds& L, const int* queue, int n,
                                            const float* __restrict__ points, int D, bool vec_ok, KnnRow<SL>& row)
{
    const int lane = lane_id();
    const int sub = lane >> 3;          // which of 8 rows of a load step
    const int piece = lane & 7;         // which 16-byte piece of the 128-byte segment
    const int my_c = lane < n ? queue[lane] : -1;
    const float* rp[8];
    bool live[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = i * 8 + sub;
        live[i] = r < n;
        const int c = live[i] ? queue[r] : 0;
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
    wave_lds_sync();
    row.offer_lanes(lane < n, my_c, acc);
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

// Screen the first n candidates of L.queue on the bfloat16 copy.  Returns, per lane,
// whether its candidate may still enter the row.
template <int SL>
__device__ __forceinline__ bool screen_batch(const ExploreLds& L, int n, const Bf16Copy& bf, int D, int Db,
                                             const KnnRow<SL>& row)
{
    const int lane = lane_id();
    const int sub = lane >> 3;
    const int piece = lane & 7;          // 16 bytes = 8 bfloat16 values
    const int my_c = lane < n ? L.queue[lane] : 0;
    const float qn = bf.norms[my_c];
    const uint16_t* rp[8];
    bool live[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = i * 8 + sub;
        live[i] = r < n;
        const int c = live[i] ? L.queue[r] : 0;
        rp[i] = bf.rows + (size_t)c * (size_t)Db;
    }
    const uint4 zero4 = make_uint4(0, 0, 0, 0);
    uint4 pre[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        pre[i] = (live[i] && piece * 8 < Db) ? *reinterpret_cast<const uint4*>(rp[i] + piece * 8) : zero4;
    float da = 0.0f, ta = 0.0f;
    const float tau = row.tau;
    const float slack = (float)(D + 8) * (1.0f / 4194304.0f);      // (D+8) 2^-22: fp32 summation error of both sums
    uint32_t* tile = reinterpret_cast<uint32_t*>(L.tile);
    bool may = lane < n;
    for (int d0 = 0; d0 < Db; d0 += kChunkB) {
        wave_lds_sync();
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *reinterpret_cast<uint4*>(&tile[(i * 8 + sub) * kPitch + piece * 4]) = pre[i];
        if (d0 + kChunkB < Db) {
            const int dn = d0 + kChunkB + piece * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                pre[i] = (live[i] && dn < Db) ? *reinterpret_cast<const uint4*>(rp[i] + dn) : zero4;
        }
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
        // lower bound of the exact distance from the dimensions seen so far
        const float e = ta * (1.02f / 128.0f) + qn * (1.05f / 65536.0f) + da * slack;
        may = lane < n && (da - e < tau);
        if (ballot64(may) == 0) break;
    }
    wave_lds_sync();
    return may;
}

template <int SL>
__global__ __launch_bounds__(64 * kWavesPerBlock) void k_explore(const float* __restrict__ points, Bf16Copy bf, int N,
                                                                  int D, int K, const int* __restrict__ old_idx,
                                                                  int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                                  int table_size, int wave_lds_ints, int dpad)
{
    extern __shared__ __align__(16) int lds_i[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int p = blockIdx.x * kWavesPerBlock + wave;
    if (p >= N) return;                                   // whole wavefront leaves together
    int* base = lds_i + (size_t)wave * (size_t)wave_lds_ints;
    ExploreLds L;
    L.tile = reinterpret_cast<float*>(base);                        // 64*kPitch words, 16-byte aligned
    L.xrow = reinterpret_cast<float*>(base + 64 * kPitch);          // dpad floats (multiple of 8)
    L.queue = base + 64 * kPitch + dpad;
    L.queue2 = L.queue + kQueue;
    L.table = L.queue2 + kQueue;
    L.srow = L.table + table_size;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    const bool use_screen = bf.rows != nullptr;
    const int Db = bf16_pitch(D);
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
    int queued = 0, queued2 = 0;                           // wave-uniform
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
                if (use_screen) {
                    const bool may = screen_batch<SL>(L, 64, bf, D, Db, row);
                    const uint64_t pm = ballot64(may);
                    if (may) L.queue2[queued2 + mask_prefix(pm)] = L.queue[lane];
                    queued2 += __popcll(pm);
                    if (queued2 >= 64) {
                        wave_lds_sync();
                        exact_batch<SL>(L, L.queue2, 64, points, D, vec_ok, row);
                        const int rest2 = queued2 - 64;
                        const int mv2 = lane < rest2 ? L.queue2[64 + lane] : 0;
                        wave_lds_sync();
                        if (lane < rest2) L.queue2[lane] = mv2;
                        queued2 = rest2;
                    }
                } else {
                    exact_batch<SL>(L, L.queue, 64, points, D, vec_ok, row);
                }
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
        if (use_screen) {
            const bool may = screen_batch<SL>(L, queued, bf, D, Db, row);
            const uint64_t pm = ballot64(may);
            if (may) L.queue2[queued2 + mask_prefix(pm)] = L.queue[lane];
            queued2 += __popcll(pm);
        } else {
            exact_batch<SL>(L, L.queue, queued, points, D, vec_ok, row);
        }
    }
    // drain the second queue (at most 127 entries)
    for (int off = 0; off < queued2; off += 64) {
        wave_lds_sync();
        exact_batch<SL>(L, L.queue2 + off, min(64, queued2 - off), points, D, vec_ok, row);
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
// bf may be null (or hold null rows): every candidate then gets the exact distance.
int launch_explore(const float* points, const Bf16Copy* bf, int N, int D, int K, int* knn_idx, float* knn_dist,
                   int* old_idx, hipStream_t stream)
{
    if (N <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 256, "exploration: K must be in 1..256");
    RSFK_HIP(hipMemcpyAsync(old_idx, knn_idx, sizeof(int) * (size_t)N * (size_t)K, hipMemcpyDeviceToDevice, stream));
    const int dpad = bf16_pitch(D);
    const int fixed = 64 * kPitch + dpad + 2 * kQueue + K;              // ints per wavefront besides the set
    RSFK_CHECK((fixed + 64) * 4 * kWavesPerBlock <= 150 * 1024, "exploration: D too large for the LDS budget");
    // set size: at least the number of distinct ids a point can meet, capped by LDS
    int table = std::max(64, next_pow2(K * K + K + 1));
    // two workgroups per CU when possible (160 KB of LDS per CU)
    const int pref_budget = 78 * 1024 / kWavesPerBlock / 4 - fixed;
    const int max_budget = 150 * 1024 / kWavesPerBlock / 4 - fixed;
    if (table > pref_budget && (table >> 1) >= K * K / 2 && (table >> 1) <= pref_budget) table >>= 1;
    while (table > max_budget && table > 64) table >>= 1;
    const int wave_ints = (fixed + table + 3) / 4 * 4;
    const size_t lds = (size_t)kWavesPerBlock * (size_t)wave_ints * sizeof(int);
    Bf16Copy b;
    if (bf) b = *bf;
    dim3 grid((unsigned)((N + kWavesPerBlock - 1) / kWavesPerBlock)), block(64 * kWavesPerBlock);
#define RSFK_EXPLORE_LAUNCH(SLV)                                                                                   \
    do {                                                                                                           \
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore<SLV>),                                \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                       \
        hipLaunchKernelGGL(k_explore<SLV>, grid, block, lds, stream, points, b, N, D, K, old_idx, knn_idx,         \
                           knn_dist, table, wave_ints, dpad);                                                      \
    } while (0)
    if (K <= 64) RSFK_EXPLORE_LAUNCH(1);
    else if (K <= 128) RSFK_EXPLORE_LAUNCH(2);
    else RSFK_EXPLORE_LAUNCH(4);
#undef RSFK_EXPLORE_LAUNCH
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
