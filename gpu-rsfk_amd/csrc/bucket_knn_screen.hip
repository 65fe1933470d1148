// Bucket K-NN for buckets of at most 64 points and K <= 64 when a bfloat16 copy of
// the points exists: same function and same results as the kernel in
// bucket_knn_small.hip (see bucket_knn.hip for the reference kernels both replace),
// but most pair distances are never computed.
//
// A pair (i, j) of a bucket changes nothing unless its distance is smaller than
// the last slot of row i or of row j.  After the first few trees that holds for a
// small fraction of the pairs, so the kernel first bounds every pair from below:
//
//   1. Gram matrix of the bucket's bfloat16 rows with the matrix cores
//      (v_mfma_f32_32x32x16_bf16, operands straight from global memory, one to
//      three 32x32 tiles): d~ = n_i + n_j - 2 G_ij approximates the distance, and
//      a bound on |d~ - exact fp32 result| follows from the norms alone.  With
//      S = n_i + n_j (norms of the bfloat16 rows), u = 2^-8:
//        rounding to bfloat16:   |d(real) - d~(real)| <= 2u sqrt(d~ Q) + u^2 Q,  Q = 2 S  (Cauchy-Schwarz)
//        Gram matrix and norms:  |d~(computed) - d~(real)| <= E1 = (D' + 16) 2^-21 S
//        fp32 chain:             result >= d(real) (1 - gamma),  gamma = (D + 8) 2^-22
//      so the pair is dropped iff  d~ - E1 - 1.01 (2u sqrt((d~ + E1) Q) + u^2 Q) >= (limit + 1e-30) / (1 - gamma),
//      limit = max(last slot of row i, last slot of row j); the inequality is evaluated
//      without the square root (both sides squared when the left side is not negative).
//      This never drops a pair that the exact arithmetic would have inserted;
//   2. the remaining pairs go to a list in LDS; the fp32 rows are staged through LDS
//      in slices of at most 52 dimensions and each thread runs the sequential fused
//      multiply-add chains (arithmetic of euclidean_distance_sqr,
//      compute_knn_from_buckets.cu:40-54) of its pairs of the list;
//   3. the exact distances land in a triangular matrix in LDS (+inf elsewhere) and
//      the rows are updated as in the other kernel; rows without any candidate below
//      their last slot are neither read nor written.
//
// Requires every K-NN row to be sorted by distance on entry (the last slot is the
// maximum); launch_sort_rows establishes that once per build.
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"

namespace rsfk {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kCap = kBucketSplit;          // largest bucket this kernel takes
static_assert(kCap == 64, "two 32-row operand halves and lane-per-candidate merge assume 64");
constexpr int kThreads = 128;
constexpr int kWaves = kThreads / 64;
constexpr int kMaxChunk = 52;               // dimensions staged at once
constexpr int kLanesPerRow = 16;            // a row of a slice is loaded by 16 lanes, 16 bytes each (13 used at most)
constexpr int kRowsPerStep = kThreads / kLanesPerRow;
constexpr int kLoads = kCap / kRowsPerStep; // 16-byte loads per thread and slice
constexpr int kMaxPairs = kCap * (kCap - 1) / 2;
constexpr int kPairsPerThread = (kMaxPairs + kThreads - 1) / kThreads;
static_assert(kMaxChunk / 4 <= kLanesPerRow, "a slice must fit the lanes of a row");

constexpr float kU = 1.0f / 256.0f;                           // unit roundoff of bfloat16 (8 significant bits)
constexpr float kC2 = 1.01f * kU * kU * 2.0001f;              // coefficient of S in the u^2 Q term
constexpr float kC3 = (2.02f * kU) * (2.02f * kU) * 2.0001f;  // (1.01 2u)^2 Q / S

// entry of pair (a, b), a < b, in the triangular matrix
__device__ __forceinline__ int tri_at(int a, int b) { return ((b * (b - 1)) >> 1) + a; }

// Screen one 32x32 tile of the Gram matrix.  Accumulator i of lane l belongs to row member
// m = mbase + 8 (i / 4) + i % 4 (mbase = first member of the operand half + 4 (l / 32)) and column
// member n.  Returns the mask of accumulators whose pair (m < n < s) must be computed exactly.
// taup = (last slot + 1e-30) / (1 - gamma) per member.
__device__ __forceinline__ uint32_t screen_tile(const f32x16& g, int mbase, int n, int s, const float* nrm,
                                                const float* taup, float kappa)
{
    const float nn = nrm[n], tn = taup[n];
    uint32_t bits = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int m = mbase + 8 * (i >> 2) + (i & 3);
        const float S = nrm[m] + nn;
        const float limit = fmaxf(taup[m], tn);
        const float dt = __builtin_fmaf(-2.0f, g[i], S);            // distance of the bfloat16 rows
        const float e1 = kappa * S;                                 // accumulation errors of G and the norms
        const float dhi = fmaxf(dt + e1, 0.0f);
        const float a = dt - e1 - kC2 * S - limit;
        const bool skip = a >= 0.0f && a * a >= kC3 * dhi * S;      // false if anything is NaN
        if (m < n && n < s && !skip) bits |= 1u << i;
    }
    return bits;
}

__global__ __launch_bounds__(kThreads, 4) void k_bucket_knn_screen(const float* __restrict__ points,
                                                                   const uint16_t* __restrict__ brows,
                                                                   const float* __restrict__ bnorms, int D, int K,
                                                                   const int* __restrict__ ids,
                                                                   const int* __restrict__ starts,
                                                                   const int* __restrict__ sizes,
                                                                   int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                                   int chunk, int pitch, int region_floats, int bpitch,
                                                                   int ksteps, float kappa, float inv_one_minus_gamma)
{
    // dynamic LDS: [rows | triangular distance matrix] (region_floats) | ids[64] | tau[64] | taup[64] | nrm[64] |
    //              n_pairs | flag[64] | list
    extern __shared__ __align__(16) float lds_f[];
    float* rows = lds_f;
    float* tri = lds_f;                      // same storage, used after the last read of rows
    int* lids = reinterpret_cast<int*>(lds_f + region_floats);
    float* tau = reinterpret_cast<float*>(lids + kCap);
    float* taup = tau + kCap;
    float* nrm = taup + kCap;
    int* n_pairs = reinterpret_cast<int*>(nrm + kCap);
    int* flag = n_pairs + 4;                 // member has a candidate below its last slot
    uint16_t* list = reinterpret_cast<uint16_t*>(flag + kCap);

    const int bkt = blockIdx.x;
    const int s = sizes[bkt];
    if (s < 2 || s > kCap) return;
    const int* bid = ids + (size_t)starts[bkt];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool vec_ok = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);

    if (tid < kCap) {
        const int id = tid < s ? bid[tid] : -1;
        const float t = id >= 0 ? knn_dist[(size_t)id * (size_t)K + (K - 1)] : 0.0f;
        lids[tid] = id;
        tau[tid] = t;
        taup[tid] = (t + 1e-30f) * inv_one_minus_gamma;
        nrm[tid] = id >= 0 ? bnorms[id] : 0.0f;
    }
    if (tid < kCap) flag[tid] = 0;
    if (tid == 0) *n_pairs = 0;
    __syncthreads();

    // fp32 rows of a slice: lane pc of a group of 16 loads piece pc of rows rg, rg + 8, ...; requested early,
    // written to LDS when the previous slice has been consumed
    const int pc = tid & (kLanesPerRow - 1), rg = tid / kLanesPerRow;
    // two slices are in flight: A holds slices 0, 2, ..., B slices 1, 3, ...
    float4 preA[kLoads], preB[kLoads];
    auto request = [&](float4 (&pre)[kLoads], int d0) {
        const int np = d0 < D ? min(chunk, (D - d0 + 3) & ~3) >> 2 : 0;      // 16-byte pieces per row in this slice
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            pre[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            const int m = rg + kRowsPerStep * i;
            if (pc < np && m < s) {
                const float* src = points + (size_t)lids[m] * (size_t)D + 4 * pc + d0;
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
        return np;
    };
    int npA = 0, npB = 0;

    // ---- 1. screen: wavefront 0 takes the tiles (half 0 x half 0) and (half 0 x half 1), wavefront 1 the
    //         tile (half 1 x half 1); members beyond s read the row of member 0 and are ignored
    {
        const bool two_halves = s > 32;
        const int hx = wave;                                     // operand half of this wavefront's first tile
        if (hx == 0 || two_halves) {
            const int mx = 32 * hx + (lane & 31), my = 32 + (lane & 31);
            const uint16_t* rx = brows + (size_t)lids[mx < s ? mx : 0] * (size_t)bpitch + 8 * (lane >> 5);
            const uint16_t* ry = brows + (size_t)lids[my < s ? my : 0] * (size_t)bpitch + 8 * (lane >> 5);
            const bool second = hx == 0 && two_halves;
            f32x16 gxx, gxy;
#pragma unroll
            for (int i = 0; i < 16; ++i) { gxx[i] = 0.0f; gxy[i] = 0.0f; }
            for (int k0 = 0; k0 < ksteps; k0 += 8) {           // operands of eight steps (128 dimensions) in flight
                bf16x8 x[8], y[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (k0 + u < ksteps) {
                        x[u] = *reinterpret_cast<const bf16x8*>(rx + 16 * (k0 + u));
                        if (second) y[u] = *reinterpret_cast<const bf16x8*>(ry + 16 * (k0 + u));
                        else y[u] = x[u];
                    }
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (k0 + u < ksteps) {
                        gxx = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[u], x[u], gxx, 0, 0, 0);
                        if (second) gxy = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[u], y[u], gxy, 0, 0, 0);
                    }
                }
            }
            // the fp32 rows of the first two slices travel while the tiles are screened
            npA = request(preA, 0);
            npB = request(preB, chunk);
            const int mbase = 32 * hx + 4 * (lane >> 5);
            for (int t = 0; t < (second ? 2 : 1); ++t) {
                const int n = t == 0 ? mx : my;
                uint32_t bits = screen_tile(t == 0 ? gxx : gxy, mbase, n, s, nrm, taup, kappa);
                const int cnt = __popc(bits);
                int at = cnt ? atomicAdd(n_pairs, cnt) : 0;
                while (bits) {
                    const int i = __ffs(bits) - 1;
                    bits &= bits - 1;
                    const int m = mbase + 8 * (i >> 2) + (i & 3);
                    list[at++] = (uint16_t)(m | (n << 6));
                }
            }
        } else {
            npA = request(preA, 0);
            npB = request(preB, chunk);
        }
    }
    __syncthreads();
    const int n_list = *n_pairs;
    const int rounds = (n_list + kThreads - 1) / kThreads;      // pairs per thread, at most kPairsPerThread

    // ---- 2. exact distances of the listed pairs
    float acc[kPairsPerThread];
#pragma unroll
    for (int k = 0; k < kPairsPerThread; ++k) acc[k] = 0.0f;
    auto consume = [&](float4 (&pre)[kLoads], int np_now, bool first) {
        if (!first) __syncthreads();                 // the previous slice has been consumed
        if (pc < np_now) {
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                const int m = rg + kRowsPerStep * i;
                if (m < s) *reinterpret_cast<float4*>(&rows[m * pitch + 4 * pc]) = pre[i];
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kPairsPerThread; ++k) {
            if (k < rounds) {
                const int p = tid + k * kThreads;
                const uint32_t e = p < n_list ? list[p] : 0u;      // idle threads compute pair (0, 0)
                const float* ra = rows + (e & 63u) * (uint32_t)pitch;
                const float* rb = rows + (e >> 6) * (uint32_t)pitch;
                float a = acc[k];
                for (int q = 0; q < np_now; ++q) {
                    const float4 x = *reinterpret_cast<const float4*>(ra + 4 * q);
                    const float4 y = *reinterpret_cast<const float4*>(rb + 4 * q);
                    float df;
                    df = x.x - y.x; a = __builtin_fmaf(df, df, a);
                    df = x.y - y.y; a = __builtin_fmaf(df, df, a);
                    df = x.z - y.z; a = __builtin_fmaf(df, df, a);
                    df = x.w - y.w; a = __builtin_fmaf(df, df, a);
                }
                acc[k] = a;
            }
        }
    };
    for (int d0 = 0; d0 < D; d0 += 2 * chunk) {
        consume(preA, npA, d0 == 0);
        if (d0 + 2 * chunk < D) npA = request(preA, d0 + 2 * chunk);
        if (d0 + chunk < D) {
            consume(preB, npB, false);
            if (d0 + 3 * chunk < D) npB = request(preB, d0 + 3 * chunk);
        }
    }
    __syncthreads();                           // rows no longer needed: the region becomes the distance matrix
    const int n_tri = (s * (s - 1)) >> 1;
    for (int i = tid; i < n_tri; i += kThreads) tri[i] = INFINITY;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kPairsPerThread; ++k) {
        const int p = tid + k * kThreads;
        if (p < n_list) {
            const uint32_t e = list[p];
            const int r = (int)(e & 63u), c = (int)(e >> 6);
            const float d = acc[k];
            tri[tri_at(r, c)] = d;
            if (d <= tau[r]) flag[r] = 1;            // plain stores of the same value: no ordering needed
            if (d <= tau[c]) flag[c] = 1;
        }
    }
    __syncthreads();

    // ---- 3. top-K update.  A wavefront owns every second member and walks those that have a candidate below
    //         their last slot, with the rows of the next two in flight.
    const int my_id = lids[lane];
    // bit u: member wave + 2 u has a candidate
    uint32_t active = (uint32_t)ballot64(lane < 32 && flag[(wave + kWaves * lane) & (kCap - 1)] != 0);
    auto candidate = [&](int i) {
        const int a = min(i, lane), b = max(i, lane);
        return (lane < s && lane != i) ? tri[tri_at(a, b)] : INFINITY;
    };
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
            const float d = candidate(i);
            KnnRow<1> row;
            row.idx[0] = cur_ri[u];
            row.dist[0] = cur_rd[u];
            row.init_sorted(K);
            row.merge(lane < s && lane != i, my_id, d);
            if (row.changed) {
                const size_t at = (size_t)lids[i] * (size_t)K;
                row.store(knn_idx + at, knn_dist + at);
            }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) { cur_i[u] = nxt_i[u]; cur_ri[u] = nxt_ri[u]; cur_rd[u] = nxt_rd[u]; }
    }
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
    RSFK_CHECK(K >= 1 && K <= 256, "sort rows: K must be in 1..256");
    const dim3 grid((unsigned)((N + 3) / 4)), block(256);
    if (K <= 64) hipLaunchKernelGGL(k_sort_rows<1>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    else if (K <= 128) hipLaunchKernelGGL(k_sort_rows<2>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    else hipLaunchKernelGGL(k_sort_rows<4>, grid, block, 0, stream, knn_idx, knn_dist, N, K);
    RSFK_HIP(hipGetLastError());
    return 0;
}

// Buckets of at most 64 points given by (starts, sizes); rows sorted on entry.
int launch_bucket_knn_screen(const float* points, const Bf16Copy& bf, int D, int K, const int* ids, const int* starts,
                             const int* sizes, int n_buckets, int* knn_idx, float* knn_dist, hipStream_t stream)
{
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 64, "screened small-bucket kernel: K must be in 1..64");
    RSFK_CHECK(bf.rows != nullptr && bf.norms != nullptr && starts != nullptr, "screened small-bucket kernel: missing input");
    const int dpad = (D + 3) & ~3;
    const int n_slices = (dpad + kMaxChunk - 1) / kMaxChunk;
    const int chunk = (((dpad + n_slices - 1) / n_slices) + 3) & ~3;
    RSFK_CHECK(chunk >= 4 && chunk <= kMaxChunk, "screened small-bucket kernel: slice width");
    int pitch = chunk;
    if (((pitch >> 2) & 1) == 0) pitch += 4;              // odd number of 16-byte units: rows start in different banks
    RSFK_CHECK(kCap * pitch < 65536, "screened small-bucket kernel: LDS offsets must fit 16 bits");
    const int region = std::max(kCap * pitch, kMaxPairs);
    const int region_floats = (region + 3) & ~3;
    const size_t lds = (size_t)region_floats * 4 + (size_t)(5 * kCap + 4) * 4 + (size_t)kMaxPairs * 2;
    const int ksteps = (bf16_valid(D) + 15) / 16;
    RSFK_CHECK(ksteps * 16 <= bf16_pitch(D), "screened small-bucket kernel: bfloat16 rows too short");
    const float kappa = (float)(ksteps * 16 + 16) * (1.0f / 2097152.0f);            // (Dp + 16) 2^-21
    const float one_minus_gamma = 1.0f - (float)(D + 8) * (1.0f / 4194304.0f);      // 1 - (D + 8) 2^-22
    RSFK_CHECK(one_minus_gamma > 0.5f, "screened small-bucket kernel: D too large");
    const float inv_one_minus_gamma = 1.000001f / one_minus_gamma;                  // rounded up
    RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_bucket_knn_screen),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(k_bucket_knn_screen, dim3((unsigned)n_buckets), dim3(kThreads), lds, stream, points, bf.rows,
                       bf.norms, D, K, ids, starts, sizes, knn_idx, knn_dist, chunk, pitch, region_floats,
                       bf16_pitch(D), ksteps, kappa, inv_one_minus_gamma);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
