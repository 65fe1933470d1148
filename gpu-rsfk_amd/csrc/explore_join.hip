// Candidate generation for the neighbourhood exploration as a join over the reversed
// graph.  Same candidates as nearest_neighbors_exploring
// (src/kernels/nearest_neighbors_exploring.cu:41-146) looks at -- for a point p the
// neighbours c of its neighbours q -- but enumerated from the middle: for every q, all
// pairs (p, c) with p in R(q) = {points that list q} and c in N(q).  The rows of N(q)
// and R(q) are then loaded once per q instead of once per pair, and the pair distances
// of a 32 x 32 tile come from one chain of matrix-core instructions on the bfloat16
// copy of the points (v_mfma_f32_32x32x16_bf16: Gram matrix G, d~ = n_p + n_c - 2 G).
//
// d~ is only used to discard.  With S = n_p + n_c (norms of the bfloat16 rows), u = 2^-8:
//   rounding to bfloat16:   |d(real) - d~(real)| <= 2u sqrt(d~ Q) + u^2 Q,  Q = 2 S  (Cauchy-Schwarz)
//   Gram matrix and norms:  |d~(computed) - d~(real)| <= E1 = (D' + 16) 2^-21 S
//   fp32 chain:             result >= d(real) (1 - gamma),  gamma = (D + 8) 2^-22
// so L = (d~ - E1 - 1.01 (2u sqrt((d~ + E1) Q) + u^2 Q)) (1 - gamma) is a lower bound of the exact fp32
// distance, and a pair is dropped when L is above the last slot of row p.
// The outcome is one bit per (entry of the graph, neighbour slot): pass[j] for entry j
// of the reversed graph (p lists q) has bit n set iff neighbour n of q may enter row p.
// The exploration kernel of point p finds its entries through fwd2rev, gathers the
// few ids whose bit is set (a few per cent), computes their exact distances and
// merges them.  Nothing is decided here that the exact arithmetic would decide
// otherwise; no atomics on shared counters, no buffer that can overflow.
//
// For the merge kernel that works through a point's candidates in the order of their
// bounds (explore.hip: rows with many candidates), L itself is kept for every marked
// pair, rounded down to a bfloat16 number (16 bits per pair of the join).
//
// Steps: in-degree count -> exclusive scan -> fill R (compressed rows) and the map
// from graph entries to their place in R -> join.
#include "rsfk_common.hpp"
#include "wave64.hpp"
#include "forest.hpp"
#include <algorithm>
#include <cstdlib>

namespace rsfk {

struct ExploreWorkspace {
    int N = 0, K = 0, MW = 0;  // MW = 32-bit words per entry of pass
    int* rev = nullptr;        // N*K: R lists, compressed rows
    int* fwd2rev = nullptr;    // N*K: entry (p, k) of the graph -> its place in rev (-1: no valid neighbour there)
    int* offs = nullptr;       // N+1: start of R(q)
    int* deg = nullptr;        // N: in-degree (counted, then consumed by the fill)
    int* totals = nullptr;     // per scan block
    uint32_t* pass = nullptr;  // N*K*MW
    uint16_t* bounds = nullptr; // N*K*32*MW lower bounds of the marked pairs (bfloat16, rounded down), or null
    int* todo = nullptr;       // two lists of N+1 ints: points left over by a launch; entry N = their number
    int* host_count = nullptr; // pinned
    int n_blocks = 0;
};
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kScanBlock = 1024;            // elements per workgroup of the scan (256 threads x 4)
constexpr float kU = 1.0f / 256.0f;         // unit roundoff of bfloat16

__global__ void k_zero(int* a, int n, int* counter0, int* counter1)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) a[i] = 0;
    if (i == 0) { *counter0 = 0; *counter1 = 0; }
}

__global__ void k_degree(const int* __restrict__ old_idx, size_t total, int N, int* __restrict__ deg)
{
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const int q = old_idx[e];
        if (q >= 0 && q < N) atomicAdd(&deg[q], 1);
    }
}

// exclusive scan of 256 values, one per thread; returns the block total in *total
__device__ __forceinline__ int block_scan_256(int v, int* total, int* lds4)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
    }
    if (lane == 63) lds4[wave] = incl;
    __syncthreads();
    int woff = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) { const int x = lds4[w]; if (w < wave) woff += x; tot += x; }
    __syncthreads();
    *total = tot;
    return woff + incl - v;
}

__global__ __launch_bounds__(256) void k_scan_blocks(const int* __restrict__ deg, int N, int* __restrict__ offs,
                                                     int* __restrict__ totals)
{
    __shared__ int lds4[4];
    const int i0 = blockIdx.x * kScanBlock + threadIdx.x * 4;
    int v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = i0 + j < N ? deg[i0 + j] : 0;
    const int mine = v[0] + v[1] + v[2] + v[3];
    int tot;
    int run = block_scan_256(mine, &tot, lds4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (i0 + j < N) offs[i0 + j] = run;
        run += v[j];
    }
    if (threadIdx.x == 0) totals[blockIdx.x] = tot;
}

// exclusive scan of the block totals in place, one workgroup; also writes the grand total to *last
__global__ __launch_bounds__(256) void k_scan_totals(int* __restrict__ totals, int n_blocks, int* __restrict__ last)
{
    __shared__ int lds4[4];
    int carry = 0;
    for (int b0 = 0; b0 < n_blocks; b0 += 256) {
        const int i = b0 + threadIdx.x;
        const int v = i < n_blocks ? totals[i] : 0;
        int tot;
        const int ex = block_scan_256(v, &tot, lds4);
        if (i < n_blocks) totals[i] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0) *last = carry;
}

__global__ __launch_bounds__(256) void k_scan_add(int* __restrict__ offs, int N, const int* __restrict__ totals)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < N) offs[i] += totals[i / kScanBlock];
}

__global__ void k_fill_rev(const int* __restrict__ old_idx, size_t total, int N, int K, int* __restrict__ deg,
                           const int* __restrict__ offs, int* __restrict__ rev, int* __restrict__ fwd2rev)
{
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const int q = old_idx[e];
        int j = -1;
        if (q >= 0 && q < N) {
            j = offs[q] + atomicSub(&deg[q], 1) - 1;
            rev[j] = (int)(e / (size_t)K);
        }
        fwd2rev[e] = j;
    }
}

// One wavefront per q.  Per-wavefront LDS (ints): cq[KP] | pid[32] | pn[32] | ptau[32], KP = K rounded up to 32.
template <int WAVES, bool BOUNDS>
__global__ __launch_bounds__(64 * WAVES) void k_explore_join(Bf16Copy bf, int N, int K, const int* __restrict__ old_idx,
                                                              const float* __restrict__ knn_dist,
                                                              const int* __restrict__ offs, const int* __restrict__ rev,
                                                              uint32_t* __restrict__ pass, uint16_t* __restrict__ bounds, int KP, int bpitch, int ksteps,
                                                              float kappa, float one_minus_gamma, int wave_lds_ints)
{
    extern __shared__ __align__(16) int lds_join[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int q = blockIdx.x * WAVES + wave;
    if (q >= N) return;                                   // whole wavefront leaves together
    const int r0 = offs[q], R = offs[q + 1] - r0;
    if (R <= 0) return;
    int* cq = lds_join + (size_t)wave * (size_t)wave_lds_ints;
    int* pid = cq + KP;
    float* pn = reinterpret_cast<float*>(pid + 32);
    float* ptau = pn + 32;
    const int MW = KP >> 5;

    for (int k = lane; k < KP; k += 64) {
        int c = k < K ? old_idx[(size_t)q * K + k] : -1;
        if (c < 0 || c >= N) c = -1;
        cq[k] = c;
    }

    for (int pt0 = 0; pt0 < R; pt0 += 32) {
        const int np = min(32, R - pt0);
        wave_lds_sync();                                  // reads of the previous tile are done (and cq is written)
        if (lane < 32) {
            const int p = lane < np ? rev[(size_t)r0 + pt0 + lane] : -1;
            pid[lane] = p;
            pn[lane] = p >= 0 ? bf.norms[p] : 0.0f;
            ptau[lane] = p >= 0 ? knn_dist[(size_t)p * K + (K - 1)] : 0.0f;
        }
        wave_lds_sync();

        const int pm = pid[lane & 31];
        const uint16_t* ra = bf.rows + (size_t)(pm >= 0 ? pm : q) * (size_t)bpitch + 8 * (lane >> 5);
        const int mbase = 4 * (lane >> 5);
        for (int ct = 0; ct < MW; ++ct) {
            const int cid = cq[ct * 32 + (lane & 31)];
            const uint16_t* rb = bf.rows + (size_t)(cid >= 0 ? cid : q) * (size_t)bpitch + 8 * (lane >> 5);
            const float cn = cid >= 0 ? bf.norms[cid] : 0.0f;
            f32x16 g;
#pragma unroll
            for (int i = 0; i < 16; ++i) g[i] = 0.0f;
            for (int k0 = 0; k0 < ksteps; k0 += 4) {
                bf16x8 a[4], b[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (k0 + u < ksteps) {
                        a[u] = *reinterpret_cast<const bf16x8*>(ra + 16 * (k0 + u));
                        b[u] = *reinterpret_cast<const bf16x8*>(rb + 16 * (k0 + u));
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (k0 + u < ksteps) g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u], b[u], g, 0, 0, 0);
            }
            // Accumulator i of lane l: point m = 4 (l / 32) + 8 (i / 4) + i % 4 of the tile, column = neighbour l % 32
            // of this group of 32.  The ballot over the wavefront therefore holds the 32-bit masks of two points:
            // low half for m = 8 (i / 4) + i % 4, high half for m + 4.
            uint32_t mine = 0;                            // mask of the point this lane stores (lanes 0..31)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int m = mbase + 8 * (i >> 2) + (i & 3);
                const float S = pn[m] + cn;
                const float dt = __builtin_fmaf(-2.0f, g[i], S);
                const float e1 = kappa * S;
                const float dhi = fmaxf(dt + e1, 0.0f);
                const float Q = 2.0001f * S;
                const float ebf = 1.01f * (2.0f * kU * __builtin_sqrtf(dhi * Q) + kU * kU * Q);
                const float lower = (dt - e1 - ebf) * one_minus_gamma - 1e-30f;
                const bool skip = lower > ptau[m];        // false if anything is NaN; a tie at the last slot may still enter (smaller index)
                const bool marked = cid >= 0 && !skip;
                const uint64_t bm = ballot64(marked);
                if (BOUNDS && marked && m < np) {
                    // a bound below zero (or NaN) says nothing: 0.  Dropping the low half of a positive float rounds down.
                    const uint32_t lb = lower > 0.0f ? __float_as_uint(lower) >> 16 : 0u;
                    bounds[((size_t)r0 + pt0 + m) * (size_t)KP + ct * 32 + (lane & 31)] = (uint16_t)lb;
                }
                const int m_lo = 8 * (i >> 2) + (i & 3);
                if (lane == m_lo) mine = (uint32_t)bm;
                if (lane == m_lo + 4) mine = (uint32_t)(bm >> 32);
            }
            if (lane < np) pass[((size_t)r0 + pt0 + lane) * MW + ct] = mine;
        }
    }
}

}  // namespace

// The join is used unless RSFK_EXPLORE_JOIN=0 is set or the graph has 2^31 or more entries.
bool explore_join_enabled(int N, int K)
{
    const char* env = std::getenv("RSFK_EXPLORE_JOIN");
    if (env && env[0] == '0') return false;
    return (size_t)N * (size_t)K < ((size_t)1 << 31);
}

size_t explore_ws_bytes(int N, int K)
{
    const size_t mw = (size_t)((K + 31) / 32);
    return (size_t)N * ((size_t)K * 4 * (2 + mw) + 24) + 4096;
}

int explore_ws_alloc(ExploreWorkspace** out, int N, int K, bool with_bounds)
{
    *out = nullptr;
    auto* w = new ExploreWorkspace();
    w->N = N;
    w->K = K;
    w->MW = (K + 31) / 32;
    w->n_blocks = (N + kScanBlock - 1) / kScanBlock;
    auto dm = [](void* p, size_t n) { return ws_alloc(reinterpret_cast<void**>(p), std::max<size_t>(n, 1) * sizeof(int)) ? hipErrorOutOfMemory : hipSuccess; };
    if (dm(&w->rev, (size_t)N * K) != hipSuccess || dm(&w->fwd2rev, (size_t)N * K) != hipSuccess ||
        dm(&w->offs, (size_t)N + 1) != hipSuccess || dm(&w->deg, (size_t)N) != hipSuccess ||
        dm(&w->totals, (size_t)w->n_blocks + 1) != hipSuccess || dm(&w->pass, (size_t)N * K * w->MW) != hipSuccess ||
        dm(&w->todo, 2 * ((size_t)N + 1)) != hipSuccess ||
        hipHostMalloc(reinterpret_cast<void**>(&w->host_count), sizeof(int)) != hipSuccess) {
        explore_ws_free(w);
        set_last_error("exploration workspace: out of device memory");
        return 1;
    }
    if (with_bounds) {
        // 2 bytes per pair of the join; without them the merge still works, in the order of the marks
        void* b = nullptr;
        if (ws_alloc(&b, (size_t)N * K * w->MW * 32 * sizeof(uint16_t)) == 0) w->bounds = static_cast<uint16_t*>(b);
    }
    *out = w;
    return 0;
}

void explore_ws_free(ExploreWorkspace* w)
{
    if (!w) return;
    void* bufs[] = {w->rev, w->fwd2rev, w->offs, w->deg, w->totals, w->pass, w->todo, w->bounds};
    for (void* b : bufs)
        ws_free(b);
    if (w->host_count) (void)hipHostFree(w->host_count);
    delete w;
}

const int* explore_ws_fwd2rev(const ExploreWorkspace* w) { return w->fwd2rev; }
const uint32_t* explore_ws_pass(const ExploreWorkspace* w) { return w->pass; }
const uint16_t* explore_ws_bounds(const ExploreWorkspace* w) { return w->bounds; }
int* explore_ws_todo(ExploreWorkspace* w, int which) { return w->todo + (size_t)which * ((size_t)w->N + 1); }
int* explore_ws_host_count(ExploreWorkspace* w) { return w->host_count; }

// Fill pass and fwd2rev from the snapshot old_idx and the current last slots of knn_dist (rows sorted by distance).
int launch_explore_join(ExploreWorkspace* w, const Bf16Copy& bf, int N, int D, int K, const int* old_idx,
                        const float* knn_dist, hipStream_t stream)
{
    RSFK_CHECK(w && w->N == N && w->K == K, "exploration join: workspace does not match");
    RSFK_CHECK(K >= 1 && K <= 256, "exploration join: K must be in 1..256");
    RSFK_CHECK((size_t)N * (size_t)K < ((size_t)1 << 31), "exploration join: N*K must be below 2^31");
    const size_t total = (size_t)N * (size_t)K;
    const int nb = w->n_blocks;
    const unsigned wide = (unsigned)std::min<size_t>((total + 255) / 256, 65536);
    hipLaunchKernelGGL(k_zero, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream, w->deg, N, w->todo + N, w->todo + 2 * (size_t)N + 1);
    hipLaunchKernelGGL(k_degree, dim3(wide), dim3(256), 0, stream, old_idx, total, N, w->deg);
    hipLaunchKernelGGL(k_scan_blocks, dim3((unsigned)nb), dim3(256), 0, stream, w->deg, N, w->offs, w->totals);
    hipLaunchKernelGGL(k_scan_totals, dim3(1), dim3(256), 0, stream, w->totals, nb, w->offs + N);
    hipLaunchKernelGGL(k_scan_add, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream, w->offs, N, w->totals);
    hipLaunchKernelGGL(k_fill_rev, dim3(wide), dim3(256), 0, stream, old_idx, total, N, K, w->deg, w->offs, w->rev,
                       w->fwd2rev);
    RSFK_HIP(hipGetLastError());

    constexpr int kWaves = 4;
    const int KP = (K + 31) & ~31;
    const int wave_ints = (KP + 96 + 3) & ~3;
    const size_t lds = (size_t)kWaves * (size_t)wave_ints * sizeof(int);
    const int ksteps = (bf16_valid(D) + 15) / 16;
    RSFK_CHECK(ksteps * 16 <= bf16_pitch(D), "exploration join: bfloat16 rows too short");
    const float kappa = (float)(ksteps * 16 + 16) * (1.0f / 2097152.0f);            // (Dp + 16) 2^-21
    const float one_minus_gamma = 1.0f - (float)(D + 8) * (1.0f / 4194304.0f);      // 1 - (D + 8) 2^-22
    RSFK_CHECK(one_minus_gamma > 0.5f, "exploration join: D too large");
    if (w->bounds)
        hipLaunchKernelGGL((k_explore_join<kWaves, true>), dim3((unsigned)((N + kWaves - 1) / kWaves)), dim3(64 * kWaves), lds,
                           stream, bf, N, K, old_idx, knn_dist, w->offs, w->rev, w->pass, w->bounds, KP, bf16_pitch(D), ksteps,
                           kappa, one_minus_gamma, wave_ints);
    else
        hipLaunchKernelGGL((k_explore_join<kWaves, false>), dim3((unsigned)((N + kWaves - 1) / kWaves)), dim3(64 * kWaves), lds,
                           stream, bf, N, K, old_idx, knn_dist, w->offs, w->rev, w->pass, w->bounds, KP, bf16_pitch(D), ksteps,
                           kappa, one_minus_gamma, wave_ints);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
