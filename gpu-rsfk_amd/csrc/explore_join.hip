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
// The outcome is one bit per (entry of the graph, neighbour slot): pass[p K + k] for the
// entry (p, k) = q has bit n set iff neighbour n of q may enter row p (an element of R(q)
// is the number p K + k of the entry, so the join knows where to write and the merge
// kernel of p reads its K words in one piece).  The exploration kernel of point p gathers
// the few ids whose bit is set (a few per cent), computes their exact distances and
// merges them.  Nothing is decided here that the exact arithmetic would decide
// otherwise; no atomics on shared counters, no buffer that can overflow.
//
// For the merge kernel that works through a point's candidates in the order of their
// bounds (explore.hip: rows with many candidates), L itself is kept for every marked
// pair, rounded down to a bfloat16 number (16 bits per pair of the join).
//
// Steps: R in compressed rows (counting sort of the graph entries by neighbour, see k_bin_count) -> join.
#include "rsfk_common.hpp"
#include "wave64.hpp"
#include "forest.hpp"
#include <algorithm>
#include <cstdlib>

namespace rsfk {

struct ExploreWorkspace {
    int N = 0, K = 0, MW = 0;  // MW = 32-bit words per entry of pass
    int shift = 0;             // a bin of the reversed-graph builder = 2^shift consecutive points
    int n_bins = 0;
    int n_parts = 0;           // workgroups of the two passes over the graph; each owns a contiguous range of entries
    int per_part = 0;          // entries per such range
    uint32_t div_m = 0;        // e / K == (div_m * e) >> div_s for 0 <= e < 2^31
    int div_s = 0;
    int* rev = nullptr;        // N*K: R lists in compressed rows; an element is the number p K + k of a graph entry
    int* offs = nullptr;       // N+1: start of R(q)
    int2* bin_eq = nullptr;    // N*K: (entry number, neighbour minus the first point of its bin), grouped by the bin of
                               // the neighbour; one 8-byte store per entry
    int* bin_size = nullptr;   // n_bins
    int* bin_start = nullptr;  // n_bins + 1
    int* part_off = nullptr;   // n_parts x n_bins: where the entries of a part start inside a bin
    uint32_t* pass = nullptr;  // N*K*MW, indexed by entry number
    float2* norm_tau = nullptr; // N: norm of the bfloat16 row and last slot of the K-NN row of a point, side by side
    uint16_t* bounds = nullptr; // N*K*32*MW lower bounds of the marked pairs (bfloat16, rounded down), or null
    // the builder for large graphs (staged_rev_*): two scatters through LDS instead of one straight to memory
    bool staged = false;
    int fshift = 0, cshift = 0; // fine bins of 2^fshift points (their rows are assembled in LDS), coarse bins of 2^cshift
    int n_fine = 0, n_coarse = 0;
    int n_sub = 0;              // sub-parts of the coarse bins at the second level (an upper bound)
    int2* bin_eq2 = nullptr;    // N*K: the records grouped by fine bin
    int* fine_size = nullptr;   // n_coarse << (cshift - fshift)
    int* fine_start = nullptr;  // the same + 1
    int* sub_off = nullptr;     // n_sub x fine bins per coarse bin
    int* todo = nullptr;       // two lists of N+1 ints: points left over by a launch; entry N = their number
    int* host_count = nullptr; // pinned
};
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr float kU = 1.0f / 256.0f;         // unit roundoff of bfloat16
constexpr int kMaxBins = 6144;
constexpr int kMaxShift = 13;
// entry numbers are ints, and the passes over the graph look 768 entries ahead of the one they test
constexpr size_t kMaxEntries = ((size_t)1 << 31) - 4096;
constexpr int kRowsBlock = 512;             // threads of k_bin_rows

// RSFK_JOIN_WG=0: the wavefront-per-q join also where the workgroup-per-q one applies.
bool join_wg_on()
{
    static const bool on = [] {
        const char* e = std::getenv("RSFK_JOIN_WG");
        return !(e && e[0] == '0');
    }();
    return on;
}

// Bins of the reversed-graph builder for N points: false if N is too large for it.
bool rev_bins(int N, int* shift, int* n_bins)
{
    // measured: small bins make the placement of k_bin_rows local (1M points: 0.25 ms with bins of 256 points, 0.62 ms
    // with 1024), many bins make the runs k_bin_scatter writes short (0.49 against 0.36 ms)
    int s = 8;
    if (const char* e = std::getenv("RSFK_REV_SHIFT")) s = std::max(8, std::min(kMaxShift, std::atoi(e)));
    while (s < kMaxShift && (((N - 1) >> s) + 1) > kMaxBins) ++s;
    *shift = s;
    *n_bins = N > 0 ? ((N - 1) >> s) + 1 : 1;
    return *n_bins <= kMaxBins;
}

__global__ void k_zero(int* a, int n, int* counter0, int* counter1)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) a[i] = 0;
    if (i == 0) { *counter0 = 0; *counter1 = 0; }
}

// exclusive scan of one value per thread over the workgroup (blockDim.x a multiple of 64, at most 1024); returns the
// total in *total.  lds: one int per wavefront.
__device__ __forceinline__ int block_excl_scan(int v, int* total, int* lds)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
    }
    if (lane == 63) lds[wave] = incl;
    __syncthreads();
    int woff = 0, tot = 0;
    for (int w = 0; w < waves; ++w) { const int x = lds[w]; if (w < wave) woff += x; tot += x; }
    __syncthreads();
    *total = tot;
    return woff + incl - v;
}

// The reversed graph R(q) = {entries (p, k) of the graph that hold q}, in compressed rows, without an atomic operation
// on device memory per entry (device-wide atomics are carried out at the memory side of the fabric, about 27 G of them
// a second: 2.8 ms for the 32 M entries of a 1 M x 32 graph, counting and placing).  Counting sort in two levels:
// the points are cut into bins of 2^shift, (1) every part of the graph counts its entries per bin in LDS and reserves
// its share of each bin with one atomic per bin, (2) the entries are moved to their bins -- entry number and neighbour
// minus the start of the bin -- (3) one workgroup per bin counts its neighbours in LDS, scans, writes the row offsets
// and places the entries.  The order of the entries inside R(q) is arbitrary; nothing downstream depends on it.
__global__ __launch_bounds__(256) void k_bin_count(const int* __restrict__ old_idx, int total, int per_part, int N, int shift,
                                                   int n_bins, int* __restrict__ bin_size, int* __restrict__ part_off)
{
    extern __shared__ int hist[];
    for (int b = threadIdx.x; b < n_bins; b += 256) hist[b] = 0;
    __syncthreads();
    const long long first = (long long)blockIdx.x * per_part;
    const int e0 = (int)min((long long)total, first), e1 = (int)min((long long)total, first + per_part);
    for (int e = e0 + (int)threadIdx.x; e < e1; e += 1024) {
        int q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) q[u] = e + 256 * u < e1 ? old_idx[e + 256 * u] : -1;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (q[u] >= 0 && q[u] < N) atomicAdd(&hist[q[u] >> shift], 1);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < n_bins; b += 256) {
        const int c = hist[b];
        part_off[(size_t)blockIdx.x * n_bins + b] = c ? atomicAdd(&bin_size[b], c) : 0;
    }
}

// bin_start = exclusive scan of bin_size (one workgroup); the number of valid entries goes to bin_start[n_bins] and *last
__global__ __launch_bounds__(256) void k_bin_scan(const int* __restrict__ bin_size, int n_bins, int* __restrict__ bin_start,
                                                  int* __restrict__ last)
{
    __shared__ int lds4[4];
    int carry = 0;
    for (int b0 = 0; b0 < n_bins; b0 += 256) {
        const int i = b0 + threadIdx.x;
        const int v = i < n_bins ? bin_size[i] : 0;
        int tot;
        const int ex = block_excl_scan(v, &tot, lds4);
        if (i < n_bins) bin_start[i] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0) { bin_start[n_bins] = carry; *last = carry; }
}

__global__ __launch_bounds__(256) void k_bin_scatter(const int* __restrict__ old_idx, int total, int per_part, int N, int shift,
                                                     int n_bins, const int* __restrict__ bin_start,
                                                     const int* __restrict__ part_off, int2* __restrict__ bin_eq)
{
    extern __shared__ int cursor[];
    for (int b = threadIdx.x; b < n_bins; b += 256) cursor[b] = bin_start[b] + part_off[(size_t)blockIdx.x * n_bins + b];
    __syncthreads();
    const int low = (1 << shift) - 1;
    const long long first = (long long)blockIdx.x * per_part;
    const int e0 = (int)min((long long)total, first), e1 = (int)min((long long)total, first + per_part);
    for (int e = e0 + (int)threadIdx.x; e < e1; e += 1024) {
        int q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) q[u] = e + 256 * u < e1 ? old_idx[e + 256 * u] : -1;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (q[u] >= 0 && q[u] < N) {
                const int at = atomicAdd(&cursor[q[u] >> shift], 1);
                bin_eq[at] = make_int2(e + 256 * u, q[u] & low);
            }
        }
    }
}

// One workgroup per bin.  LDS: one counter per point of the bin.
__global__ __launch_bounds__(kRowsBlock) void k_bin_rows(const int2* __restrict__ bin_eq,
                                                         const int* __restrict__ bin_start, int shift, int N,
                                                         int* __restrict__ offs, int* __restrict__ rev)
{
    extern __shared__ int cnt[];
    __shared__ int wave_lds[kRowsBlock / 64];
    const int R = 1 << shift;
    const int b = blockIdx.x;
    const int s0 = bin_start[b], s1 = bin_start[b + 1];
    const int q0 = b << shift;
    for (int i = threadIdx.x; i < R; i += kRowsBlock) cnt[i] = 0;
    __syncthreads();
    for (int i = s0 + (int)threadIdx.x; i < s1; i += kRowsBlock) atomicAdd(&cnt[bin_eq[i].y], 1);
    __syncthreads();
    int carry = 0;
    for (int c0 = 0; c0 < R; c0 += kRowsBlock) {
        const int c = c0 + (int)threadIdx.x;
        const bool in = c < R;                            // (a bin may have fewer points than the workgroup has threads)
        const int v = in ? cnt[c] : 0;
        int tot;
        const int ex = block_excl_scan(v, &tot, wave_lds);
        if (in) {
            cnt[c] = carry + ex;
            if (q0 + c < N) offs[q0 + c] = s0 + carry + ex;
        }
        carry += tot;
    }
    __syncthreads();
    for (int i = s0 + (int)threadIdx.x; i < s1; i += kRowsBlock) {
        const int2 eq = bin_eq[i];
        const int at = atomicAdd(&cnt[eq.y], 1);
        rev[s0 + at] = eq.x;
    }
}

// ---------------------------------------------------------------------------
// The same reversed graph for large inputs.  k_bin_scatter sends every record straight to one of several thousand
// bins and k_bin_rows every entry straight to its row: stores of 8 and 4 bytes whose cache lines leave the L2 long
// before their neighbours arrive (10 M x 32: 9.4 GB and 8.6 GB written for 2.56 GB and 1.28 GB of payload).  Here
// every store to memory is a run: (1) the records go to a few hundred coarse bins, a tile of 4096 at a time sorted by
// bin in LDS first, so a bin receives a run of records per tile; (2) inside a coarse bin the same again to its fine
// bins; (3) a fine bin is small enough for all of its rows to be assembled in LDS and written whole.  Counting comes
// before every scatter as in the one-level builder (no atomics on device memory per entry).  A record is
// (entry number, neighbour).
constexpr int kStTile = 4096;               // records sorted in LDS at a time
constexpr int kStSub = 32768;               // records of a sub-part of a coarse bin
constexpr int kStMaxBins = 1024;            // bins a scatter step distinguishes (LDS counters)
constexpr int kStRowsCap = 24576;           // entries of a fine bin whose rows are assembled in LDS

// (The counts of the parts of the graph per coarse bin are k_bin_count and k_bin_scan with shift = cshift.)

// Sorts up to kStTile records (rec[i], bin[i] for the thread's 16 records) by bin in LDS and writes them to
// out[cursor[bin] + rank inside (tile, bin)]; cursor (LDS, n_bins ints) moves on by the tile's counts.
// LDS: cnt[n_bins] | first[n_bins] | stage[kStTile] (int2).
__device__ __forceinline__ void staged_tile_out(const int2 (&rec)[16], const int (&bin)[16], int n_bins, int* cnt, int* first,
                                                int2* stage, unsigned short* sbin, int* cursor, int* wave_lds,
                                                int2* __restrict__ out)
{
    const int tid = threadIdx.x;
    for (int b = tid; b < n_bins; b += 256) cnt[b] = 0;
    __syncthreads();
    int rank[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) rank[u] = bin[u] >= 0 ? atomicAdd(&cnt[bin[u]], 1) : 0;
    __syncthreads();
    // exclusive scan of the counts (n_bins <= 1024: four per thread)
    {
        int v[4], sum = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) { const int b = 4 * tid + j; v[j] = b < n_bins ? cnt[b] : 0; sum += v[j]; }
        int tot;
        int ex = block_excl_scan(sum, &tot, wave_lds);
#pragma unroll
        for (int j = 0; j < 4; ++j) { const int b = 4 * tid + j; if (b < n_bins) first[b] = ex; ex += v[j]; }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        if (bin[u] >= 0) {
            const int at = first[bin[u]] + rank[u];
            stage[at] = rec[u];
            sbin[at] = (unsigned short)bin[u];
        }
    }
    __syncthreads();
    const int n_tile = first[n_bins - 1] + cnt[n_bins - 1];
    for (int i = tid; i < n_tile; i += 256) {
        const int b = sbin[i];
        out[(size_t)cursor[b] + (size_t)(i - first[b])] = stage[i];
    }
    __syncthreads();
    for (int b = tid; b < n_bins; b += 256) cursor[b] += cnt[b];
    __syncthreads();
}

constexpr size_t staged_lds_bytes(int n_bins)
{
    return (size_t)3 * n_bins * sizeof(int) + 8 + (size_t)kStTile * (sizeof(int2) + sizeof(unsigned short));
}

// (1) a part of the graph to the coarse bins.  part_off / bin_start as left by k_bin_count / k_bin_scan at shift = cshift.
__global__ __launch_bounds__(256) void k_staged_scatter1(const int* __restrict__ old_idx, int total, int per_part, int N, int cshift,
                                                         int n_coarse, const int* __restrict__ bin_start,
                                                         const int* __restrict__ part_off, int2* __restrict__ out)
{
    extern __shared__ __align__(16) int lds_st[];
    __shared__ int wave_lds[4];
    int* cursor = lds_st;
    int* cnt = cursor + n_coarse;
    int* first = cnt + n_coarse;
    int2* stage = reinterpret_cast<int2*>(first + n_coarse + (n_coarse & 1));
    unsigned short* sbin = reinterpret_cast<unsigned short*>(stage + kStTile);
    for (int b = threadIdx.x; b < n_coarse; b += 256) cursor[b] = bin_start[b] + part_off[(size_t)blockIdx.x * n_coarse + b];
    __syncthreads();
    const long long begin = (long long)blockIdx.x * per_part;
    const int e0 = (int)min((long long)total, begin), e1 = (int)min((long long)total, begin + per_part);
    for (int t0 = e0; t0 < e1; t0 += kStTile) {
        int2 rec[16];
        int bin[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int e = t0 + 256 * u + (int)threadIdx.x;
            const int q = e < e1 ? old_idx[e] : -1;
            const bool ok = q >= 0 && q < N;
            rec[u] = make_int2(e, q);
            bin[u] = ok ? q >> cshift : -1;
        }
        staged_tile_out(rec, bin, n_coarse, cnt, first, stage, sbin, cursor, wave_lds, out);
    }
}

// Sub-parts of coarse bin cb: records [start + s kStSub, ...) for s = 0, 1, ...; their number in the global list of
// sub-parts is start / kStSub + cb + s (increasing, no two alike: a coarse bin has at most size / kStSub + 1 of them).
__device__ __forceinline__ int staged_sub_id(int start, int cb, int s) { return start / kStSub + cb + s; }

// (2a) counts of the sub-parts of the coarse bins per fine bin; grid (x: sub-parts walked in turn, y: coarse bin)
__global__ __launch_bounds__(256) void k_staged_count2(const int2* __restrict__ rec1, const int* __restrict__ cstart, int cshift,
                                                       int fshift, int* __restrict__ fine_size, int* __restrict__ sub_off)
{
    extern __shared__ int hist2[];
    const int per = 1 << (cshift - fshift);
    const int cb = blockIdx.y;
    const int s0 = cstart[cb], s1 = cstart[cb + 1];
    const int low = (1 << cshift) - 1;
    for (int s = blockIdx.x; s0 + (long long)s * kStSub < s1; s += gridDim.x) {
        for (int b = threadIdx.x; b < per; b += 256) hist2[b] = 0;
        __syncthreads();
        const int a = s0 + s * kStSub, z = min(s1, a + kStSub);
        for (int i = a + (int)threadIdx.x; i < z; i += 256) atomicAdd(&hist2[(rec1[i].y & low) >> fshift], 1);
        __syncthreads();
        const size_t row = (size_t)staged_sub_id(s0, cb, s) * per;
        for (int b = threadIdx.x; b < per; b += 256) {
            const int c = hist2[b];
            sub_off[row + b] = c ? atomicAdd(&fine_size[(size_t)cb * per + b], c) : 0;
        }
        __syncthreads();
    }
}

// (2b) the records of the sub-parts to their fine bins
__global__ __launch_bounds__(256) void k_staged_scatter2(const int2* __restrict__ rec1, const int* __restrict__ cstart, int cshift,
                                                         int fshift, const int* __restrict__ fine_start,
                                                         const int* __restrict__ sub_off, int2* __restrict__ out)
{
    extern __shared__ __align__(16) int lds_st[];
    __shared__ int wave_lds[4];
    const int per = 1 << (cshift - fshift);
    int* cursor = lds_st;
    int* cnt = cursor + per;
    int* first = cnt + per;
    int2* stage = reinterpret_cast<int2*>(first + per + (per & 1));
    unsigned short* sbin = reinterpret_cast<unsigned short*>(stage + kStTile);
    const int cb = blockIdx.y;
    const int s0 = cstart[cb], s1 = cstart[cb + 1];
    const int low = (1 << cshift) - 1;
    for (int s = blockIdx.x; s0 + (long long)s * kStSub < s1; s += gridDim.x) {
        const size_t row = (size_t)staged_sub_id(s0, cb, s) * per;
        for (int b = threadIdx.x; b < per; b += 256) cursor[b] = fine_start[(size_t)cb * per + b] + sub_off[row + b];
        __syncthreads();
        const int a = s0 + s * kStSub, z = min(s1, a + kStSub);
        for (int t0 = a; t0 < z; t0 += kStTile) {
            int2 rec[16];
            int bin[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int i = t0 + 256 * u + (int)threadIdx.x;
                rec[u] = i < z ? rec1[i] : make_int2(-1, -1);
                bin[u] = i < z ? (rec[u].y & low) >> fshift : -1;
            }
            staged_tile_out(rec, bin, per, cnt, first, stage, sbin, cursor, wave_lds, out);
        }
        __syncthreads();
    }
}

// (3) one workgroup per fine bin: row offsets of its points, and its rows -- assembled in LDS and written whole when the
// bin has at most kStRowsCap entries, entry by entry otherwise.  LDS: cnt[2^fshift] | stage[kStRowsCap].
__global__ __launch_bounds__(kRowsBlock) void k_staged_rows(const int2* __restrict__ rec2, const int* __restrict__ fine_start,
                                                            int fshift, int N, int* __restrict__ offs, int* __restrict__ rev)
{
    extern __shared__ int lds_rows[];
    __shared__ int wave_lds[kRowsBlock / 64];
    const int R = 1 << fshift;
    int* cnt = lds_rows;
    int* stage = cnt + R;
    const int b = blockIdx.x;
    const int s0 = fine_start[b], s1 = fine_start[b + 1];
    const int q0 = b << fshift;
    const int low = R - 1;
    for (int i = threadIdx.x; i < R; i += kRowsBlock) cnt[i] = 0;
    __syncthreads();
    for (int i = s0 + (int)threadIdx.x; i < s1; i += kRowsBlock) atomicAdd(&cnt[rec2[i].y & low], 1);
    __syncthreads();
    int carry = 0;
    for (int c0 = 0; c0 < R; c0 += kRowsBlock) {
        const int c = c0 + (int)threadIdx.x;
        const bool in = c < R;
        const int v = in ? cnt[c] : 0;
        int tot;
        const int ex = block_excl_scan(v, &tot, wave_lds);
        if (in) {
            cnt[c] = carry + ex;
            if (q0 + c < N) offs[q0 + c] = s0 + carry + ex;
        }
        carry += tot;
    }
    __syncthreads();
    const bool in_lds = s1 - s0 <= kStRowsCap;
    for (int i = s0 + (int)threadIdx.x; i < s1; i += kRowsBlock) {
        const int2 eq = rec2[i];
        const int at = atomicAdd(&cnt[eq.y & low], 1);
        if (in_lds) stage[at] = eq.x;
        else rev[s0 + at] = eq.x;
    }
    if (in_lds) {
        __syncthreads();
        for (int i = threadIdx.x; i < s1 - s0; i += kRowsBlock) rev[s0 + i] = stage[i];
    }
}

// What the join needs of a point besides its row, in one 8-byte record (one gather instead of two).
__global__ void k_norm_tau(const float* __restrict__ norms, const float* __restrict__ knn_dist, int N, int K,
                           float2* __restrict__ out)
{
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p < N) out[p] = make_float2(norms[p], knn_dist[(size_t)p * K + (K - 1)]);
}

// One wavefront per q.  Per-wavefront LDS (ints): cq[KP] | pid[32] | pn[32] | ptau[32] | pe[32], KP = K rounded up to 32.
template <int WAVES, bool BOUNDS>
__global__ __launch_bounds__(64 * WAVES) void k_explore_join(Bf16Copy bf, int N, int K, const int* __restrict__ old_idx,
                                                              const float2* __restrict__ norm_tau,
                                                              const int* __restrict__ offs, const int* __restrict__ rev,
                                                              uint32_t* __restrict__ pass, uint16_t* __restrict__ bounds, int KP, int bpitch, int ksteps,
                                                              float kappa, float one_minus_gamma, int wave_lds_ints,
                                                              uint32_t div_m, int div_s, const int* __restrict__ order)
{
    extern __shared__ __align__(16) int lds_join[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int item = die_local_place(blockIdx.x, gridDim.x) * WAVES + wave;
    if (item >= N) return;                                // whole wavefront leaves together
    const int q = order ? order[item] : item;
    const int r0 = offs[q], R = offs[q + 1] - r0;
    if (R <= 0) return;
    int* cq = lds_join + (size_t)wave * (size_t)wave_lds_ints;
    int* pid = cq + KP;
    float* pn = reinterpret_cast<float*>(pid + 32);
    float* ptau = pn + 32;
    int* pe = reinterpret_cast<int*>(ptau + 32);
    const int MW = KP >> 5;

    for (int k = lane; k < KP; k += 64) {
        int c = k < K ? old_idx[(size_t)q * K + k] : -1;
        if (c < 0 || c >= N) c = -1;
        cq[k] = c;
    }

    for (int pt0 = 0; pt0 < R; pt0 += 32) {
        const int np = min(32, R - pt0);
        wave_lds_sync();                                  // reads of the previous tile are done (and cq is written)
        int my_e = -1;                                    // lanes 0..31: the graph entry (p, k) with q = neighbour k of p
        if (lane < 32) {
            my_e = lane < np ? rev[(size_t)r0 + pt0 + lane] : -1;
            const int p = my_e >= 0 ? (int)(((uint64_t)div_m * (uint64_t)(uint32_t)my_e) >> div_s) : -1;
            pid[lane] = p;
            pe[lane] = my_e;
            const float2 nt = p >= 0 ? norm_tau[p] : make_float2(0.0f, 0.0f);
            pn[lane] = nt.x;
            ptau[lane] = nt.y;
        }
        wave_lds_sync();

        const int pm = pid[lane & 31];
        const uint16_t* ra = bf.rows + (size_t)(pm >= 0 ? pm : q) * (size_t)bpitch + 8 * (lane >> 5);
        const int mbase = 4 * (lane >> 5);
        for (int ct = 0; ct < MW; ++ct) {
            const int cid = cq[ct * 32 + (lane & 31)];
            const uint16_t* rb = bf.rows + (size_t)(cid >= 0 ? cid : q) * (size_t)bpitch + 8 * (lane >> 5);
            const float cn = cid >= 0 ? norm_tau[cid].x : 0.0f;
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
                    bounds[(size_t)pe[m] * (size_t)KP + ct * 32 + (lane & 31)] = (uint16_t)lb;
                }
                const int m_lo = 8 * (i >> 2) + (i & 3);
                if (lane == m_lo) mine = (uint32_t)bm;
                if (lane == m_lo + 4) mine = (uint32_t)(bm >> 32);
            }
            if (lane < np) pass[(size_t)my_e * MW + ct] = mine;
        }
    }
}

// The join for rows of at most 32 neighbours and points of at most 128 dimensions (KS = steps of 16 dimensions, fixed
// at compile time: 2, 4 or 8).  One word of marks per graph entry; the rows of the neighbours of q are loaded once
// and stay in registers for all tiles of R(q); the norm and last slot of the points of a tile travel while their rows
// are fetched.  A wavefront then has three dependent trips to memory per q (row offsets and neighbours | their rows
// and the elements of R(q) | the rows of those points) instead of five, and short rows leave room for twice the
// wavefronts per SIMD.  The bound is that of k_explore_join, term by term.
template <int WAVES, int KS>
__global__ __launch_bounds__(64 * WAVES) void k_explore_join_short(Bf16Copy bf, int N, int K, const int* __restrict__ old_idx,
                                                                    const float2* __restrict__ norm_tau,
                                                                    const int* __restrict__ offs, const int* __restrict__ rev,
                                                                    uint32_t* __restrict__ pass, int bpitch, int ksteps,
                                                                    float kappa, float one_minus_gamma, uint32_t div_m, int div_s,
                                                                    const int* __restrict__ order)
{
    __shared__ int pid_s[WAVES][32];
    __shared__ float pn_s[WAVES][32], ptau_s[WAVES][32];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int item = die_local_place(blockIdx.x, gridDim.x) * WAVES + wave;
    if (item >= N) return;                                // whole wavefront leaves together
    const int q = order ? order[item] : item;
    const int r0 = offs[q], R = offs[q + 1] - r0;
    const int col = lane & 31, hi = lane >> 5;
    int cid = col < K ? old_idx[(size_t)q * K + col] : -1;
    if (R <= 0) return;
    if (cid < 0 || cid >= N) cid = -1;
    const uint16_t* rb = bf.rows + (size_t)(cid >= 0 ? cid : q) * (size_t)bpitch + 8 * hi;
    bf16x8 b[KS];
#pragma unroll
    for (int u = 0; u < KS; ++u) {
#pragma unroll
        for (int i = 0; i < 8; ++i) b[u][i] = (__bf16)0.0f;
        if (u < ksteps) b[u] = *reinterpret_cast<const bf16x8*>(rb + 16 * u);
    }
    const float cn = cid >= 0 ? norm_tau[cid].x : 0.0f;
    const int mbase = 4 * hi;
    int* pid = pid_s[wave];
    float* pn = pn_s[wave];
    float* ptau = ptau_s[wave];

    for (int pt0 = 0; pt0 < R; pt0 += 32) {
        const int np = min(32, R - pt0);
        int my_e = -1;                                    // lanes 0..31: the graph entry (p, k) with q = neighbour k of p
        float2 nt = make_float2(0.0f, 0.0f);
        if (lane < 32) {
            my_e = lane < np ? rev[(size_t)r0 + pt0 + lane] : -1;
            const int p = my_e >= 0 ? (int)(((uint64_t)div_m * (uint64_t)(uint32_t)my_e) >> div_s) : -1;
            pid[lane] = p;
            if (p >= 0) nt = norm_tau[p];
        }
        wave_lds_sync();
        const int pm = pid[col];
        const uint16_t* ra = bf.rows + (size_t)(pm >= 0 ? pm : q) * (size_t)bpitch + 8 * hi;
        bf16x8 a[KS];
#pragma unroll
        for (int u = 0; u < KS; ++u) {
#pragma unroll
            for (int i = 0; i < 8; ++i) a[u][i] = (__bf16)0.0f;
            if (u < ksteps) a[u] = *reinterpret_cast<const bf16x8*>(ra + 16 * u);
        }
        f32x16 g;
#pragma unroll
        for (int i = 0; i < 16; ++i) g[i] = 0.0f;
#pragma unroll
        for (int u = 0; u < KS; ++u) g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u], b[u], g, 0, 0, 0);
        if (lane < 32) {
            pn[lane] = nt.x;
            ptau[lane] = nt.y;
        }
        wave_lds_sync();
        // Accumulator i of lane l: point m = 4 (l / 32) + 8 (i / 4) + i % 4 of the tile, column = neighbour l % 32.
        uint32_t mine = 0;                                // mask of the point this lane stores (lanes 0..31)
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
            const bool skip = lower > ptau[m];            // false if anything is NaN; a tie at the last slot may still enter
            const uint64_t bm = ballot64(cid >= 0 && !skip);
            const int m_lo = 8 * (i >> 2) + (i & 3);
            if (lane == m_lo) mine = (uint32_t)bm;
            if (lane == m_lo + 4) mine = (uint32_t)(bm >> 32);
            if ((i & 3) == 3) __builtin_amdgcn_sched_barrier(0);   // four at a time: all sixteen at once take too many registers
        }
        if (lane < np) pass[(size_t)my_e] = mine;
        wave_lds_sync();                                  // the tile's LDS values are read before the next tile writes them
    }
}

// The join with one workgroup (four wavefronts) per q, for rows of more than 32 neighbours.  k_explore_join loads the rows of a tile of R(q) again for every group of 32 neighbours and the rows of
// the neighbours again for every tile of R(q): at K = 90 (three groups, three tiles) every row three times.  Here 96
// points of R(q) and all neighbours of q pass through LDS together, 64 dimensions at a time (the next 64 are requested
// while these are used), and the wavefronts share the pairs (tile of R(q), group of neighbours) among them, each
// keeping the accumulators of its pairs: every row is read once per 96 points of R(q).  Bound and outputs are those
// of k_explore_join.  NPW = pairs per wavefront (3: K <= 128, 6: K <= 256).
constexpr int kJwP = 96;                    // points of R(q) worked on together (three tiles)
constexpr int kJwRowBytes = 144;            // 64 bfloat16 values + 16 bytes: rows start in different banks

template <bool BOUNDS, int NPW>
__global__ __launch_bounds__(256) void k_explore_join_wg(Bf16Copy bf, int N, int K, const int* __restrict__ old_idx,
                                                         const float2* __restrict__ norm_tau, const int* __restrict__ offs,
                                                         const int* __restrict__ rev, uint32_t* __restrict__ pass,
                                                         uint16_t* __restrict__ bounds, int KP, int bpitch, int ksteps,
                                                         float kappa, float one_minus_gamma, uint32_t div_m, int div_s,
                                                         const int* __restrict__ order)
{
    constexpr int kPieces = (kJwP + (NPW == 3 ? 128 : 256)) * 8 / 256;      // 16-byte pieces a thread stages per step
    extern __shared__ __align__(16) unsigned char lds_jw[];
    unsigned char* rowsb = lds_jw;                                         // kJwP + KP rows of 144 bytes
    int* cq = reinterpret_cast<int*>(rowsb + (size_t)(kJwP + KP) * kJwRowBytes);
    float* cn = reinterpret_cast<float*>(cq + KP);
    int* pid = reinterpret_cast<int*>(cn + KP);
    int* pe = pid + kJwP;
    float* pn = reinterpret_cast<float*>(pe + kJwP);
    float* ptau = pn + kJwP;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, h = lane >> 5;
    const int item = die_local_place(blockIdx.x, gridDim.x);
    if (item >= N) return;                                                 // the whole workgroup leaves together
    const int q = order ? order[item] : item;
    const int r0 = offs[q], R = offs[q + 1] - r0;
    if (R <= 0) return;
    const int MW = KP >> 5;
    const int nrows = kJwP + KP;
    for (int k = tid; k < KP; k += 256) {
        int c = k < K ? old_idx[(size_t)q * K + k] : -1;
        if (c < 0 || c >= N) c = -1;
        cq[k] = c;
        cn[k] = c >= 0 ? norm_tau[c].x : 0.0f;
    }
    for (int pg = 0; pg < R; pg += kJwP) {
        const int npg = min(kJwP, R - pg);
        const int npairs = ((npg + 31) >> 5) * MW;
        __syncthreads();                                                   // the previous group is done with the LDS
        if (tid < kJwP) {
            const int e = tid < npg ? rev[(size_t)r0 + pg + tid] : -1;
            const int p = e >= 0 ? (int)(((uint64_t)div_m * (uint64_t)(uint32_t)e) >> div_s) : -1;
            const float2 nt = p >= 0 ? norm_tau[p] : make_float2(0.0f, 0.0f);
            pid[tid] = p;
            pe[tid] = e;
            pn[tid] = nt.x;
            ptau[tid] = nt.y;
        }
        __syncthreads();
        f32x16 acc[NPW];
#pragma unroll
        for (int i = 0; i < NPW; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[i][j] = 0.0f;
        // pieces this thread stages: piece i = tid + 256 j of the (row, 16-byte piece) grid
        uint4 pre[kPieces];
        auto request = [&](int c0) {
#pragma unroll
            for (int j = 0; j < kPieces; ++j) {
                const int i = tid + 256 * j;
                pre[j] = make_uint4(0u, 0u, 0u, 0u);
                if (i < nrows * 8) {
                    const int r = i >> 3, pc = i & 7;
                    const int id = r < kJwP ? pid[r] : cq[r - kJwP];
                    const int el = c0 * 16 + pc * 8;
                    if (id >= 0 && el < ksteps * 16)
                        pre[j] = *reinterpret_cast<const uint4*>(bf.rows + (size_t)id * (size_t)bpitch + el);
                }
            }
        };
        request(0);
        for (int c0 = 0; c0 < ksteps; c0 += 4) {
            if (c0 > 0) __syncthreads();                                   // the previous step's values have been used
#pragma unroll
            for (int j = 0; j < kPieces; ++j) {
                const int i = tid + 256 * j;
                if (i < nrows * 8) *reinterpret_cast<uint4*>(rowsb + (size_t)(i >> 3) * kJwRowBytes + (i & 7) * 16) = pre[j];
            }
            __syncthreads();
            if (c0 + 4 < ksteps) request(c0 + 4);
#pragma unroll
            for (int i = 0; i < NPW; ++i) {
                const int pair = wave + 4 * i;
                if (pair < npairs) {
                    const int pt = pair / MW, ct = pair - pt * MW;
                    const unsigned char* ra = rowsb + (size_t)(pt * 32 + n) * kJwRowBytes + h * 16;
                    const unsigned char* rb = rowsb + (size_t)(kJwP + ct * 32 + n) * kJwRowBytes + h * 16;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (c0 + u < ksteps) {
                            const bf16x8 a = *reinterpret_cast<const bf16x8*>(ra + 32 * u);
                            const bf16x8 b = *reinterpret_cast<const bf16x8*>(rb + 32 * u);
                            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);                         // one pair after the other (registers)
            }
        }
        // Accumulator j of lane l: point 4 (l / 32) + 8 (j / 4) + j % 4 of the tile, column = neighbour l % 32 of the group.
#pragma unroll
        for (int i = 0; i < NPW; ++i) {
            const int pair = wave + 4 * i;
            if (pair < npairs) {
                const int pt = pair / MW, ct = pair - pt * MW;
                const int col = ct * 32 + n;
                const int cid = cq[col];
                const float cnv = cn[col];
                uint32_t mine = 0;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int m = pt * 32 + 4 * h + 8 * (j >> 2) + (j & 3);
                    const float S = pn[m] + cnv;
                    const float dt = __builtin_fmaf(-2.0f, acc[i][j], S);
                    const float e1 = kappa * S;
                    const float dhi = fmaxf(dt + e1, 0.0f);
                    const float Q = 2.0001f * S;
                    const float ebf = 1.01f * (2.0f * kU * __builtin_sqrtf(dhi * Q) + kU * kU * Q);
                    const float lower = (dt - e1 - ebf) * one_minus_gamma - 1e-30f;
                    const bool skip = lower > ptau[m];            // false if anything is NaN; a tie at the last slot may still enter
                    const bool marked = cid >= 0 && !skip;
                    const uint64_t bm = ballot64(marked);
                    if (BOUNDS && marked && m < npg) {
                        // a bound below zero (or NaN) says nothing: 0.  Dropping the low half of a positive float rounds down.
                        const uint32_t lb = lower > 0.0f ? __float_as_uint(lower) >> 16 : 0u;
                        bounds[(size_t)pe[m] * (size_t)KP + col] = (uint16_t)lb;
                    }
                    const int m_lo = 8 * (j >> 2) + (j & 3);
                    if (lane == m_lo) mine = (uint32_t)bm;
                    if (lane == m_lo + 4) mine = (uint32_t)(bm >> 32);
                    if ((j & 3) == 3) __builtin_amdgcn_sched_barrier(0);   // four at a time (registers)
                }
                if (lane < 32 && pt * 32 + lane < npg) pass[(size_t)pe[pt * 32 + lane] * MW + ct] = mine;
            }
        }
    }
}

}  // namespace

// The join is used unless RSFK_EXPLORE_JOIN=0 is set, K is above 256, the graph has about 2^31 or more entries or N is beyond what the
// builder of the reversed graph takes (6144 bins of 2^13 points).
bool explore_join_enabled(int N, int K)
{
    const char* env = std::getenv("RSFK_EXPLORE_JOIN");
    if (env && env[0] == '0') return false;
    if (K > kMaxKJoin) return false;          // (rows of more than 256 neighbours: the general kernel only)
    int shift, n_bins;
    return (size_t)N * (size_t)K < kMaxEntries && rev_bins(N, &shift, &n_bins);
}

size_t explore_ws_bytes(int N, int K)
{
    const size_t mw = (size_t)((K + 31) / 32);
    return (size_t)N * ((size_t)K * (12 + 4 * mw) + 32) + ((size_t)20 << 20);
}

int explore_ws_alloc(ExploreWorkspace** out, int N, int K, bool with_bounds)
{
    *out = nullptr;
    auto* w = new ExploreWorkspace();
    w->N = N;
    w->K = K;
    w->MW = (K + 31) / 32;
    if (!rev_bins(N, &w->shift, &w->n_bins) || (size_t)N * (size_t)K >= kMaxEntries) {
        delete w;
        set_last_error("exploration workspace: graph too large for the join");
        return 1;
    }
    const size_t total = (size_t)N * (size_t)K;
    w->n_parts = (int)std::min<size_t>(512, std::max<size_t>(1, (total + 8191) / 8192));
    w->per_part = (int)(((total + w->n_parts - 1) / w->n_parts + 1023) / 1024 * 1024);
    int l = 0;
    while ((1 << l) < K) ++l;
    w->div_s = 31 + l;
    w->div_m = (uint32_t)((((uint64_t)1 << w->div_s) + (uint64_t)K - 1) / (uint64_t)K);
    auto dm = [](void* p, size_t n) { return ws_alloc(reinterpret_cast<void**>(p), std::max<size_t>(n, 1) * sizeof(int)) ? hipErrorOutOfMemory : hipSuccess; };
    // Large graphs (2^26 entries and more; RSFK_REV_STAGED=1|0 says otherwise) take the builder that stages its stores
    // in LDS: fine bins whose rows fit into LDS with room to spare, about as many fine bins per coarse bin as there
    // are coarse bins.
    {
        const char* e = std::getenv("RSFK_REV_STAGED");
        bool want = total >= ((size_t)1 << 26);
        if (e && e[0] == '1') want = true;
        if (e && e[0] == '0') want = false;
        if (want) {
            int fs = 5;
            while (fs < 12 && ((size_t)3 << (fs + 1)) * (size_t)K <= (size_t)2 * kStRowsCap) ++fs;    // 1.5 K 2^fs <= cap
            const int n_fine = (int)(((size_t)N + ((size_t)1 << fs) - 1) >> fs);
            int lp = 4;
            while (lp < 10 && ((size_t)1 << (2 * (lp + 1))) <= (size_t)n_fine) ++lp;                   // 2^lp about sqrt(n_fine)
            while (lp < 10 && (((size_t)N - 1) >> (fs + lp)) + 1 > (size_t)kStMaxBins) ++lp;
            const int n_coarse = (int)((((size_t)N - 1) >> (fs + lp)) + 1);
            // (the parts' counters and the bins' sizes and starts are the arrays of the one-level builder)
            if (n_coarse <= kStMaxBins && n_coarse <= w->n_bins) {
                w->staged = true;
                w->fshift = fs;
                w->cshift = fs + lp;
                w->n_coarse = n_coarse;
                w->n_fine = n_coarse << lp;
                w->n_sub = (int)(total / kStSub) + n_coarse + 2;
            }
        }
    }
    if (w->staged &&
        (dm(&w->bin_eq2, 2 * total) != hipSuccess || dm(&w->fine_size, (size_t)w->n_fine) != hipSuccess ||
         dm(&w->fine_start, (size_t)w->n_fine + 1) != hipSuccess ||
         dm(&w->sub_off, (size_t)w->n_sub << (w->cshift - w->fshift)) != hipSuccess)) {
        explore_ws_free(w);
        set_last_error("exploration workspace: out of device memory");
        return 1;
    }
    if (dm(&w->rev, total) != hipSuccess || dm(&w->bin_eq, 2 * total) != hipSuccess ||
        dm(&w->offs, (size_t)N + 1) != hipSuccess || dm(&w->bin_size, (size_t)w->n_bins) != hipSuccess ||
        dm(&w->bin_start, (size_t)w->n_bins + 1) != hipSuccess ||
        dm(&w->part_off, (size_t)w->n_parts * (size_t)w->n_bins) != hipSuccess || dm(&w->pass, total * w->MW) != hipSuccess || dm(&w->norm_tau, 2 * (size_t)N) != hipSuccess ||
        dm(&w->todo, 2 * ((size_t)N + 1)) != hipSuccess ||
        hipHostMalloc(reinterpret_cast<void**>(&w->host_count), sizeof(int)) != hipSuccess) {
        explore_ws_free(w);
        set_last_error("exploration workspace: out of device memory");
        return 1;
    }
    if (with_bounds) {
        // 2 bytes per pair of the join; without them the merge still works, in the order of the marks.  The array grows
        // with N K^2 (17 GB at N = 1M, K = 90): it is only asked for up to 16 GiB, and as a block the call can do
        // without (no idle block is given up for it, a refusal leaves no error text behind)
        const size_t bytes = total * w->MW * 32 * sizeof(uint16_t);
        void* b = nullptr;
        if (bytes <= ((size_t)16 << 30) && ws_try_alloc(&b, bytes) == 0) w->bounds = static_cast<uint16_t*>(b);
    }
    *out = w;
    return 0;
}

void explore_ws_free(ExploreWorkspace* w)
{
    if (!w) return;
    void* bufs[] = {w->rev, w->bin_eq, w->offs, w->bin_size, w->bin_start, w->part_off, w->pass, w->norm_tau, w->todo, w->bounds,
                    w->bin_eq2, w->fine_size, w->fine_start, w->sub_off};
    for (void* b : bufs)
        ws_free(b);
    if (w->host_count) (void)hipHostFree(w->host_count);
    delete w;
}

const uint32_t* explore_ws_pass(const ExploreWorkspace* w) { return w->pass; }
const uint16_t* explore_ws_bounds(const ExploreWorkspace* w) { return w->bounds; }
int* explore_ws_todo(ExploreWorkspace* w, int which) { return w->todo + (size_t)which * ((size_t)w->N + 1); }
int* explore_ws_host_count(ExploreWorkspace* w) { return w->host_count; }

// Fill pass (and bounds) from the snapshot old_idx and the current last slots of knn_dist (rows sorted by distance).
int launch_explore_join(ExploreWorkspace* w, const Bf16Copy& bf, int N, int D, int K, const int* old_idx,
                        const float* knn_dist, hipStream_t stream, const int* order)
{
    RSFK_CHECK(w && w->N == N && w->K == K, "exploration join: workspace does not match");
    RSFK_CHECK(K >= 1 && K <= 256, "exploration join: K must be in 1..256");
    RSFK_CHECK((size_t)N * (size_t)K < kMaxEntries, "exploration join: N*K must be below 2^31 - 4096");
    const int total = (int)((size_t)N * (size_t)K);
    if (w->staged) {
        const int nc = w->n_coarse, per = 1 << (w->cshift - w->fshift);
        hipLaunchKernelGGL(k_zero, dim3((unsigned)((nc + 255) / 256)), dim3(256), 0, stream, w->bin_size, nc, w->todo + N,
                           w->todo + 2 * (size_t)N + 1);
        hipLaunchKernelGGL(k_zero, dim3((unsigned)((w->n_fine + 255) / 256)), dim3(256), 0, stream, w->fine_size, w->n_fine,
                           w->todo + N, w->todo + 2 * (size_t)N + 1);
        hipLaunchKernelGGL(k_bin_count, dim3((unsigned)w->n_parts), dim3(256), (size_t)nc * sizeof(int), stream, old_idx, total,
                           w->per_part, N, w->cshift, nc, w->bin_size, w->part_off);
        hipLaunchKernelGGL(k_bin_scan, dim3(1), dim3(256), 0, stream, w->bin_size, nc, w->bin_start, w->offs + N);
        hipLaunchKernelGGL(k_staged_scatter1, dim3((unsigned)w->n_parts), dim3(256), staged_lds_bytes(nc), stream, old_idx, total,
                           w->per_part, N, w->cshift, nc, w->bin_start, w->part_off, w->bin_eq);
        // sub-parts of a coarse bin walked by a few workgroups each (four times the mean number of sub-parts per bin)
        const unsigned walkers = (unsigned)std::max<size_t>(1, std::min<size_t>(64, 4 * ((size_t)total / kStSub / (size_t)nc + 1)));
        hipLaunchKernelGGL(k_staged_count2, dim3(walkers, (unsigned)nc), dim3(256), (size_t)per * sizeof(int), stream, w->bin_eq,
                           w->bin_start, w->cshift, w->fshift, w->fine_size, w->sub_off);
        hipLaunchKernelGGL(k_bin_scan, dim3(1), dim3(256), 0, stream, w->fine_size, w->n_fine, w->fine_start, w->offs + N);
        hipLaunchKernelGGL(k_staged_scatter2, dim3(walkers, (unsigned)nc), dim3(256), staged_lds_bytes(per), stream, w->bin_eq,
                           w->bin_start, w->cshift, w->fshift, w->fine_start, w->sub_off, w->bin_eq2);
        const size_t rows_lds = ((size_t)(1 << w->fshift) + kStRowsCap) * sizeof(int);
        RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_staged_rows), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)rows_lds));
        hipLaunchKernelGGL(k_staged_rows, dim3((unsigned)w->n_fine), dim3(kRowsBlock), rows_lds, stream, w->bin_eq2, w->fine_start,
                           w->fshift, N, w->offs, w->rev);
    } else {
    const int nbins = w->n_bins;
    const size_t bin_lds = (size_t)nbins * sizeof(int);
    hipLaunchKernelGGL(k_zero, dim3((unsigned)((nbins + 255) / 256)), dim3(256), 0, stream, w->bin_size, nbins, w->todo + N,
                       w->todo + 2 * (size_t)N + 1);
    hipLaunchKernelGGL(k_bin_count, dim3((unsigned)w->n_parts), dim3(256), bin_lds, stream, old_idx, total, w->per_part, N,
                       w->shift, nbins, w->bin_size, w->part_off);
    hipLaunchKernelGGL(k_bin_scan, dim3(1), dim3(256), 0, stream, w->bin_size, nbins, w->bin_start, w->offs + N);
    hipLaunchKernelGGL(k_bin_scatter, dim3((unsigned)w->n_parts), dim3(256), bin_lds, stream, old_idx, total, w->per_part, N,
                       w->shift, nbins, w->bin_start, w->part_off, w->bin_eq);
    hipLaunchKernelGGL(k_bin_rows, dim3((unsigned)nbins), dim3(kRowsBlock), sizeof(int) << w->shift, stream, w->bin_eq,
                       w->bin_start, w->shift, N, w->offs, w->rev);
    }
    hipLaunchKernelGGL(k_norm_tau, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream, bf.norms, knn_dist, N, K, w->norm_tau);
    RSFK_HIP(hipGetLastError());

    constexpr int kWaves = 4;
    const int KP = (K + 31) & ~31;
    const int wave_ints = (KP + 128 + 3) & ~3;
    const size_t lds = (size_t)kWaves * (size_t)wave_ints * sizeof(int);
    const int ksteps = (bf16_valid(D) + 15) / 16;
    RSFK_CHECK(ksteps * 16 <= bf16_pitch(D), "exploration join: bfloat16 rows too short");
    const float kappa = (float)(ksteps * 16 + 16) * (1.0f / 2097152.0f);            // (Dp + 16) 2^-21
    const float one_minus_gamma = 1.0f - (float)(D + 8) * (1.0f / 4194304.0f);      // 1 - (D + 8) 2^-22
    RSFK_CHECK(one_minus_gamma > 0.5f, "exploration join: D too large");
    if (!w->bounds && KP == 32 && ksteps <= 8) {
        const dim3 grid(grid_for_dies(((size_t)N + kWaves - 1) / kWaves)), block(64 * kWaves);
#define RSFK_JOIN_SHORT(KSV)                                                                                                \
        hipLaunchKernelGGL((k_explore_join_short<kWaves, KSV>), grid, block, 0, stream, bf, N, K, old_idx, w->norm_tau, w->offs, \
                           w->rev, w->pass, bf16_pitch(D), ksteps, kappa, one_minus_gamma, w->div_m, w->div_s, order)
        if (ksteps <= 2) RSFK_JOIN_SHORT(2);
        else if (ksteps <= 4) RSFK_JOIN_SHORT(4);
        else RSFK_JOIN_SHORT(8);
#undef RSFK_JOIN_SHORT
    } else if (KP > 32 && join_wg_on()) {
        // one workgroup per q: every row once per 96 points of R(q).  (Rows of at most 32 neighbours have one pair per
        // tile of R(q): too little for four wavefronts; 1M x 256, K = 32: 8.1 ms against 12.6.)
        const size_t lds_wg = (size_t)(kJwP + KP) * kJwRowBytes + (size_t)KP * 8 + (size_t)kJwP * 16;
#define RSFK_JOIN_WG(BV, NV)                                                                                                \
        do {                                                                                                               \
            RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(k_explore_join_wg<BV, NV>),                         \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_wg));                       \
            hipLaunchKernelGGL((k_explore_join_wg<BV, NV>), dim3(grid_for_dies((size_t)N)), dim3(256), lds_wg, stream, bf, N, K,  \
                               old_idx, w->norm_tau, w->offs, w->rev, w->pass, w->bounds, KP, bf16_pitch(D), ksteps, kappa,  \
                               one_minus_gamma, w->div_m, w->div_s, order);                                                \
        } while (0)
        if (w->bounds && KP <= 128) RSFK_JOIN_WG(true, 3);
        else if (w->bounds) RSFK_JOIN_WG(true, 6);
        else if (KP <= 128) RSFK_JOIN_WG(false, 3);
        else RSFK_JOIN_WG(false, 6);
#undef RSFK_JOIN_WG
    } else if (w->bounds)
        hipLaunchKernelGGL((k_explore_join<kWaves, true>), dim3(grid_for_dies(((size_t)N + kWaves - 1) / kWaves)), dim3(64 * kWaves), lds,
                           stream, bf, N, K, old_idx, w->norm_tau, w->offs, w->rev, w->pass, w->bounds, KP, bf16_pitch(D), ksteps,
                           kappa, one_minus_gamma, wave_ints, w->div_m, w->div_s, order);
    else
        hipLaunchKernelGGL((k_explore_join<kWaves, false>), dim3(grid_for_dies(((size_t)N + kWaves - 1) / kWaves)), dim3(64 * kWaves), lds,
                           stream, bf, N, K, old_idx, w->norm_tau, w->offs, w->rev, w->pass, w->bounds, KP, bf16_pitch(D), ksteps,
                           kappa, one_minus_gamma, wave_ints, w->div_m, w->div_s, order);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
