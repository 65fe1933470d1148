// Symmetrised K-NN graph in compressed-row form: row p holds every neighbour stored for p and every point that
// stores p as a neighbour, once, with the squared distance of the pair; columns ascend inside a row.  This is what
// consumers of the K-NN graph (t-SNE, UMAP, spectral methods) build first.  Replaces the three kernels the reference
// keeps commented out next to its spectral experiment (symmetric_knn_graph_edge_count / _offset / _add_edges,
// src/rsfk.cu:1229-1299: one thread per point, a serial prefix sum by a single thread, row order = arrival order of
// atomics).
//
// Steps: (1) a wavefront per point looks its own number up in the rows of its neighbours (coalesced row reads, four
// neighbours in flight) and counts, per point, the stored neighbours and the missing reverse edges; (2) prefix sum of
// the row lengths; (3) the edges are written to their rows: the stored ones at compacted positions, the added ones
// behind them in arrival order; (4) a segmented sort by column (rocPRIM) makes the rows independent of that order.
#include "forest.hpp"
#include "wave64.hpp"
#include <cstring>
#include <mutex>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/device/device_segmented_radix_sort.hpp>

namespace rsfk {

namespace {

constexpr unsigned char kNoEdge = 0, kMutual = 1, kOneWay = 2;

__device__ __forceinline__ bool usable(int c, int p, int N, int drop_self) { return c >= 0 && c < N && !(drop_self && c == p); }

// flag[p*K + k]: kNoEdge (empty slot, out of range, or a dropped self edge), kMutual (the neighbour stores p too),
// kOneWay (it does not: the reverse edge has to be added).  n_own[p] = stored edges of p, extra[p] (zero on entry) =
// reverse edges row p receives.
template <int SL>
__global__ __launch_bounds__(256) void k_sym_flags(const int* __restrict__ idx, int N, int K, int drop_self,
                                                   unsigned char* __restrict__ flag, int* __restrict__ n_own,
                                                   int* __restrict__ extra)
{
    const int lane = threadIdx.x & 63;
    const int p = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p >= N) return;
    int mine[SL];
#pragma unroll
    for (int s = 0; s < SL; ++s) {
        const int k = lane + 64 * s;
        mine[s] = k < K ? idx[(size_t)p * K + k] : -1;
    }
    int own = 0;
    for (int k0 = 0; k0 < K; k0 += 4) {
        int pn[4];
        bool ok[4];
        int theirs[4][SL];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = k0 + u;
            int c = -1;
#pragma unroll
            for (int s = 0; s < SL; ++s)
                if ((k >> 6) == s) c = read_lane_i(mine[s], k & 63);
            pn[u] = c;
            ok[u] = k < K && usable(c, p, N, drop_self);
#pragma unroll
            for (int s = 0; s < SL; ++s) {
                const int kk = lane + 64 * s;
                theirs[u][s] = (ok[u] && kk < K) ? idx[(size_t)c * K + kk] : -1;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            bool hit = false;
#pragma unroll
            for (int s = 0; s < SL; ++s) hit |= theirs[u][s] == p;
            const bool mutual = ballot64(hit) != 0;
            if (k0 + u < K && lane == 0) {
                flag[(size_t)p * K + k0 + u] = !ok[u] ? kNoEdge : (mutual ? kMutual : kOneWay);
                if (ok[u] && !mutual) atomicAdd(&extra[pn[u]], 1);
            }
            own += ok[u] ? 1 : 0;
        }
    }
    if (lane == 0) n_own[p] = own;
}

// len[p] = length of row p; extra is set back to zero (it becomes the cursor of the added edges); len[N] = 0
__global__ __launch_bounds__(256) void k_sym_len(const int* __restrict__ n_own, int* __restrict__ extra, int N, int* __restrict__ len)
{
    const int p = blockIdx.x * 256 + threadIdx.x;
    if (p < N) { len[p] = n_own[p] + extra[p]; extra[p] = 0; }
    else if (p == N) len[p] = 0;
}

// Lane k of the wavefront of p writes the stored edge k to its compacted place in row p and, for a one-way edge, the
// reverse edge into the row of the neighbour behind that row's stored edges.
template <int SL>
__global__ __launch_bounds__(256) void k_sym_fill(const int* __restrict__ idx, const float* __restrict__ dist, int N, int K,
                                                  const unsigned char* __restrict__ flag, const int* __restrict__ n_own,
                                                  int* __restrict__ cursor, const int* __restrict__ indptr,
                                                  int* __restrict__ cols, float* __restrict__ vals)
{
    const int lane = threadIdx.x & 63;
    const int p = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p >= N) return;
    const int row0 = indptr[p];
    int before = 0;
#pragma unroll
    for (int s = 0; s < SL; ++s) {
        const int k = lane + 64 * s;
        const size_t e = (size_t)p * K + k;
        const int f = k < K ? flag[e] : kNoEdge;
        const uint64_t m = ballot64(f != kNoEdge);
        if (f != kNoEdge) {
            const int c = idx[e];
            const float d = dist ? dist[e] : 0.0f;
            const int at = row0 + before + __popcll(m & ((1ull << lane) - 1ull));
            cols[at] = c;
            vals[at] = d;
            if (f == kOneWay) {
                const int ra = indptr[c] + n_own[c] + atomicAdd(&cursor[c], 1);
                cols[ra] = p;
                vals[ra] = d;
            }
        }
        before += __popcll(m);
    }
}

int sym_launch_flags(const int* idx, int N, int K, int drop_self, unsigned char* flag, int* n_own, int* extra, hipStream_t stream)
{
    const dim3 grid((unsigned)((N + 3) / 4)), block(256);
    if (K <= 64) hipLaunchKernelGGL(k_sym_flags<1>, grid, block, 0, stream, idx, N, K, drop_self, flag, n_own, extra);
    else if (K <= 128) hipLaunchKernelGGL(k_sym_flags<2>, grid, block, 0, stream, idx, N, K, drop_self, flag, n_own, extra);
    else if (K <= 256) hipLaunchKernelGGL(k_sym_flags<4>, grid, block, 0, stream, idx, N, K, drop_self, flag, n_own, extra);
    else if (K <= 512) hipLaunchKernelGGL(k_sym_flags<8>, grid, block, 0, stream, idx, N, K, drop_self, flag, n_own, extra);
    else hipLaunchKernelGGL(k_sym_flags<16>, grid, block, 0, stream, idx, N, K, drop_self, flag, n_own, extra);
    RSFK_HIP(hipGetLastError());
    return 0;
}

int sym_launch_fill(const int* idx, const float* dist, int N, int K, const unsigned char* flag, const int* n_own, int* cursor,
                    const int* indptr, int* cols, float* vals, hipStream_t stream)
{
    const dim3 grid((unsigned)((N + 3) / 4)), block(256);
    if (K <= 64)
        hipLaunchKernelGGL(k_sym_fill<1>, grid, block, 0, stream, idx, dist, N, K, flag, n_own, cursor, indptr, cols, vals);
    else if (K <= 128)
        hipLaunchKernelGGL(k_sym_fill<2>, grid, block, 0, stream, idx, dist, N, K, flag, n_own, cursor, indptr, cols, vals);
    else if (K <= 256)
        hipLaunchKernelGGL(k_sym_fill<4>, grid, block, 0, stream, idx, dist, N, K, flag, n_own, cursor, indptr, cols, vals);
    else if (K <= 512)
        hipLaunchKernelGGL(k_sym_fill<8>, grid, block, 0, stream, idx, dist, N, K, flag, n_own, cursor, indptr, cols, vals);
    else
        hipLaunchKernelGGL(k_sym_fill<16>, grid, block, 0, stream, idx, dist, N, K, flag, n_own, cursor, indptr, cols, vals);
    RSFK_HIP(hipGetLastError());
    return 0;
}

struct Buf {
    void* p = nullptr;
    ~Buf() { if (p) ws_free(p); }
};

}  // namespace

// d_idx / d_dist: N x K (d_dist may be null: the values are then zero).  d_indptr: N + 1 ints.  d_cols / d_vals: room for
// `cap` entries, or both null to obtain only d_indptr and *nnz.  Entries that are negative or >= N are no edges;
// drop_self removes p from its own row.  A row must not hold a point twice.
int symmetrize_device(const int* d_idx, const float* d_dist, int N, int K, int drop_self, int* d_indptr, int* d_cols,
                      float* d_vals, long long cap, long long* nnz, hipStream_t stream)
{
    RSFK_CHECK(N >= 1 && K >= 1 && K <= kMaxK, "graph export: N must be positive and K in 1..1024");
    RSFK_CHECK((long long)N * K < (1ll << 30), "graph export: N * K of 2^30 and more is not supported");
    RSFK_CHECK(d_idx && d_indptr && nnz, "graph export: null argument");
    RSFK_CHECK((d_cols == nullptr) == (d_vals == nullptr), "graph export: indices and data go together");
    Buf flag, own, extra, len;
    if (ws_alloc(&flag.p, (size_t)N * K) || ws_alloc(&own.p, sizeof(int) * (size_t)N) ||
        ws_alloc(&extra.p, sizeof(int) * (size_t)N) || ws_alloc(&len.p, sizeof(int) * ((size_t)N + 1)))
        return 1;
    int* n_own = static_cast<int*>(own.p);
    int* ext = static_cast<int*>(extra.p);
    RSFK_HIP(hipMemsetAsync(ext, 0, sizeof(int) * (size_t)N, stream));
    if (sym_launch_flags(d_idx, N, K, drop_self, static_cast<unsigned char*>(flag.p), n_own, ext, stream)) return 1;
    hipLaunchKernelGGL(k_sym_len, dim3((unsigned)(N / 256 + 1)), dim3(256), 0, stream, n_own, ext, N, static_cast<int*>(len.p));
    RSFK_HIP(hipGetLastError());
    size_t tmp_bytes = 0;
    RSFK_HIP(rocprim::exclusive_scan(nullptr, tmp_bytes, static_cast<int*>(len.p), d_indptr, 0, (size_t)N + 1,
                                     rocprim::plus<int>(), stream));
    {
        Buf tmp;
        if (ws_alloc(&tmp.p, tmp_bytes ? tmp_bytes : 256)) return 1;
        RSFK_HIP(rocprim::exclusive_scan(tmp.p, tmp_bytes, static_cast<int*>(len.p), d_indptr, 0, (size_t)N + 1,
                                         rocprim::plus<int>(), stream));
        int total = 0;
        RSFK_HIP(hipMemcpyAsync(&total, d_indptr + N, sizeof(int), hipMemcpyDeviceToHost, stream));
        RSFK_HIP(hipStreamSynchronize(stream));
        *nnz = total;
    }
    if (!d_cols || *nnz == 0) return 0;
    RSFK_CHECK(*nnz <= cap, "graph export: the output arrays are too small for the graph");
    const size_t n = (size_t)*nnz;
    Buf cols, vals;
    if (ws_alloc(&cols.p, sizeof(int) * n) || ws_alloc(&vals.p, sizeof(float) * n)) return 1;
    if (sym_launch_fill(d_idx, d_dist, N, K, static_cast<unsigned char*>(flag.p), n_own, ext, d_indptr,
                        static_cast<int*>(cols.p), static_cast<float*>(vals.p), stream))
        return 1;
    int bits = 1;
    while (bits < 31 && (1ll << bits) < (long long)N) ++bits;          // columns are below N
    size_t sort_bytes = 0;
    RSFK_HIP(rocprim::segmented_radix_sort_pairs(nullptr, sort_bytes, static_cast<int*>(cols.p), d_cols,
                                                 static_cast<float*>(vals.p), d_vals, (unsigned)n, (unsigned)N, d_indptr,
                                                 d_indptr + 1, 0, (unsigned)bits, stream));
    Buf tmp;
    if (ws_alloc(&tmp.p, sort_bytes ? sort_bytes : 256)) return 1;
    RSFK_HIP(rocprim::segmented_radix_sort_pairs(tmp.p, sort_bytes, static_cast<int*>(cols.p), d_cols,
                                                 static_cast<float*>(vals.p), d_vals, (unsigned)n, (unsigned)N, d_indptr,
                                                 d_indptr + 1, 0, (unsigned)bits, stream));
    RSFK_HIP(hipStreamSynchronize(stream));
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------------
// The count-only call (row lengths, d_indptr and the number of entries) for callers that cannot allocate device memory:
// tight serving loops, harnesses that forbid hipMalloc, code that records a HIP graph.  With nnz == nullptr the call
// only enqueues kernels (the count is left in d_indptr[N] on the device); with nnz != nullptr it also copies the
// count to the host and synchronises the stream, which a stream under capture refuses.  Its working memory -- the edge
// flags, the three per-point counters and the temporary storage of the prefix sum, which symmetrize_device takes from
// the workspace pool -- lives in a file-scope device array of fixed size.  Every GPU the library runs on holds its
// own copy of that array until the process ends; its address on a device is looked up once per device and kept.
// All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race.
// ---------------------------------------------------------------------------------------------------------------------
namespace {

constexpr int kNaMaxPoints = 1 << 20;                     // N
constexpr long long kNaMaxSlots = 1ll << 25;              // N * K
constexpr size_t kNaScanBytes = (size_t)1 << 20;          // temporary storage of the prefix sum over N + 1 row lengths
constexpr size_t kNaCounterBytes = ((sizeof(int) * ((size_t)kNaMaxPoints + 1) + 255) / 256) * 256;
constexpr size_t kNaFlagOff = 0;
constexpr size_t kNaOwnOff = kNaFlagOff + (size_t)kNaMaxSlots;
constexpr size_t kNaExtraOff = kNaOwnOff + kNaCounterBytes;
constexpr size_t kNaLenOff = kNaExtraOff + kNaCounterBytes;
constexpr size_t kNaScanOff = kNaLenOff + kNaCounterBytes;
constexpr size_t kNaBytes = kNaScanOff + kNaScanBytes;    // 32 MiB + 3 x 4 MiB + 1 MiB

static __device__ __align__(256) unsigned char scratch[kNaBytes];

constexpr int kNaMaxDevices = 64;
unsigned char* g_scratch_ptr[kNaMaxDevices];              // device address of `scratch` on each device, once known
std::mutex g_scratch_mutex;

// The device address of the array on the current device.  The array's name is only a host-side handle.
int scratch_on_current_device(unsigned char** out)
{
    int dev = -1;
    RSFK_HIP(hipGetDevice(&dev));
    RSFK_CHECK(dev >= 0 && dev < kNaMaxDevices, "graph export: device number out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        RSFK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        RSFK_CHECK(p != nullptr, "graph export: no device address for the working memory");
        g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

__global__ __launch_bounds__(256) void k_zero_counters(int* __restrict__ v, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) v[i] = 0;
}

}  // namespace

int symmetrize_count_noalloc(const int* d_idx, int N, int K, int drop_self, int* d_indptr, long long* nnz, hipStream_t stream)
{
    RSFK_CHECK(d_idx && d_indptr, "graph export: null argument");
    RSFK_CHECK(N >= 1 && K >= 1 && K <= kMaxK, "graph export: N must be positive and K in 1..1024");
    RSFK_CHECK(N <= kNaMaxPoints && (long long)N * K <= kNaMaxSlots,
               "graph export without allocation: at most 2^20 points and 2^25 neighbour slots (N * K)");
    unsigned char* base = nullptr;
    if (scratch_on_current_device(&base)) return 1;
    unsigned char* flag = base + kNaFlagOff;
    int* n_own = reinterpret_cast<int*>(base + kNaOwnOff);
    int* ext = reinterpret_cast<int*>(base + kNaExtraOff);
    int* len = reinterpret_cast<int*>(base + kNaLenOff);
    void* scan_tmp = base + kNaScanOff;
    size_t tmp_bytes = 0;
    RSFK_HIP(rocprim::exclusive_scan(nullptr, tmp_bytes, len, d_indptr, 0, (size_t)N + 1, rocprim::plus<int>(), stream));
    RSFK_CHECK(tmp_bytes <= kNaScanBytes, "graph export without allocation: the prefix sum needs more temporary storage than reserved");
    // the counters of the reverse edges must start at zero; the array keeps the previous call's contents
    hipLaunchKernelGGL(k_zero_counters, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream, ext, N);
    RSFK_HIP(hipGetLastError());
    if (sym_launch_flags(d_idx, N, K, drop_self, flag, n_own, ext, stream)) return 1;
    hipLaunchKernelGGL(k_sym_len, dim3((unsigned)(N / 256 + 1)), dim3(256), 0, stream, n_own, ext, N, len);
    RSFK_HIP(hipGetLastError());
    RSFK_HIP(rocprim::exclusive_scan(scan_tmp, tmp_bytes, len, d_indptr, 0, (size_t)N + 1, rocprim::plus<int>(), stream));
    if (nnz == nullptr) return 0;                       // the count stays in d_indptr[N]; nothing but kernels was queued
    int total = 0;
    RSFK_HIP(hipMemcpyAsync(&total, d_indptr + N, sizeof(int), hipMemcpyDeviceToHost, stream));
    RSFK_HIP(hipStreamSynchronize(stream));
    *nnz = total;
    return 0;
}

int symmetrize_host(const int* idx, const float* dist, int N, int K, int drop_self, int* indptr, int* cols, float* vals,
                    long long cap, long long* nnz)
{
    RSFK_CHECK(N >= 1 && K >= 1, "graph export: N and K must be positive");
    RSFK_CHECK(idx && indptr && nnz, "graph export: null argument");
    RSFK_CHECK((cols == nullptr) == (vals == nullptr), "graph export: indices and data go together");
    Buf di, dd, dp, dc, dv;
    const size_t nk = (size_t)N * K;
    if (ws_alloc(&di.p, nk * sizeof(int)) || ws_alloc(&dp.p, ((size_t)N + 1) * sizeof(int))) return 1;
    RSFK_HIP(hipMemcpy(di.p, idx, nk * sizeof(int), hipMemcpyHostToDevice));
    if (dist) {
        if (ws_alloc(&dd.p, nk * sizeof(float))) return 1;
        RSFK_HIP(hipMemcpy(dd.p, dist, nk * sizeof(float), hipMemcpyHostToDevice));
    }
    if (cols && cap > 0) {
        if (ws_alloc(&dc.p, (size_t)cap * sizeof(int)) || ws_alloc(&dv.p, (size_t)cap * sizeof(float))) return 1;
    }
    const int rc = symmetrize_device(static_cast<const int*>(di.p), static_cast<const float*>(dd.p), N, K, drop_self,
                                     static_cast<int*>(dp.p), static_cast<int*>(dc.p), static_cast<float*>(dv.p), cap, nnz,
                                     nullptr);
    if (rc) return rc;
    RSFK_HIP(hipMemcpy(indptr, dp.p, ((size_t)N + 1) * sizeof(int), hipMemcpyDeviceToHost));
    if (dc.p && *nnz > 0) {
        RSFK_HIP(hipMemcpy(cols, dc.p, (size_t)*nnz * sizeof(int), hipMemcpyDeviceToHost));
        RSFK_HIP(hipMemcpy(vals, dv.p, (size_t)*nnz * sizeof(float), hipMemcpyDeviceToHost));
    }
    return 0;
}

}  // namespace rsfk
