// Side tests of the first levels of a batch of trees, taken point by point instead of node by node.
//
// At the first levels of a tree every point is a member of a node that is still being split
// (build_tree_check_points_side.cu:131-149 tests each of them against the hyperplane of its node), and a batch of
// trees has few nodes per level: 2^l per tree.  The node-by-node kernel (k_side) gathers the screening row of every
// point once per tree and level, in the order of the tree's permutation.  Here the rows are streamed once per level
// in their natural order for all trees of the batch, and the tests become small integer matrix products on the
// matrix cores:
//
//   * the normal of a node is written as n_d = s1 m1_d + s2 m2_d + r_d with signed 8-bit m1, m2 (s1 = 254 s2 about
//     max|n| / 127) and a residual r of about 2^-16 max|n|;
//   * a tile of 32 points (their 8-bit rows, shifted to signed) is multiplied with the two 8-bit parts of 16
//     hyperplanes at a time by v_mfma_i32_32x32x32_i8: exact integer sums I1 = sum m1_d (q_d - 128),
//     I2 = sum m2_d (q_d - 128);
//   * n.x ~ lo sum n_d + scale s2 (254 I1 + I2 + 128 (254 sum m1 + sum m2)); the row's quantisation error is
//     bounded by e1 ||n||_1 (header of the 8-bit row, bf16.hpp), the residual by (|lo| + 255 scale) sum |r_d|; a
//     point whose value is farther from the offset than these bounds has the side the exact fp32 test would give
//     it, the others (one or two per cent) are marked and get the exact test (k_pm_resolve: the arithmetic of
//     resolve_exact in tree_build.hip);
//   * which node a point belongs to is kept as the sequence of its sides so far (one byte per point and tree); a
//     table maps such a path to the node of the level's queue, so nodes that were merged into a sibling or have gone
//     to the tail queue need no special case in the sweep.
//
// The sides are left as one bit per point and tree; k_pm_mark writes them into the permutation entries and counts
// the left members of every chunk, which is what k_side leaves for k_scatter.
#pragma once
#include "rsfk_common.hpp"
#include "wave64.hpp"
#include "bf16.hpp"
#include <type_traits>

namespace rsfk {
namespace pm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kMaxLevels = 8;                       // levels 0 .. 7 of a tree can be swept this way
constexpr int kPaths = 1 << (kMaxLevels - 1);       // paths (and nodes) per tree at the last such level
constexpr int kSlots = 16;                          // hyperplanes per operand block (two 8-bit rows each)
constexpr int kMaxGroups = kPaths / kSlots;

// One hyperplane as the sweep needs it.
struct PlaneQ {
    float b, hp1, hp2, s2;      // offset, bound of ||n||_1, sum of the components, scale of the second 8-bit part
    float c0, rres, pad;        // 128 s2 (254 sum m1 + sum m2), bound of sum |r_d| (and of what 254 s2 != s1 does)
    int ni;                     // node of the level's queue, or -1: the points with this path are not split any more
};
static_assert(sizeof(PlaneQ) == 32, "two 16-byte loads");

__device__ __forceinline__ float wave_sum_f(float v)
{
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// the value the lane 32 places away holds (v_permlane32_swap: no trip through LDS)
__device__ __forceinline__ int other_half(int x)
{
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)x, (unsigned)x, false, false);
    return (int)(lane_id() < 32 ? r[1] : r[0]);
}

// pmap of the next level from the children of the nodes of this one: child[ni] = queue places of the left and right
// child of node ni (-1: not in the next level's queue).
__global__ void k_pm_next_map(const int* __restrict__ pmap, int* __restrict__ pmap_next, const int2* __restrict__ child,
                              int n_paths, int nb)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nb * n_paths) return;
    const int t = i / n_paths, v = i - t * n_paths;
    const int ni = pmap[t * kPaths + v];
    const int2 c = ni >= 0 ? child[ni] : make_int2(-1, -1);
    pmap_next[t * kPaths + 2 * v] = c.x;
    pmap_next[t * kPaths + 2 * v + 1] = c.y;
}

// 8-bit parts and scalars of the hyperplanes of a level, one wavefront per (tree, path).  planes: records of
// k_level_planes ([offset, bound of the 1-norm, sum of the components, 0 | normal]), rec floats each.
// Aq: [tree][group] blocks of 32 rows x rowbytes, row j of a block = first part of the group's path j, row 16 + j =
// second part, stored in the order the sweep's lanes read them: bytes 32 k + 16 h .. + 15 of row r are the 16-byte
// piece number 64 k + 32 h + r of the block (a wavefront's load of step k is one contiguous kilobyte).
// With s2 about max|n| / (127 x 254) and s1 = fl(254 s2): m1 = round(n / s1), m2 = round((n - s1 m1) / s2), both
// clamped to +-127, r = n - s1 m1 - s2 m2 as computed.  The sweep evaluates s2 (254 I1 + I2), i.e. it takes
// 254 s2 for s1: that is off by a relative 2^-24, far below the 2^-18 ||n||_1 added to the bound of the residuals.
__global__ __launch_bounds__(256) void k_pm_planes(const float* __restrict__ planes, int rec, int D, int rowbytes,
                                                   const int* __restrict__ pmap, int n_paths, int nb,
                                                   PlaneQ* __restrict__ sc, int8_t* __restrict__ Aq)
{
    const int lane = threadIdx.x & 63;
    const int wg = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (wg >= nb * n_paths) return;
    const int t = wg / n_paths, v = wg - t * n_paths;
    const int ni = pmap[t * kPaths + v];
    PlaneQ* out = sc + (size_t)t * kPaths + v;
    if (ni < 0) {
        if (lane == 0) out->ni = -1;
        return;
    }
    const float* r = planes + (size_t)ni * rec;
    const float* nvec = r + 4;
    float mx = 0.0f;
    for (int d = lane; d < D; d += 64) mx = fmaxf(mx, fabsf(nvec[d]));
    mx = wave_max(mx);
    const float s2 = mx * (1.000001f / 32258.0f);
    const float s1 = 254.0f * s2;
    const float inv1 = s1 > 1e-30f ? 1.0f / s1 : 0.0f;
    const float inv2 = s2 > 1e-30f ? 1.0f / s2 : 0.0f;
    int8_t* block = Aq + (size_t)(t * kMaxGroups + v / kSlots) * 32 * rowbytes;
    const int r1 = v % kSlots, r2 = r1 + kSlots;
    float rs = 0.0f;
    int M = 0;
    for (int d = lane; d < rowbytes; d += 64) {
        const float n = d < D ? nvec[d] : 0.0f;
        const float m1 = fminf(fmaxf(__builtin_rintf(n * inv1), -127.0f), 127.0f);
        const float e = __builtin_fmaf(-s1, m1, n);
        const float m2 = fminf(fmaxf(__builtin_rintf(e * inv2), -127.0f), 127.0f);
        const float rr = __builtin_fmaf(-s2, m2, e);
        rs += fabsf(rr);                                  // NaN (a normal with NaN or infinite components) stays NaN
        const int i1 = (int)m1, i2 = (int)m2;
        M += 254 * i1 + i2;
        const int piece = 64 * (d >> 5) + 32 * ((d >> 4) & 1);
        block[(piece + r1) * 16 + (d & 15)] = (int8_t)i1;
        block[(piece + r2) * 16 + (d & 15)] = (int8_t)i2;
    }
    rs = wave_sum_f(rs);
    M = wave_sum_i(M);
    if (lane == 0) {
        PlaneQ q;
        q.b = r[0]; q.hp1 = r[1]; q.hp2 = r[2]; q.s2 = s2;
        q.c0 = s2 * (float)(128 * M);                     // |128 M| <= 128 x 127 x 255 D < 2^31 for D <= 256
        // the residuals are known to a relative 2^-7 or so of their size (they are differences of fp32 numbers of
        // the size of s1); 2^-18 of the 1-norm covers that, the rounding of their sum and of c0, and s1 != 254 s2
        q.rres = 1.01f * rs + r[1] * (1.0f / 262144.0f);
        q.pad = 0.0f;
        q.ni = ni;
        *out = q;
    }
}

// The value as something the optimiser cannot look through.  (Selects between elements of a vector would otherwise be
// turned into one extraction with a variable index: a chain of 15 compares and selects, or a trip through memory.)
__device__ __forceinline__ int opaque(int x)
{
    asm volatile("" : "+v"(x));
    return x;
}

// a[BASE + idx], idx in 0..7 given by its bits, for an index that differs from lane to lane: a tree of selects
template <int BASE>
__device__ __forceinline__ int pick8(const v16i& a, bool b0, bool b1, bool b2)
{
    const int e0 = opaque(a[BASE + 0]), e1 = opaque(a[BASE + 1]), e2 = opaque(a[BASE + 2]), e3 = opaque(a[BASE + 3]);
    const int e4 = opaque(a[BASE + 4]), e5 = opaque(a[BASE + 5]), e6 = opaque(a[BASE + 6]), e7 = opaque(a[BASE + 7]);
    const int x0 = b0 ? e1 : e0, x1 = b0 ? e3 : e2, x2 = b0 ? e5 : e4, x3 = b0 ? e7 : e6;
    const int y0 = b1 ? x1 : x0, y1 = b1 ? x3 : x2;
    return b2 ? y1 : y0;
}

// The sweep.  A wavefront keeps two tiles of 32 points -- their 8-bit rows as matrix-core operands: lane (n, h) holds
// bytes 32 j + 16 h .. + 15 of the row of point n of either tile, j < KS -- and walks the trees of the batch.  For
// everything that is per point (path, scalars of the hyperplane, decision) lane (n, h) stands for point n of tile h.
//
// path: one byte per point and tree, [point][Bs] (Bs = trees of a batch rounded up to 16): the sides of the point at
// the levels before this one, first level in the highest bit.  sidebits / undec: one bit per point and tree,
// [tree][W] words: on entry sidebits holds the sides of the previous level (level > 0), on return those of this
// level for the points the screen decided (0 = left) and undec marks the points that are left to the exact test.
// A wavefront reads all of that for its 64 points and all trees at the start (into LDS) and writes it at the end;
// inside the loop only the hyperplanes are fetched -- the operand block two steps ahead, a point's scalars two
// steps before its tree begins -- into rings of three whose slots are fixed at compile time (a step = one block of
// 16 hyperplanes of one tree).
template <int KS>
__global__ __launch_bounds__(256) void k_pm_sweep(const uint8_t* __restrict__ q8, int N, int D, int nb, int Bs, int level,
                                                  int W, uint8_t* __restrict__ path, uint32_t* __restrict__ sidebits,
                                                  uint32_t* __restrict__ undec, const int8_t* __restrict__ Aq,
                                                  const PlaneQ* __restrict__ sc)
{
    constexpr int kPathPitch = 68;                       // 17 words: lanes read their bytes from different banks
    __shared__ __align__(16) uint8_t path_s[4][64 * kPathPitch];
    __shared__ uint32_t win_s[4][2][64], rout_s[4][2][64], uout_s[4][2][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 31, h = lane >> 5;
    const int tile0 = (blockIdx.x * 4 + wave) * 2;
    if (tile0 >= W) return;
    const size_t pitch = (size_t)q8_pitch(D);
    const int payload = (int)pitch - 16;
    constexpr int kRowBytes = 32 * KS;
    const int lg = level <= 4 ? 0 : level - 4;
    const int n_groups = 1 << lg;
    const int total = nb << lg;

    v4i brow[2][KS];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int pu = (tile0 + u) * 32 + n;
        const uint8_t* row = q8 + (size_t)(pu < N ? pu : 0) * pitch + 16;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            const int off = 32 * j + 16 * h;
            v4i w = {0, 0, 0, 0};
            if (pu < N && off + 16 <= payload) w = *reinterpret_cast<const v4i*>(row + off);
            brow[u][j] = w ^ (int)0x80808080;
        }
    }
    const int po = (tile0 + h) * 32 + n;            // the point this lane decides
    const bool valid = po < N;
    float lo, scale, e1;
    {
        const uint4 head = *reinterpret_cast<const uint4*>(q8 + (size_t)(valid ? po : 0) * pitch);
        lo = __uint_as_float(head.y);
        scale = __uint_as_float(head.z);
        e1 = __uint_as_float(head.w);
    }
    const float mag = fabsf(lo) + 255.0f * scale;

    // paths and previous sides of the wavefront's points, all trees
    uint8_t* my_path = path_s[wave] + lane * kPathPitch;
    if (level > 0) {
        const uint8_t* src = path + (size_t)(valid ? po : 0) * Bs;
        for (int q = 0; q < Bs; q += 16) {
            const uint4 w = *reinterpret_cast<const uint4*>(src + q);
            uint32_t* dst = reinterpret_cast<uint32_t*>(my_path + q);
            dst[0] = w.x; dst[1] = w.y; dst[2] = w.z; dst[3] = w.w;
        }
        if (n < nb) win_s[wave][h][n] = sidebits[(size_t)n * W + tile0 + h];
        if (n + 32 < nb) win_s[wave][h][n + 32] = sidebits[(size_t)(n + 32) * W + tile0 + h];
    }
    wave_lds_sync();
    auto path_of = [&](int t) -> int {
        if (level == 0) return 0;
        return 2 * (int)my_path[t] + (int)((win_s[wave][h][t] >> n) & 1u);
    };

    // (bases that are the same for all lanes plus 32-bit offsets: the loads take the base from scalar registers)
    const uint32_t a_off = (uint32_t)(lane * 16);
    auto load_a = [&](int t, int g, v4i (&a)[KS]) {
        const int8_t* src = Aq + (size_t)(t * kMaxGroups + g) * (32 * kRowBytes);
#pragma unroll
        for (int j = 0; j < KS; ++j) a[j] = *reinterpret_cast<const v4i*>(src + (a_off + 1024u * j));
    };
    auto load_q = [&](int t, int v, float4& qa, float4& qb) {
        const float4* src = reinterpret_cast<const float4*>(sc + (size_t)t * kPaths);
        qa = src[2u * (uint32_t)v];
        qb = src[2u * (uint32_t)v + 1u];
    };

    v4i a_r[3][KS];
    float4 qa_r[3], qb_r[3], qa, qb;
    int v_r[3], v = 0;
    bool active = false;
    int vt[2] = {-1, -1}, cand[2] = {0, 0};

    // what step `it` will need, into slot SLOT of the rings
    auto request = [&](int it, auto slot_c) {
        constexpr int SLOT = decltype(slot_c)::value;
        if (it >= total) return;
        const int t = it >> lg, g = it & (n_groups - 1);
        load_a(t, g, a_r[SLOT]);
        if (g == 0) {
            v_r[SLOT] = path_of(t);
            load_q(t, v_r[SLOT], qa_r[SLOT], qb_r[SLOT]);
        }
    };
    auto step = [&](int it, auto slot_c) {
        constexpr int SLOT = decltype(slot_c)::value;
        const int t = it >> lg, g = it & (n_groups - 1);
        request(it + 2, std::integral_constant<int, (SLOT + 2) % 3>());
        if (g == 0) {
            v = v_r[SLOT];
            qa = qa_r[SLOT];
            qb = qb_r[SLOT];
            active = valid && __float_as_int(qb.w) >= 0;
            my_path[t] = (uint8_t)v;
            // paths of point n of tile 0 and of tile 1 (-1: not tested), in both lanes that hold its operands
            const int vv = active ? v : -1;
            const auto r = __builtin_amdgcn_permlane32_swap((unsigned)vv, (unsigned)vv, false, false);
            vt[0] = (int)r[0];
            vt[1] = (int)r[1];
            cand[0] = 0;
            cand[1] = 0;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const bool here = vt[u] >= 0 && (vt[u] >> 4) == g;
            if (ballot64(here) != 0) {
                v16i acc;
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = 0;
#pragma unroll
                for (int j = 0; j < KS; ++j)
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_r[SLOT][j], brow[u][j], acc, 0, 0, 0);
                // rows 8 q + 4 h + r of the product sit in lane (n, h): path slot s = 8 q + 4 h' + r has its
                // first part in row s and its second in row 16 + s, both in the lane with h = h'
                const int s = vt[u];
                const bool b0 = s & 1, b1 = s & 2, b2 = s & 8;
                const int comb = 254 * pick8<0>(acc, b0, b1, b2) + pick8<8>(acc, b0, b1, b2);
                if (here && h == ((s >> 2) & 1)) cand[u] = comb;
            }
        }
        if (g == n_groups - 1) {
            // the sum of this lane's own point is in cand[h] of this lane or of the lane 32 places away
            const int own = h ? cand[1] : cand[0];
            const int oth = other_half(h ? cand[0] : cand[1]);
            const int I = h == ((v >> 2) & 1) ? own : oth;
            const float b = qa.x, hp1 = qa.y, hp2 = qa.z, s2 = qa.w, c0 = qb.x, rres = qb.y;
            const float T = __builtin_fmaf(s2, (float)I, c0);
            const float approx = __builtin_fmaf(scale, T, lo * hp2);
            const float band = __builtin_fmaf(e1, hp1, mag * rres);
            const bool certain = fabsf(approx - b) > band;                 // false if anything is NaN
            const uint64_t rm = ballot64(active && certain && approx < b);
            const uint64_t um = ballot64(active && !certain);
            if (n == 0) {
                rout_s[wave][h][t] = h ? (uint32_t)(rm >> 32) : (uint32_t)rm;
                uout_s[wave][h][t] = h ? (uint32_t)(um >> 32) : (uint32_t)um;
            }
        }
    };

    const std::integral_constant<int, 0> c0;
    const std::integral_constant<int, 1> c1;
    const std::integral_constant<int, 2> c2;
    request(0, c0);
    request(1, c1);
    int it = 0;
    for (; it + 2 < total; it += 3) {
        step(it, c0);
        step(it + 1, c1);
        step(it + 2, c2);
    }
    if (it < total) step(it, c0);
    if (it + 1 < total) step(it + 1, c1);

    wave_lds_sync();
    if (valid) {
        uint8_t* dst = path + (size_t)po * Bs;
        for (int q = 0; q < Bs; q += 16) {
            const uint32_t* src = reinterpret_cast<const uint32_t*>(my_path + q);
            *reinterpret_cast<uint4*>(dst + q) = make_uint4(src[0], src[1], src[2], src[3]);
        }
    }
    if (n < nb) {
        sidebits[(size_t)n * W + tile0 + h] = rout_s[wave][h][n];
        undec[(size_t)n * W + tile0 + h] = uout_s[wave][h][n];
    }
    if (n + 32 < nb) {
        sidebits[(size_t)(n + 32) * W + tile0 + h] = rout_s[wave][h][n + 32];
        undec[(size_t)(n + 32) * W + tile0 + h] = uout_s[wave][h][n + 32];
    }
}

// Exact side tests of the marked points: the arithmetic of resolve_exact (32 lane-strided fused multiply-add chains
// and the xor butterfly, build_tree_check_points_side.cu:131-149).  A wavefront takes 64 words of undec (word
// tree * W + tile), lists their marked points, looks up the hyperplanes of 64 of them at a time (one per lane) and
// then tests them, one half wavefront per point, two points per half wavefront in flight.
__global__ __launch_bounds__(256) void k_pm_resolve(const float* __restrict__ points, int D, int W, int Bs,
                                                    size_t total_words, const uint8_t* __restrict__ path,
                                                    const PlaneQ* __restrict__ sc, const float* __restrict__ planes,
                                                    int rec, uint32_t* __restrict__ sidebits,
                                                    const uint32_t* __restrict__ undec,
                                                    unsigned long long* __restrict__ stat)
{
    __shared__ uint16_t list_s[4][2048];
    __shared__ int e_ni[4][64], e_pt[4][64];
    __shared__ float e_b[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, hl = lane & 31;
    const size_t w0 = ((size_t)blockIdx.x * 4 + wave) * 64;
    if (w0 >= total_words) return;
    const uint32_t bits = w0 + lane < total_words ? undec[w0 + lane] : 0u;
    const int cnt = __popc(bits);
    const int off = wave_excl_scan_i(cnt);
    const int total = read_lane_i(off + cnt, 63);
    if (total == 0) return;
    // (count of the points left to the exact test, for the report of a build: slots a cache line apart)
    if (stat && lane == 0) atomicAdd(&stat[32 * (blockIdx.x & 63) + 1], (unsigned long long)total);
    uint16_t* list = list_s[wave];
    {
        uint32_t w = bits;
        int o = off;
        while (w != 0u) {
            const int bit = __ffs(w) - 1;
            w &= w - 1;
            list[o++] = (uint16_t)((lane << 5) | bit);
        }
    }
    wave_lds_sync();
    for (int base = 0; base < total; base += 64) {
        const int m = min(64, total - base);
        if (lane < m) {
            const int e = list[base + lane];
            const size_t wi = w0 + (e >> 5);
            const int t = (int)(wi / (size_t)W);
            const int pt = (int)(wi - (size_t)t * W) * 32 + (e & 31);
            const int v = path[(size_t)pt * Bs + t];
            const PlaneQ* q = sc + (size_t)t * kPaths + v;
            e_ni[wave][lane] = q->ni;
            e_b[wave][lane] = q->b;
            e_pt[wave][lane] = pt;
        }
        wave_lds_sync();
        for (int k = 0; k < m; k += 4) {
            const int ia = k + h, ib = k + 2 + h;
            const bool va = ia < m && e_ni[wave][ia < m ? ia : 0] >= 0;
            const bool vb = ib < m && e_ni[wave][ib < m ? ib : 0] >= 0;
            const float* xa = points + (size_t)(va ? e_pt[wave][ia] : 0) * D;
            const float* xb = points + (size_t)(vb ? e_pt[wave][ib] : 0) * D;
            const float* na = planes + (size_t)(va ? e_ni[wave][ia] : 0) * rec + 4;
            const float* nb_ = planes + (size_t)(vb ? e_ni[wave][ib] : 0) * rec + 4;
            float sa = 0.0f, sb = 0.0f;
            for (int d0 = hl; d0 < D; d0 += 256) {
                float xv[8], yv[8], nx[8], ny[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const bool in = d0 + 32 * q < D;
                    xv[q] = (va && in) ? xa[d0 + 32 * q] : 0.0f;
                    nx[q] = (va && in) ? na[d0 + 32 * q] : 0.0f;
                    yv[q] = (vb && in) ? xb[d0 + 32 * q] : 0.0f;
                    ny[q] = (vb && in) ? nb_[d0 + 32 * q] : 0.0f;
                }
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    if (d0 + 32 * q < D) {
                        sa = __builtin_fmaf(nx[q], xv[q], sa);
                        sb = __builtin_fmaf(ny[q], yv[q], sb);
                    }
                }
            }
            sa = half_butterfly_sum(sa);
            sb = half_butterfly_sum(sb);
            if (hl == 0) {
                if (va && sa < e_b[wave][ia]) {
                    const int e = list[base + ia];
                    atomicOr(&sidebits[w0 + (e >> 5)], 1u << (e & 31));
                }
                if (vb && sb < e_b[wave][ib]) {
                    const int e = list[base + ib];
                    atomicOr(&sidebits[w0 + (e >> 5)], 1u << (e & 31));
                }
            }
        }
        wave_lds_sync();
    }
}

}  // namespace pm
}  // namespace rsfk
