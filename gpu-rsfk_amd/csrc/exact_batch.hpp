// Exact distances of a batch of up to 64 candidates to one point, by one wavefront, and their merge into the
// point's K-NN row: shared by the exploration kernels and the query-set search.
//
// The candidates' fp32 rows are gathered with coalesced segments (several lanes per row), transposed through a
// tile in LDS, and every lane runs the sequential fused multiply-add chain of "its" candidate (the arithmetic
// of euclidean_distance_sqr, compute_knn_from_buckets.cu:40-54, so a pair of points has one distance value
// everywhere in the library).
#pragma once
#include "rsfk_common.hpp"
#include "knn_list.hpp"

namespace rsfk {

constexpr int kChunk = 32;              // fp32 dimensions per staging step (default)

struct ExploreLds {          // per wavefront; sizes fixed at launch
    int* table;              // hash set / candidate list, table_size ints
    int* srow;               // snapshot of the point's own row, K ints
    int* queue2;             // candidates that passed the screen, waiting for the exact distance
    float* xrow;             // the point's coordinates, zero padded to bf16_valid(D)
    float* tile;             // 64 x (chunk + 4) words
};

// Load one 16-byte piece (4 dimensions) of a candidate row, zero beyond D.
__device__ __forceinline__ float4 load_piece(const float* __restrict__ row, int d, int D, bool vec_ok)
{
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d < D) {
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

// Exact distances of the first n candidates of `list` to the point, then offer them.  CH = dimensions
// staged per step (32 or 16): a step moves 64 rows x CH floats through the tile.  tau_cap: a bound the caller
// knows for the row's final last slot (candidates above it need not be finished), else +inf.  DEEP: the loads of
// two steps are in flight while a third is being used (two register buffers that take turns, so that waiting for
// one does not wait for the other): for kernels with few wavefronts per SIMD, whose gathers would otherwise wait
// for each other.  GROUP: 16-byte pieces of a row whose reads from the tile are requested together (0: one at a time, the
// form that needs the fewest registers).
template <int SL, int CH = kChunk, bool DEEP = false, int GROUP = 0>
__device__ __forceinline__ void exact_batch(const ExploreLds& L, const int* list, int n,
                                            const float* __restrict__ points, int D, bool vec_ok, KnnRow<SL>& row,
                                            float tau_cap = INFINITY)
{
    constexpr int kPieces = CH / 4;         // 16-byte pieces of a row per step = lanes per row
    constexpr int kRows = 64 / kPieces;     // rows per load instruction
    constexpr int kLoads = 64 / kRows;      // load instructions per step
    constexpr int kP = CH + 4;              // tile pitch: odd number of 16-byte units
    const int lane = lane_id();
    const int sub = lane / kPieces;         // which of the rows of a load instruction
    const int piece = lane % kPieces;       // which 16-byte piece of the segment
    const int my_c = lane < n ? list[lane] : -1;
    const float* rp[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int r = i * kRows + sub;
        rp[i] = r < n ? points + (size_t)list[r] * (size_t)D : nullptr;    // nothing is read for the rows beyond n
    }
    float4 pre[DEEP ? 2 : 1][kLoads];
    auto request = [&](float4 (&buf)[kLoads], int d0) {
        if (d0 < D) {
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                buf[i] = rp[i] ? load_piece(rp[i], d0 + piece * 4, D, vec_ok) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    float acc = 0.0f;
    const float tau0 = fminf(row.tau, tau_cap);
    // one step: the buffer's values (dimensions d0 ..) go through the tile, the buffer is refilled with the step
    // `ahead` dimensions later, the chains advance.  Returns false when no candidate can enter any more.
    auto step = [&](float4 (&buf)[kLoads], int d0, int ahead) {
        wave_lds_sync();                 // previous step's tile reads are done
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
            *reinterpret_cast<float4*>(&L.tile[(i * kRows + sub) * kP + piece * 4]) = buf[i];
        request(buf, d0 + ahead);
        wave_lds_sync();
        const int pieces = min(kPieces, (D - d0 + 3) >> 2);
        const float* mine = &L.tile[lane * kP];
        const float* xs = &L.xrow[d0];
        auto chain4 = [&](const float4& a, const float4& x) {
            float df;
            df = a.x - x.x; acc = __builtin_fmaf(df, df, acc);
            df = a.y - x.y; acc = __builtin_fmaf(df, df, acc);
            df = a.z - x.z; acc = __builtin_fmaf(df, df, acc);
            df = a.w - x.w; acc = __builtin_fmaf(df, df, acc);
        };
        if (GROUP > 0 && pieces == kPieces) {
            // a whole step: the reads of the tile and of the point for 4 GROUP dimensions are requested together, so
            // that the chain waits for LDS once per group and not once per four dimensions (8 GROUP registers)
            constexpr int kGroup = GROUP > 0 ? GROUP : 1;
            static_assert(kPieces % kGroup == 0, "a step is a whole number of groups");
#pragma unroll
            for (int q0 = 0; q0 < kPieces; q0 += kGroup) {
                float4 a[kGroup], x[kGroup];
#pragma unroll
                for (int q = 0; q < kGroup; ++q) {
                    a[q] = *reinterpret_cast<const float4*>(mine + 4 * (q0 + q));
                    x[q] = *reinterpret_cast<const float4*>(xs + 4 * (q0 + q));
                }
#pragma unroll
                for (int q = 0; q < kGroup; ++q) chain4(a[q], x[q]);
            }
        } else {
            for (int q = 0; q < pieces; ++q)
                chain4(*reinterpret_cast<const float4*>(mine + 4 * q), *reinterpret_cast<const float4*>(xs + 4 * q));
        }
        // partial sums only grow: once all of them are above the row maximum nothing can enter
        return ballot64(lane < n && acc <= tau0) != 0;
    };
    bool finished = true;
    request(pre[0], 0);
    if (DEEP) {
        request(pre[1], CH);
        for (int d0 = 0; d0 < D; d0 += 2 * CH) {
            if (!step(pre[0], d0, 2 * CH)) { finished = false; break; }
            if (d0 + CH < D && !step(pre[1], d0 + CH, 2 * CH)) { finished = false; break; }
        }
    } else {
        for (int d0 = 0; d0 < D; d0 += CH)
            if (!step(pre[0], d0, CH)) { finished = false; break; }
    }
    wave_lds_sync();
    row.merge(lane < n && finished, my_c, acc);          // unfinished sums are all above the last slot
}

// The same without the tile: lane l reads the row of candidate l itself, 32 dimensions (eight 16-byte pieces) per
// step, and runs its chain from registers; the point's coordinates come from L.xrow (every lane reads the same
// word).  For short rows: no LDS besides xrow, no synchronisation inside the batch.
template <int SL>
__device__ __forceinline__ void exact_direct(const ExploreLds& L, const int* list, int n, const float* __restrict__ points,
                                             int D, bool vec_ok, KnnRow<SL>& row, float tau_cap = INFINITY)
{
    const int lane = lane_id();
    const int my_c = lane < n ? list[lane] : -1;
    const float* rp = points + (size_t)(my_c >= 0 ? my_c : 0) * (size_t)D;
    float acc = 0.0f;
    const float tau0 = fminf(row.tau, tau_cap);
    bool finished = true;
    for (int d0 = 0; d0 < D; d0 += 32) {
        float4 v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            v[i] = my_c >= 0 ? load_piece(rp, d0 + 4 * i, D, vec_ok) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (d0 + 4 * i < D) {                         // (wave-uniform; xrow is zero beyond D like the pieces)
                const float4 x = *reinterpret_cast<const float4*>(&L.xrow[d0 + 4 * i]);
                float df;
                df = v[i].x - x.x; acc = __builtin_fmaf(df, df, acc);
                df = v[i].y - x.y; acc = __builtin_fmaf(df, df, acc);
                df = v[i].z - x.z; acc = __builtin_fmaf(df, df, acc);
                df = v[i].w - x.w; acc = __builtin_fmaf(df, df, acc);
            }
        }
        // partial sums only grow: once all of them are above the row maximum nothing can enter
        if (ballot64(lane < n && acc <= tau0) == 0) { finished = false; break; }
    }
    row.merge(lane < n && finished, my_c, acc);          // unfinished sums are all above the last slot
}

}  // namespace rsfk
