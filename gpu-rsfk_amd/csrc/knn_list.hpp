// A point's K-NN list held by one wavefront: slot k lives in lane k%64,
// register k/64 ("K divided over the lanes").
//
// Update rule.  The reference lets a candidate enter iff it is strictly closer
// than the current maximum and its index is not already in the row, and the
// candidate then displaces the maximum (src/kernels/compute_knn_from_buckets.cu:1215-1230,
// src/kernels/nearest_neighbors_exploring.cu:124-141); which of several points at
// exactly the K-th distance a row ends with then depends on the order of arrival.
// Here entries are ordered by (distance, index) and a candidate enters iff its
// (distance, index) is below the row's largest (distance, index) and its index is
// not in the row: the row always holds the K smallest (distance, index) pairs of
// everything it was offered, whatever the order.  The two rules give the same
// rows except among points tied at a row's K-th distance, where this one keeps
// the smaller index.  A candidate at +inf (or NaN) never enters, as in the
// reference.
//
// A row is kept sorted ascending by (distance, index), so the maximum is the last
// slot.  A batch of up to 64 candidates per register (one per lane) is merged by
// ranking, not by repeated insertion: for every candidate that may enter, one
// pass counts the row slots above it (a ballot and a population count) and bumps
// a per-slot and a per-candidate counter; afterwards every row slot and every
// candidate knows its place in the merged row and moves there in one step.
// Rows that arrive unsorted (anything the caller passes in) are detected on load
// and rebuilt; rows are always written back sorted.  Slot positions are not part
// of the interface.
#pragma once
#include "wave64.hpp"
#include <cmath>

namespace rsfk {

// (d1, c1) above (d2, c2) in the order of the rows
__device__ __forceinline__ bool pair_above(float d1, int c1, float d2, int c2)
{
    return d1 > d2 || (d1 == d2 && c1 > c2);
}

template <int SL>
struct KnnRow {
    int idx[SL];      // slots >= K hold (-2, +inf)
    float dist[SL];
    float tau;        // distance in slot K-1 = current maximum of the row (wave-uniform)
    int tau_i;        // index in slot K-1
    int kk;           // K
    bool changed;     // wave-uniform

    __device__ __forceinline__ void refresh_tau()
    {
        const int k = kk - 1;
        float t = read_lane_f(dist[0], k & 63);
        int ti = read_lane_i(idx[0], k & 63);
#pragma unroll
        for (int s = 1; s < SL; ++s)
            if ((k >> 6) == s) { t = read_lane_f(dist[s], k & 63); ti = read_lane_i(idx[s], k & 63); }
        tau = t;
        tau_i = ti;
    }

    // may (c, d) enter the row?  (the index test comes on top)
    __device__ __forceinline__ bool enters(int c, float d) const
    {
        return d < INFINITY && (d < tau || (d == tau && c < tau_i));
    }

    // Insert (c, d) at its sorted position; the last slot falls off.  Requires enters(c, d).
    __device__ __forceinline__ void insert_sorted(int c, float d)
    {
        const int lane = lane_id();
        float carry_d = 0.0f;
        int carry_i = 0;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            float sd = wave_shr1_f(dist[s]);          // lane l <- lane l-1, lane 0 <- 0
            int si = wave_shr1_i(idx[s]);
            if (s > 0 && lane == 0) { sd = carry_d; si = carry_i; }
            if (s == 0 && lane == 0) si = -3;         // nothing below slot 0
            if (s + 1 < SL) { carry_d = read_lane_f(dist[s], 63); carry_i = read_lane_i(idx[s], 63); }
            const bool gt = pair_above(dist[s], idx[s], d, c) && lane + s * kWave < kk;   // this slot moves up (or receives the candidate)
            const bool from_below = pair_above(sd, si, d, c);                             // the slot below moves up into this one
            const float nd = from_below ? sd : d;
            const int ni = from_below ? si : c;
            dist[s] = gt ? nd : dist[s];
            idx[s] = gt ? ni : idx[s];
        }
        refresh_tau();
        changed = true;
    }

    // values already in registers and known to be sorted
    __device__ __forceinline__ void init_sorted(int K)
    {
        kk = K;
        changed = false;
        refresh_tau();
    }

    // values already in registers (slot k = lane + 64*s); slots >= K must hold (-2, +inf)
    __device__ __forceinline__ void init_from_regs(int K)
    {
        kk = K;
        changed = false;
        const int lane = lane_id();
        // sorted already?  (distances are >= 0, the lane below lane 0 reads as 0)
        bool bad = false;
        float carry = 0.0f;
        int carry_i = -3;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            float below = wave_shr1_f(dist[s]);
            int below_i = wave_shr1_i(idx[s]);
            if (lane == 0) { below = carry; below_i = carry_i; }
            if (s + 1 < SL) { carry = read_lane_f(dist[s], 63); carry_i = read_lane_i(idx[s], 63); }
            bad |= lane + s * kWave < K && pair_above(below, below_i, dist[s], idx[s]);
        }
        if (ballot64(bad) == 0) {
            refresh_tau();
            return;
        }
        // rebuild by insertion into an empty row
        int oi[SL];
        float od[SL];
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            oi[s] = idx[s];
            od[s] = dist[s];
            const bool live = lane + s * kWave < K;
            idx[s] = live ? -1 : -2;
            dist[s] = INFINITY;
        }
        tau = INFINITY;
        tau_i = -1;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            for (int l = 0; l < kWave; ++l) {
                if (s * kWave + l >= K) break;
                const float d = read_lane_f(od[s], l);
                const int c = read_lane_i(oi[s], l);
                offer<true>(c, d);
            }
        }
        changed = true;
    }

    __device__ __forceinline__ void load(const int* __restrict__ gidx, const float* __restrict__ gdist, int K)
    {
        const int lane = lane_id();
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            int k = lane + s * kWave;
            if (k < K) { idx[s] = gidx[k]; dist[s] = gdist[k]; }
            else       { idx[s] = -2;      dist[s] = INFINITY; }
        }
        init_from_regs(K);
    }

    __device__ __forceinline__ void store(int* __restrict__ gidx, float* __restrict__ gdist) const
    {
        const int lane = lane_id();
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            int k = lane + s * kWave;
            if (k < kk) { gidx[k] = idx[s]; gdist[k] = dist[s]; }
        }
    }

    // wave-uniform candidate (c, d); CHECK_DUP = the row may already hold c
    template <bool CHECK_DUP>
    __device__ __forceinline__ void offer(int c, float d)
    {
        if (!enters(c, d)) return;
        if (CHECK_DUP) {
            bool mine = false;
#pragma unroll
            for (int s = 0; s < SL; ++s) mine |= (idx[s] == c);
            if (ballot64(mine) != 0) return;
        }
        insert_sorted(c, d);
    }

    // Ranks up to 64 CL candidates -- candidate u of a lane is (c[u], d[u]), there iff ok[u] -- against the row and
    // against each other.  Result: acc[u] = lanes whose candidate u is new to the row and below its last slot;
    // shift[s] = how many of those lie below slot (s, lane); pos[u] = place of this lane's candidate u in the merged
    // sequence (meaningful where acc[u] has the lane's bit).  The merged sequence is cut at K by the caller.
    // Returns false when no candidate enters.
    template <int CL>
    __device__ __forceinline__ bool rank(const bool (&ok)[CL], const int (&c)[CL], const float (&d)[CL], uint64_t (&acc)[CL],
                                         int (&shift)[SL], int (&pos)[CL]) const
    {
        uint64_t any = 0;
#pragma unroll
        for (int u = 0; u < CL; ++u) {
            acc[u] = ballot64(ok[u] && enters(c[u], d[u]));
            any |= acc[u];
        }
        if (any == 0) return false;
        const int lane = lane_id();
        int rr[CL];           // slots of the row below the candidate
#pragma unroll
        for (int s = 0; s < SL; ++s) shift[s] = 0;
#pragma unroll
        for (int u = 0; u < CL; ++u) { pos[u] = 0; rr[u] = 0; }
        const bool several = CL > 1 || (any & (any - 1)) != 0;
        int n_acc = 0;
#pragma unroll
        for (int u = 0; u < CL; ++u) {
            uint64_t todo = acc[u];
            while (todo != 0) {
                const int j = first_lane(todo);
                todo &= todo - 1;
                const float dj = read_lane_f(d[u], j);
                const int cj = read_lane_i(c[u], j);
                // the row holds it, or an earlier candidate of this batch is the same point
                bool mine = false;
#pragma unroll
                for (int s = 0; s < SL; ++s) mine |= (idx[s] == cj);
                uint64_t same = ballot64(mine);
                if (several) {
#pragma unroll
                    for (int u2 = 0; u2 <= u; ++u2) {
                        const uint64_t earlier = u2 < u ? acc[u2] : (acc[u] & ((1ull << j) - 1));
                        same |= ballot64(c[u2] == cj) & earlier;
                    }
                }
                if (same != 0) {
                    acc[u] &= ~(1ull << j);
                    continue;
                }
                int above = 0;
#pragma unroll
                for (int s = 0; s < SL; ++s) {
                    const bool ab = pair_above(dist[s], idx[s], dj, cj);
                    shift[s] += ab ? 1 : 0;
                    above += __popcll(ballot64(ab));
                }
                rr[u] = lane == j ? kWave * SL - above : rr[u];
                if (several) {
#pragma unroll
                    for (int u2 = 0; u2 < CL; ++u2) pos[u2] += pair_above(d[u2], c[u2], dj, cj) ? 1 : 0;
                }
                ++n_acc;
            }
        }
#pragma unroll
        for (int u = 0; u < CL; ++u) pos[u] += rr[u];
        return n_acc > 0;
    }

    // Merge a batch into the row held in registers.  scratch: 2 * 64 * SL ints of LDS that belong to this wavefront
    // for the duration of the call (the caller orders its own earlier accesses to them with wave_lds_sync()).
    // The candidates of one batch are distinct points or exact repeats (same index, same distance).
    template <int CL>
    __device__ __forceinline__ void merge(const bool (&ok)[CL], const int (&c)[CL], const float (&d)[CL], int* scratch)
    {
        uint64_t acc[CL];
        int shift[SL], pos[CL];
        if (!rank<CL>(ok, c, d, acc, shift, pos)) return;
        const int lane = lane_id();
        int* s_idx = scratch;
        int* s_dist = scratch + kWave * SL;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const int k2 = lane + s * kWave + shift[s];
            if (k2 < kk) { s_idx[k2] = idx[s]; s_dist[k2] = __float_as_int(dist[s]); }
        }
#pragma unroll
        for (int u = 0; u < CL; ++u)
            if (((acc[u] >> lane) & 1) != 0 && pos[u] < kk) { s_idx[pos[u]] = c[u]; s_dist[pos[u]] = __float_as_int(d[u]); }
        wave_lds_sync();
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const int k = lane + s * kWave;
            if (k < kk) { idx[s] = s_idx[k]; dist[s] = __int_as_float(s_dist[k]); }
        }
        wave_lds_sync();
        refresh_tau();
        changed = true;
    }

    __device__ __forceinline__ void merge(bool ok, int c, float d, int* scratch)
    {
        const bool okv[1] = {ok};
        const int cv[1] = {c};
        const float dv[1] = {d};
        merge<1>(okv, cv, dv, scratch);
    }

    // Merge a batch and write the resulting row to memory; the registers are not updated (last use of the row).
    // Only the slots that change are written, unless the row was rebuilt on load.
    template <int CL>
    __device__ __forceinline__ void merge_store(const bool (&ok)[CL], const int (&c)[CL], const float (&d)[CL],
                                                int* __restrict__ gidx, float* __restrict__ gdist)
    {
        uint64_t acc[CL];
        int shift[SL], pos[CL];
        if (!rank<CL>(ok, c, d, acc, shift, pos)) {
            if (changed) store(gidx, gdist);
            return;
        }
        const int lane = lane_id();
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const int k2 = lane + s * kWave + shift[s];
            if ((shift[s] > 0 || changed) && k2 < kk) { gidx[k2] = idx[s]; gdist[k2] = dist[s]; }
        }
#pragma unroll
        for (int u = 0; u < CL; ++u)
            if (((acc[u] >> lane) & 1) != 0 && pos[u] < kk) { gidx[pos[u]] = c[u]; gdist[pos[u]] = d[u]; }
    }
};

}  // namespace rsfk
