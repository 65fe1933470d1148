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
// The reference keeps a row unordered and rescans it for the new maximum after
// every insertion; here a row is kept sorted ascending by (distance, index), so
// the maximum is the last slot and an insertion is a one-lane shift of the tail
// (DPP wave_shr:1).  The slots above a candidate form a suffix of the row, so one
// comparison per slot gives the mask of the lanes that change, and that mask
// shifted by one gives the lanes that take the value of the slot below: no
// reduction and no re-reading of the maximum between the candidates of a batch.
// (Merging a batch by ranking -- a count per candidate and per slot, then one
// scatter -- was measured slower: about as many vector instructions per accepted
// candidate and three times the scalar ones.)
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

// Comparisons as masks over the wavefront (one bit per lane), without a boolean per lane in between.
__device__ __forceinline__ uint64_t mask_eq_i(int a, int b) { return __builtin_amdgcn_sicmp(a, b, 32 /* eq */); }
__device__ __forceinline__ uint64_t mask_pair_above(float d1, int c1, float d2, int c2)
{
    return __builtin_amdgcn_fcmpf(d1, d2, 2 /* ordered > */) |
           (__builtin_amdgcn_fcmpf(d1, d2, 1 /* ordered == */) & __builtin_amdgcn_sicmp(c1, c2, 38 /* signed > */));
}
// this lane's bit of a mask
__device__ __forceinline__ bool lane_bit(uint64_t mask) { return __builtin_amdgcn_inverse_ballot_w64(mask); }

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

    // Insert the wave-uniform candidate (c, d), finite and not in the row, at its place; the last slot falls off.
    // Returns false (and changes nothing) when the candidate is above the last slot.  tau / tau_i are not refreshed.
    __device__ __forceinline__ bool insert_at_place(int c, float d)
    {
        uint64_t above[SL];
        uint64_t any = 0;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            above[s] = mask_pair_above(dist[s], idx[s], d, c);
            const int live = kk - s * kWave;                 // slots of this register that belong to the row
            if (live < kWave) above[s] &= live > 0 ? ((1ull << live) - 1) : 0;
            any |= above[s];
        }
        if (any == 0) return false;
        float nd[SL];
        int ni[SL];
        uint64_t carry = 0;                                  // the last slot of the register below moves up too
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const uint64_t from_below = (above[s] << 1) | carry;
            carry = above[s] >> 63;
            float sd = wave_shr1_f(dist[s]);                 // lane l <- lane l-1
            int si = wave_shr1_i(idx[s]);
            if (s > 0) {
                const float bd = read_lane_f(dist[s - 1], 63);
                const int bi = read_lane_i(idx[s - 1], 63);
                sd = lane_bit(1ull) ? bd : sd;
                si = lane_bit(1ull) ? bi : si;
            }
            const float md = lane_bit(from_below) ? sd : d;
            const int mi = lane_bit(from_below) ? si : c;
            nd[s] = lane_bit(above[s]) ? md : dist[s];
            ni[s] = lane_bit(above[s]) ? mi : idx[s];
        }
#pragma unroll
        for (int s = 0; s < SL; ++s) { dist[s] = nd[s]; idx[s] = ni[s]; }
        return true;
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
        // rebuild: the old entries are merged into an empty row
        int oi[SL];
        float od[SL];
        bool okv[SL];
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            oi[s] = idx[s];
            od[s] = dist[s];
            const bool live = lane + s * kWave < K;
            okv[s] = live && oi[s] >= 0;
            idx[s] = live ? -1 : -2;
            dist[s] = INFINITY;
        }
        tau = INFINITY;
        tau_i = -1;
        merge<SL>(okv, oi, od);
        refresh_tau();
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

    // Merge a batch of up to 64 CL candidates -- candidate u of a lane is (c[u], d[u]), there iff ok[u] -- into the
    // row.  The candidates below the last slot are taken in lane order; one that the row holds already (by index), or
    // that is no longer below the last slot when its turn comes, is dropped.  A point may occur more than once in a
    // batch: its second occurrence finds it in the row.
    template <int CL>
    __device__ __forceinline__ void merge(const bool (&ok)[CL], const int (&c)[CL], const float (&d)[CL])
    {
        bool any_in = false;
#pragma unroll
        for (int u = 0; u < CL; ++u) {
            uint64_t todo = ballot64(ok[u] && enters(c[u], d[u]));
            while (todo != 0) {
                const int j = first_lane(todo);
                todo &= todo - 1;
                const float dj = read_lane_f(d[u], j);
                const int cj = read_lane_i(c[u], j);
                uint64_t same = 0;
#pragma unroll
                for (int s = 0; s < SL; ++s) same |= mask_eq_i(idx[s], cj);
                if (same != 0) continue;
                if (insert_at_place(cj, dj)) any_in = true;
            }
        }
        if (any_in) {
            refresh_tau();
            changed = true;
        }
    }

    __device__ __forceinline__ void merge(bool ok, int c, float d)
    {
        const bool okv[1] = {ok};
        const int cv[1] = {c};
        const float dv[1] = {d};
        merge<1>(okv, cv, dv);
    }
};

}  // namespace rsfk
