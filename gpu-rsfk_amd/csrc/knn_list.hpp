// A point's K-NN list held by one wavefront: slot k lives in lane k%64,
// register k/64 ("K divided over the lanes").
//
// The update rule is the reference's: a candidate enters iff it is strictly
// closer than the current maximum and its index is not already in the row, and
// it then displaces the maximum (src/kernels/compute_knn_from_buckets.cu:1215-1230,
// src/kernels/nearest_neighbors_exploring.cu:124-141).  The reference keeps a
// row unordered and rescans it for the new maximum after every insertion; here a
// row is kept sorted by distance (ascending), so the maximum is the last slot
// and an insertion is a one-lane shift of the tail (DPP wave_shr:1) -- no
// reduction per insertion.  Rows that arrive unsorted (anything the caller
// passes in) are detected on load and rebuilt by insertion; rows are always
// written back sorted.  Slot positions are not part of the interface.
#pragma once
#include "wave64.hpp"
#include <cmath>

namespace rsfk {

template <int SL>
struct KnnRow {
    int idx[SL];
    float dist[SL];
    float tau;        // distance in slot K-1 = current maximum of the row (wave-uniform)
    int kk;           // K
    bool changed;     // wave-uniform

    __device__ __forceinline__ float last_slot() const
    {
        const int k = kk - 1;
        float t = read_lane_f(dist[0], k & 63);
#pragma unroll
        for (int s = 1; s < SL; ++s)
            if ((k >> 6) == s) t = read_lane_f(dist[s], k & 63);
        return t;
    }

    // Insert (c, d) at its sorted position; the last slot falls off.  Requires d < tau.
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
            if (s + 1 < SL) { carry_d = read_lane_f(dist[s], 63); carry_i = read_lane_i(idx[s], 63); }
            const bool gt = dist[s] > d && lane + s * kWave < kk;   // this slot moves up (or receives the candidate)
            const bool from_below = sd > d;           // the slot below moves up into this one
            const float nd = from_below ? sd : d;
            const int ni = from_below ? si : c;
            dist[s] = gt ? nd : dist[s];
            idx[s] = gt ? ni : idx[s];
        }
        tau = last_slot();
        changed = true;
    }

    // values already in registers and known to be sorted
    __device__ __forceinline__ void init_sorted(int K)
    {
        kk = K;
        changed = false;
        tau = last_slot();
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
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            float below = wave_shr1_f(dist[s]);
            if (s > 0 && lane == 0) below = carry;
            if (s + 1 < SL) carry = read_lane_f(dist[s], 63);
            bad |= dist[s] < below;
        }
        if (ballot64(bad) == 0) {
            tau = last_slot();
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
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            for (int l = 0; l < kWave; ++l) {
                if (s * kWave + l >= K) break;
                const float d = read_lane_f(od[s], l);
                const int c = read_lane_i(oi[s], l);
                if (d < tau) insert_sorted(c, d);
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
        if (!(d < tau)) return;
        if (CHECK_DUP) {
            bool mine = false;
#pragma unroll
            for (int s = 0; s < SL; ++s) mine |= (idx[s] == c);
            if (ballot64(mine) != 0) return;
        }
        insert_sorted(c, d);
    }

    // Up to 64 candidates, one per lane (ok = this lane holds one).  They are
    // offered in lane order; the threshold is re-read after every insertion.
    template <bool CHECK_DUP = true>
    __device__ __forceinline__ void offer_lanes(bool ok, int c, float d)
    {
        uint64_t pend = ballot64(ok && d < tau);
        while (pend != 0) {
            const int j = first_lane(pend);
            pend &= pend - 1;
            const float dj = read_lane_f(d, j);
            const int cj = read_lane_i(c, j);
            offer<CHECK_DUP>(cj, dj);
        }
    }
};

}  // namespace rsfk
