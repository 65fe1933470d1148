// A point's K-NN list held by one wavefront: slot k lives in lane k%64,
// register k/64 ("K divided over the lanes").  The insertion rule is the
// reference's: a candidate replaces the current maximum iff it is strictly
// closer and its index is not already in the row
// (src/kernels/compute_knn_from_buckets.cu:1215-1230,
//  src/kernels/nearest_neighbors_exploring.cu:124-141).
#pragma once
#include "wave64.hpp"
#include <cmath>

namespace rsfk {

template <int SL>
struct KnnRow {
    int idx[SL];
    float dist[SL];
    float tau;        // current maximum of the row (wave-uniform)
    bool changed;     // wave-uniform

    __device__ __forceinline__ void load(const int* __restrict__ gidx, const float* __restrict__ gdist, int K)
    {
        const int lane = lane_id();
        float m = -INFINITY;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            int k = lane + s * kWave;
            if (k < K) { idx[s] = gidx[k]; dist[s] = gdist[k]; }
            else       { idx[s] = -2;      dist[s] = -INFINITY; }
            m = fmaxf(m, dist[s]);
        }
        tau = wave_max(m);
        changed = false;
    }

    __device__ __forceinline__ void store(int* __restrict__ gidx, float* __restrict__ gdist, int K) const
    {
        const int lane = lane_id();
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            int k = lane + s * kWave;
            if (k < K) { gidx[k] = idx[s]; gdist[k] = dist[s]; }
        }
    }

    // wave-uniform candidate (c, d).  Caller has checked nothing.
    __device__ __forceinline__ void offer(int c, float d)
    {
        if (!(d < tau)) return;
        bool mine = false;
#pragma unroll
        for (int s = 0; s < SL; ++s) mine |= (idx[s] == c);
        if (ballot64(mine) != 0) return;
        const int lane = lane_id();
        bool done = false;
        float m = -INFINITY;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            if (!done) {
                uint64_t at = ballot64(dist[s] == tau);
                if (at != 0) {
                    if (lane == first_lane(at)) { idx[s] = c; dist[s] = d; }
                    done = true;
                }
            }
            m = fmaxf(m, dist[s]);
        }
        tau = wave_max(m);
        changed = true;
    }

    // Up to 64 candidates, one per lane (ok = this lane holds one).  They are
    // offered in lane order; the threshold is re-read after every insertion.
    __device__ __forceinline__ void offer_lanes(bool ok, int c, float d)
    {
        uint64_t pend = ballot64(ok && d < tau);
        while (pend != 0) {
            const int j = first_lane(pend);
            pend &= pend - 1;
            const float dj = read_lane_f(d, j);
            const int cj = read_lane_i(c, j);
            offer(cj, dj);
        }
    }
};

}  // namespace rsfk
