// Wavefront-level primitives for gfx950 (64 lanes per wavefront).
//
// Cross-lane data movement uses DPP modifiers (quad_perm / row_half_mirror /
// row_mirror, no LDS traffic) inside a row of 16 lanes and v_readlane across
// rows.  All of them require every lane of the wavefront to be active; they
// are only called from wave-uniform control flow.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace rsfk {

constexpr int kWave = 64;

__device__ __forceinline__ int lane_id()
{
    return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0));
}

__device__ __forceinline__ uint64_t ballot64(bool pred) { return __ballot(pred); }

// number of set bits of mask below the calling lane
__device__ __forceinline__ int mask_prefix(uint64_t mask)
{
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
}

__device__ __forceinline__ int first_lane(uint64_t mask) { return __ffsll((unsigned long long)mask) - 1; }

__device__ __forceinline__ float read_lane_f(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ int read_lane_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }

// DPP controls
constexpr int kDppXor1 = 0xB1;          // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;          // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;   // lane i <-> 7-i inside each group of 8
constexpr int kDppMirror = 0x140;       // lane i <-> 15-i inside each row of 16

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}

// lane l <- lane l-1 across the whole wavefront, lane 0 <- 0
__device__ __forceinline__ float wave_shr1_f(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x138, 0xf, 0xf, true));
}
__device__ __forceinline__ int wave_shr1_i(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, 0x138, 0xf, 0xf, true);
}

// Sum over the 32 lanes of each half of the wavefront with the addition tree of
// the xor butterfly 1,2,4,8,16 of a 32-wide warp reduction
// (src/kernels/build_tree_check_points_side.cu:139-143); every lane of a half
// ends with the same bits.  After the xor-1 and xor-2 steps the four lanes of a
// quad hold identical bits, so the partner of the xor-4 step may be any lane of
// the other quad of the group of 8 (row_half_mirror picks lane 7-i); likewise
// row_mirror serves the xor-8 step.  The xor-16 step adds the two row sums of
// the half (a+b and b+a round identically).
__device__ __forceinline__ float half_butterfly_sum(float v)
{
    v += dpp_f<kDppXor1>(v);
    v += dpp_f<kDppXor2>(v);
    v += dpp_f<kDppHalfMirror>(v);
    v += dpp_f<kDppMirror>(v);
    const float r0 = read_lane_f(v, 0), r1 = read_lane_f(v, 16);
    const float r2 = read_lane_f(v, 32), r3 = read_lane_f(v, 48);
    const float lo = r0 + r1, hi = r2 + r3;
    return lane_id() < 32 ? lo : hi;
}

// maximum over all 64 lanes, returned in every lane (wave-uniform value)
__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, dpp_f<kDppXor1>(v));
    v = fmaxf(v, dpp_f<kDppXor2>(v));
    v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f<kDppMirror>(v));
    const float r0 = read_lane_f(v, 0), r1 = read_lane_f(v, 16);
    const float r2 = read_lane_f(v, 32), r3 = read_lane_f(v, 48);
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// Orders LDS accesses of one wavefront as seen by its own lanes.  The hardware
// executes a wavefront's LDS operations in order; this only keeps the compiler
// from moving LDS accesses across the point.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ int wave_sum_i(int v)
{
    v += dpp_i<kDppXor1>(v);
    v += dpp_i<kDppXor2>(v);
    v += dpp_i<kDppHalfMirror>(v);
    v += dpp_i<kDppMirror>(v);
    return read_lane_i(v, 0) + read_lane_i(v, 16) + read_lane_i(v, 32) + read_lane_i(v, 48);
}

// bitwise or over all 64 lanes, returned in every lane (wave-uniform value)
__device__ __forceinline__ uint32_t wave_or_u32(uint32_t x)
{
    int v = (int)x;
    v |= dpp_i<kDppXor1>(v);
    v |= dpp_i<kDppXor2>(v);
    v |= dpp_i<kDppHalfMirror>(v);
    v |= dpp_i<kDppMirror>(v);
    return (uint32_t)(read_lane_i(v, 0) | read_lane_i(v, 16) | read_lane_i(v, 32) | read_lane_i(v, 48));
}

// exclusive prefix sum over the lanes of the wavefront
__device__ __forceinline__ int wave_excl_scan_i(int v)
{
    const int lane = lane_id();
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
    }
    return incl - v;
}

}  // namespace rsfk
