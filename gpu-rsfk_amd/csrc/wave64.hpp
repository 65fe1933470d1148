// Wavefront-level primitives for gfx950 (64 lanes per wavefront).
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

// Sum over the 32 lanes of each half of the wavefront with the xor butterfly
// 1,2,4,8,16: every lane of a half ends with the same bits, and the tree of
// additions is the one of a 32-wide warp reduction
// (src/kernels/build_tree_check_points_side.cu:139-143).
__device__ __forceinline__ float half_butterfly_sum(float v)
{
    v += __shfl_xor(v, 1, kWave);
    v += __shfl_xor(v, 2, kWave);
    v += __shfl_xor(v, 4, kWave);
    v += __shfl_xor(v, 8, kWave);
    v += __shfl_xor(v, 16, kWave);
    return v;
}

// maximum over all 64 lanes, returned in every lane
__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, __shfl_xor(v, 1, kWave));
    v = fmaxf(v, __shfl_xor(v, 2, kWave));
    v = fmaxf(v, __shfl_xor(v, 4, kWave));
    v = fmaxf(v, __shfl_xor(v, 8, kWave));
    v = fmaxf(v, __shfl_xor(v, 16, kWave));
    v = fmaxf(v, __shfl_xor(v, 32, kWave));
    return v;
}

__device__ __forceinline__ int wave_sum_i(int v)
{
    v += __shfl_xor(v, 1, kWave);
    v += __shfl_xor(v, 2, kWave);
    v += __shfl_xor(v, 4, kWave);
    v += __shfl_xor(v, 8, kWave);
    v += __shfl_xor(v, 16, kWave);
    v += __shfl_xor(v, 32, kWave);
    return v;
}

}  // namespace rsfk
