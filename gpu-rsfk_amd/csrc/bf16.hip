#include "bf16.hpp"
#include "wave64.hpp"
#include <algorithm>

namespace rsfk {

namespace {

// one wavefront per row: convert, pad, and sum the squares of the rounded values
__global__ __launch_bounds__(256) void k_to_bf16(const float* __restrict__ points, uint16_t* __restrict__ out,
                                                 float* __restrict__ norms, int N, int D, int Db)
{
    const int lane = threadIdx.x & 63;
    const int wave_global = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int n_waves = (gridDim.x * blockDim.x) >> 6;
    for (int r = wave_global; r < N; r += n_waves) {
        const float* src = points + (size_t)r * (size_t)D;
        uint16_t* dst = out + (size_t)r * (size_t)Db;
        float q = 0.0f;
        for (int d = lane; d < Db; d += 64) {
            uint32_t u = d < D ? __float_as_uint(src[d]) : 0u;
            if ((u & 0x7f800000u) != 0x7f800000u) u += 0x7fffu + ((u >> 16) & 1u);      // finite: round to nearest even
            else if (u & 0x007fffffu) u |= 0x00400000u;                                  // NaN stays NaN
            u &= 0xffff0000u;
            dst[d] = (uint16_t)(u >> 16);
            const float v = __uint_as_float(u);
            q = __builtin_fmaf(v, v, q);
        }
        // any summation order will do: the consumers add a relative margin
        q += __shfl_xor(q, 1, 64); q += __shfl_xor(q, 2, 64); q += __shfl_xor(q, 4, 64);
        q += __shfl_xor(q, 8, 64); q += __shfl_xor(q, 16, 64); q += __shfl_xor(q, 32, 64);
        if (lane == 0) norms[r] = q;
    }
}

}  // namespace

size_t bf16_copy_bytes(int N, int D) { return (size_t)N * ((size_t)bf16_pitch(D) * 2 + 4); }

int bf16_copy_alloc(Bf16Copy* c, int N, int D)
{
    RSFK_HIP(hipMalloc(reinterpret_cast<void**>(&c->rows), std::max<size_t>((size_t)N * bf16_pitch(D) * 2, 16)));
    RSFK_HIP(hipMalloc(reinterpret_cast<void**>(&c->norms), std::max<size_t>((size_t)N * 4, 16)));
    return 0;
}

void bf16_copy_free(Bf16Copy* c)
{
    if (c->rows) (void)hipFree(c->rows);
    if (c->norms) (void)hipFree(c->norms);
    c->rows = nullptr;
    c->norms = nullptr;
}

int bf16_copy_fill(const Bf16Copy& c, const float* points, int N, int D, hipStream_t stream)
{
    const int grid = std::min((N + 3) / 4, 65536);
    hipLaunchKernelGGL(k_to_bf16, dim3(grid), dim3(256), 0, stream, points, c.rows, c.norms, N, D, bf16_pitch(D));
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
