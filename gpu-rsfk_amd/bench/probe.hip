// Measurement aid: the gather of scattered rows on its own.
//
// The bucket K-NN kernels read every point of a tree's buckets once, in the order of the tree's permutation: rows of
// 4 D bytes at scattered places (compute_knn_from_buckets.cu:1035-1099 reads them the same way, lane by lane).  How
// fast the device delivers such rows bounds those kernels from below whatever they compute; this kernel does nothing
// else -- one wavefront per row, 16-byte pieces, eight rows in flight per wavefront -- so that bench.py can report the
// rate next to the rate of the bucket kernel.
//
// Built into its own small shared library (librsfk_probe.so, next to this file): it is an aid of the benchmark and
// not part of the product's interface, so librsfk.so neither contains nor exports it.
#include <hip/hip_runtime.h>
#include <cstdint>

namespace {

constexpr int kProbeBlocks = 4096;

__global__ __launch_bounds__(256) void k_probe_gather(const float* __restrict__ points, int N, int D,
                                                      const int* __restrict__ ids, long long n_ids, float* __restrict__ sums)
{
    __shared__ float part[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long n_waves = (long long)gridDim.x * 4;
    const long long w = (long long)blockIdx.x * 4 + wave;
    const bool vec = (D & 3) == 0 && ((reinterpret_cast<uintptr_t>(points) & 15) == 0);
    float acc = 0.0f;
    for (long long r0 = w * 8; r0 < n_ids; r0 += n_waves * 8) {
        int id[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            id[u] = r0 + u < n_ids ? ids[r0 + u] : -1;
            if (id[u] >= N) id[u] = -1;
        }
        if (vec) {
            for (int d = 4 * lane; d < D; d += 256) {
                float4 v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    v[u] = id[u] >= 0 ? *reinterpret_cast<const float4*>(points + (size_t)id[u] * (size_t)D + d)
                                      : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int u = 0; u < 8; ++u) acc += (v[u].x + v[u].y) + (v[u].z + v[u].w);
            }
        } else {
            for (int d = lane; d < D; d += 64) {
#pragma unroll
                for (int u = 0; u < 8; ++u) acc += id[u] >= 0 ? points[(size_t)id[u] * (size_t)D + d] : 0.0f;
            }
        }
    }
    acc += __shfl_xor(acc, 1, 64); acc += __shfl_xor(acc, 2, 64); acc += __shfl_xor(acc, 4, 64);
    acc += __shfl_xor(acc, 8, 64); acc += __shfl_xor(acc, 16, 64); acc += __shfl_xor(acc, 32, 64);
    if (lane == 0) part[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) sums[blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
}

}  // namespace

// Reads the rows ids[0..n_ids) of the N x D matrix d_points once (ids >= N are skipped) and adds them up into
// d_sums (one float per workgroup launched: at least 4096 floats).  stream: a hipStream_t or null.
// Returns 0, 1 on a launch error, 2 on bad arguments.
extern "C" __attribute__((visibility("default"))) int rsfk_probe_gather_device(const float* d_points, int N, int D,
                                                                               const int* d_ids, long long n_ids,
                                                                               float* d_sums, void* stream)
{
    if (N < 1 || D < 1 || n_ids < 0 || !d_points || !d_ids || !d_sums) return 2;
    hipLaunchKernelGGL(k_probe_gather, dim3(kProbeBlocks), dim3(256), 0, static_cast<hipStream_t>(stream), d_points, N, D,
                       d_ids, n_ids, d_sums);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}
