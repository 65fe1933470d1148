// Bucket K-NN for buckets of at most 64 points (two wavefronts per bucket) or of
// 65..72 points (three) and K <= 64: the shapes the default parameters (bucket size
// K+1 .. 2(K+1), K <= 32) produce.  Same function as the general kernel in
// bucket_knn.hip (see there for the reference kernels it replaces).
//
//   1. the rows of the bucket, 64 dimensions at a time, are requested from HBM at
//      once and written to LDS; a row is read by consecutive lanes, 16 bytes each
//      (coalesced);
//   2. the pair matrix is cut into 2x2 blocks (members 2a, 2a+1 against 2b, 2b+1);
//      the blocks of the upper triangle are dealt out to the threads round by round
//      and a thread accumulates the 4 distances of a block with sequential fused
//      multiply-add chains (arithmetic of euclidean_distance_sqr,
//      compute_knn_from_buckets.cu:40-54).  Small blocks keep the lanes busy whatever
//      the bucket size: a bucket of 50 points has 325 blocks = 3 rounds of 128 threads,
//      where one 4x4 block per thread left 50 of 128 lanes idle for 16 distances;
//   3. the distance matrix replaces the rows in LDS; a wavefront owns every second
//      (third) point: per point, the candidates below the row's last slot are
//      inserted into the sorted row unless the row holds them already
//      (knn_list.hpp); the rows of the next four points are in flight meanwhile, and
//      points without any such candidate are skipped when the rows are known to be
//      sorted.
// Registers are kept near 100 and LDS near 20 KB per workgroup so that four
// wavefronts per SIMD are resident: the kernel alternates between an arithmetic
// phase and a latency-bound merge phase, and only other resident workgroups can
// fill the gaps.
#include "rsfk_common.hpp"
#include "knn_list.hpp"
#include "forest.hpp"
#include "bucket_small_body.hpp"

namespace rsfk {

namespace {

using namespace small_bucket;

template <int CAP, int THREADS, int SPACING>
__global__ __launch_bounds__(THREADS, 4) void k_bucket_knn_small(const float* __restrict__ points, int D, int K,
                                                                 const int* __restrict__ ids,
                                                                 const int* __restrict__ starts,
                                                                 const int* __restrict__ sizes, int stride, int min_size,
                                                                 int* __restrict__ knn_idx, float* __restrict__ knn_dist,
                                                                 int chunk, int pitch, int region_floats, int rows_sorted)
{
    extern __shared__ __align__(16) float lds_f[];
    small_bucket_body<CAP, THREADS, SPACING>(lds_f, points, D, K, ids, starts, sizes, stride, min_size, knn_idx, knn_dist, chunk,
                                             pitch, region_floats, rows_sorted, nullptr, 0);
}

}  // namespace

int small_bucket_cap() { return kBucketSplit; }
int medium_bucket_cap() { return 72; }

namespace {

template <int CAP, int THREADS, int SPACING>
int launch_cfg(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes, int n_buckets,
               int stride, int min_size, bool rows_sorted, int* knn_idx, float* knn_dist, hipStream_t stream)
{
    int chunk, pitch;
    small_bucket_shape(D, &chunk, &pitch);
    const int region_floats = small_bucket_region_floats<CAP, THREADS, SPACING>(pitch);
    const size_t lds = small_bucket_lds_bytes<CAP, THREADS, SPACING>(pitch);
    auto kern = k_bucket_knn_small<CAP, THREADS, SPACING>;
    RSFK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3((unsigned)n_buckets), dim3(THREADS), lds, stream, points, D, K, ids, starts, sizes, stride,
                       min_size, knn_idx, knn_dist, chunk, pitch, region_floats, rows_sorted ? 1 : 0);
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace

// Buckets of 2..64 points.  rows_sorted: every K-NN row is known to be sorted by distance (then members without
// a candidate below their last slot are skipped).
int launch_bucket_knn_small(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                            int n_buckets, int stride, bool rows_sorted, int* knn_idx, float* knn_dist, hipStream_t stream)
{
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 64, "small-bucket kernel: K must be in 1..64");
    return launch_cfg<64, 128, 33>(points, D, K, ids, starts, sizes, n_buckets, stride, 2, rows_sorted, knn_idx, knn_dist,
                                   stream);
}

// Buckets of 65..72 points (what a leaf limit of 2 (K + 1) with K = 32 leaves just above 64); other sizes are skipped.
int launch_bucket_knn_medium(const float* points, int D, int K, const int* ids, const int* starts, const int* sizes,
                             int n_buckets, int stride, bool rows_sorted, int* knn_idx, float* knn_dist, hipStream_t stream)
{
    if (n_buckets <= 0) return 0;
    RSFK_CHECK(K >= 1 && K <= 64, "small-bucket kernel: K must be in 1..64");
    return launch_cfg<72, 192, 37>(points, D, K, ids, starts, sizes, n_buckets, stride, 65, rows_sorted, knn_idx, knn_dist,
                                   stream);
}

}  // namespace rsfk
