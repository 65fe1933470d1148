// Shared definitions of the gfx950 RSFK library: error handling, the
// counter-based random numbers of the tree build and the record types that
// travel between the tree-build kernels, the bucket K-NN kernel and the host.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <string>

namespace rsfk {

// ---------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------
void set_last_error(const std::string& msg);
const char* last_error();

// workspace.hip: device memory for working buffers, kept for the next call after use
int ws_alloc(void** out, size_t bytes);
int ws_try_alloc(void** out, size_t bytes);      // optional block: fails quietly, releases nothing
void ws_free(void* p);
void ws_release_all();

// Both macros leave the function on failure.  Work that was queued before may still be running and the
// callers' guards hand their buffers back for reuse on the way out, so the device is drained first.
#define RSFK_HIP(call)                                                                   \
    do {                                                                                 \
        hipError_t e_ = (call);                                                          \
        if (e_ != hipSuccess) {                                                          \
            ::rsfk::set_last_error(std::string(#call) + ": " + hipGetErrorString(e_) +   \
                                   " (" __FILE__ ":" + std::to_string(__LINE__) + ")");  \
            (void)hipDeviceSynchronize();                                                \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

#define RSFK_CHECK(cond, msg)                      \
    do {                                           \
        if (!(cond)) {                             \
            ::rsfk::set_last_error(msg);           \
            (void)hipDeviceSynchronize();          \
            return 2;                              \
        }                                          \
    } while (0)

// ---------------------------------------------------------------------------
// Which item a workgroup takes when neighbouring items should meet in the same L2 cache.  The device has eight dies
// (XCDs), each with its own L2, and workgroup b of a launch runs on die b mod 8: with a grid that is a multiple of 8,
// workgroup b takes place (b mod 8) * (grid / 8) + b / 8, so that each die works through one contiguous eighth of the
// items in order.  (Places beyond the number of items are for the caller to skip.)
// ---------------------------------------------------------------------------
constexpr int kDies = 8;
__device__ __forceinline__ int die_local_place(int block, int grid) { return (block & (kDies - 1)) * (grid / kDies) + block / kDies; }
inline unsigned grid_for_dies(size_t n_blocks) { return (unsigned)((n_blocks + kDies - 1) / kDies * kDies); }

// ---------------------------------------------------------------------------
// counter-based random numbers.  A node of a tree is identified by a 64-bit key
// derived from the tree seed and the left/right path to the node, so a tree is
// a pure function of (points, MIN, MAX, MAX_DEPTH, seed) whatever the launch
// geometry.  (The reference seeds cuRAND from the thread index:
// src/kernels/build_tree_create_nodes.cu:64-68.)
// ---------------------------------------------------------------------------
__host__ __device__ inline uint64_t mix64(uint64_t z)
{
    z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ULL;
    z ^= z >> 27; z *= 0x94D049BB133111EBULL;
    z ^= z >> 31;
    return z;
}
__host__ __device__ inline uint64_t root_key(int seed)
{
    return mix64((uint64_t)(int64_t)seed ^ 0x5253464B524F4F54ULL);
}
__host__ __device__ inline uint64_t child_key(uint64_t key, int side)
{
    return mix64(key + 0x9E3779B97F4A7C15ULL * (uint64_t)(side + 1));
}
__host__ __device__ inline uint32_t draw_u32(uint64_t key, uint32_t i)
{
    return (uint32_t)(mix64(key ^ (0xD6E8FEB86659FD93ULL * (uint64_t)(i + 1))) >> 32);
}
// Two member ranks in [0,count); the second is redrawn while equal to the first
// (src/kernels/build_tree_create_nodes.cu:96-100), bounded so it always ends.
__host__ __device__ inline void pick_pair(uint64_t key, int count, int& r1, int& r2)
{
    uint32_t c = (uint32_t)count;
    uint32_t a = draw_u32(key, 0) % c;
    uint32_t b = draw_u32(key, 1) % c;
    if (count >= 2) {
        uint32_t i = 2;
        while (b == a && i < 66) { b = draw_u32(key, i) % c; ++i; }
        if (b == a) b = (a + 1) % c;
    }
    r1 = (int)a; r2 = (int)b;
}

// ---------------------------------------------------------------------------
// records
// ---------------------------------------------------------------------------
// A node of a tree under construction.  Its members are perm[buf][tree*N + start
// .. + count); the point pair that defines its hyperplane is drawn from the
// sub-range [dstart, dstart+dcount) (the larger side, after a min-size merge).
struct TreeNode {
    int tree;
    int start, count;
    int dstart, dcount;
    int depth;        // level of the node, root = 0
    int buf;          // which of the two permutation buffers holds the members
    int leaf;         // 1 = already decided to be a bucket
    int rec;          // where the node is written in the index of the tree (only when an index is recorded)
    int pad_;
    uint64_t key;
};

// Index of a tree for routing query points (recorded only on request).  Internal node with two children: a, b =
// the drawn pair of points, c0 / c1 = records of the left / right child.  Bucket: a = start of its segment of the
// tree's permutation, b = its size, c0 = c1 = -1.  A node with one child has no record (its child stands in its
// place).  Record 0 is the root.
struct TreeRec {
    int a, b, c0, c1;
};

// Buckets of at most this many points are handled by the small-bucket K-NN kernel; the
// tree builder keeps them apart from the larger ones.
constexpr int kBucketSplit = 64;

// A K-NN row is the register state of one wavefront: slot k in lane k % 64, register k / 64 (knn_list.hpp).  The
// kernels are compiled for 1, 2, 4, 8 and 16 registers per lane, so K may be at most 1024.  (The reference scans a row
// of any K from global memory: src/kernels/compute_knn_from_buckets.cu:1035-1099.)
constexpr int kMaxK = 1024;
inline int row_slots(int K) { return K <= 64 ? 1 : (K <= 128 ? 2 : (K <= 256 ? 4 : (K <= 512 ? 8 : 16))); }
// Rows of more than this many neighbours take the general kernels only: the specialised ones (reversed-graph join,
// merge kernels, pair matrix on the matrix cores) keep per-neighbour state of a row in 256 threads or in LDS.
constexpr int kMaxKJoin = 256;

// bit 31 of a permutation entry marks "right side" during a split; ids use the low 31 bits
constexpr int kIdMask = 0x7fffffff;

// Parameters of one tree-building batch (B trees built level-synchronously).
struct TreeParams {
    int N, D;
    int MIN, MAX, MAX_DEPTH;
    int small;        // nodes with at most this many points are finished by one workgroup
    int chunk;        // points per workgroup in the wide (global) passes
    float band;       // half-width of the undecided band of the bfloat16 side screen, relative to sum |n_d||x~_d|
};

}  // namespace rsfk
