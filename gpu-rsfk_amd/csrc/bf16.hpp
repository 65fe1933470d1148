// bfloat16 screening copy of the points.
//
// Row p of the copy holds the coordinates of point p rounded to bfloat16 (round to
// nearest even), padded with zeros to a multiple of 8 values so that rows and
// 16-byte pieces of rows are aligned; norms[p] = sum of the squares of the rounded
// coordinates.  The copy halves the bytes of every pass that only has to decide an
// inequality (side of a hyperplane, "is this candidate closer than the row
// maximum"): the kernels evaluate the inequality on the copy with a rigorous error
// bound and fall back to the fp32 row inside the band where the bound cannot
// decide, so results are those of the fp32 arithmetic.
#pragma once
#include "rsfk_common.hpp"

namespace rsfk {

// Row pitch in values: rows start on 64-byte boundaries so that a row touches the
// minimum number of memory sectors.  bf16_valid(D) <= bf16_pitch(D) is the length the
// kernels loop over (whole 16-byte pieces); values between D and the pitch are zero.
__host__ __device__ inline int bf16_pitch(int D) { return (D + 31) & ~31; }
__host__ __device__ inline int bf16_valid(int D) { return (D + 7) & ~7; }

struct Bf16Copy {
    uint16_t* rows = nullptr;     // N x bf16_pitch(D)
    float* norms = nullptr;       // N
};

size_t bf16_copy_bytes(int N, int D);
int bf16_copy_alloc(Bf16Copy* c, int N, int D);
void bf16_copy_free(Bf16Copy* c);
int bf16_copy_fill(const Bf16Copy& c, const float* points, int N, int D, hipStream_t stream);

}  // namespace rsfk
