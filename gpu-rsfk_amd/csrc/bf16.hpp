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

//
// A copy can be centred: the rows then hold x - mu rounded (first to fp32, then to bfloat16) with mu the
// column means.  Distances do not change under a common shift, and the rounding errors -- proportional to the
// magnitude of what is rounded -- shrink with the norms, so distance screens pass fewer candidates on data that
// sits away from the origin.  fl(x - mu) adds a relative 2^-24 to the 2^-8 of the bfloat16 rounding; the bounds
// of the consumers carry one per cent of slack for such terms.  Only screens of distances may use a centred copy.
struct Bf16Copy {
    uint16_t* rows = nullptr;     // N x bf16_pitch(D)
    float* norms = nullptr;       // N
    float* mu = nullptr;          // D column means the rows were shifted by, or null
};

// 8-bit screening copy of the points, used by the side test of the tree build when the rows have a narrow
// range of values (half the bytes of the bfloat16 copy).
//
// Row p, q8_pitch(D) bytes on a 64-byte boundary: a 16-byte header (pad, lo, scale, e1 as four floats), then one
// byte per coordinate, q_d = round((x_d - lo) / scale) in 0..255 with lo = min_d x_d and scale = (max_d x_d - lo) / 255,
// zeros up to the end of the row.  e1 bounds what the quantisation can do to a dot product per unit of the
// 1-norm of the other vector: for any n, |n.x - (lo sum_d n_d + scale sum_d n_d q_d)| <= e1 ||n||_1, including
// the fp32 evaluation of either side with at most D/8-term chains (see k_to_q8).  mean_rho (host, after
// q8_copy_fill has completed) compares e1 with the corresponding quantity of the bfloat16 copy,
// 2^-8 mean_d |x_d|, averaged over the rows: the 8-bit copy pays off while it is below about 6.
__host__ __device__ inline int q8_pitch(int D) { return (16 + D + 63) & ~63; }
__host__ __device__ inline int q8_padded(int D) { return (D + 15) & ~15; }      // coordinates in whole 16-byte pieces

struct Q8Copy {
    uint8_t* rows = nullptr;      // N x q8_pitch(D)
    float* rho_sum = nullptr;     // device scalar: sum over the rows of e1 / (2^-8 mean |x_d|)
};

int q8_copy_alloc(Q8Copy* c, int N, int D);
void q8_copy_free(Q8Copy* c);
int q8_copy_fill(const Q8Copy& c, const float* points, int N, int D, hipStream_t stream);
int q8_copy_mean_rho(const Q8Copy& c, int N, float* mean_rho, hipStream_t stream);     // synchronises the stream

size_t bf16_copy_bytes(int N, int D);
int bf16_copy_alloc(Bf16Copy* c, int N, int D, bool centred = false);
void bf16_copy_free(Bf16Copy* c);
int bf16_copy_fill(const Bf16Copy& c, const float* points, int N, int D, hipStream_t stream);

}  // namespace rsfk
