// fp32 values as matrix-core operands: every value is split into two bfloat16 numbers,
// x = hi + lo + r with |r| <= 2^-16 |x| (round to nearest twice), so that three
// v_mfma_f32_32x32x16_bf16 (hi hi' + hi lo' + lo hi') give an inner product of fp32
// rows to within a bound that follows from the norms alone (stated where it is used).
#pragma once
#include "rsfk_common.hpp"

namespace rsfk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// Two fp32 values -> their bfloat16 heads (packed) and the bfloat16 heads of what the first rounding left over.
__device__ __forceinline__ void split2(float a, float b, uint32_t& hi, uint32_t& lo)
{
    const f32x2 v = {a, b};
    hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    const f32x2 r = {a - __uint_as_float(hi << 16), b - __uint_as_float(hi & 0xffff0000u)};
    lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(r, bf16x2));
}

// Eight consecutive values of a row in LDS -> matrix-core operands (heads and remainders); adds their squares to nrm.
__device__ __forceinline__ void load_split(const float* __restrict__ p, bf16x8& hi, bf16x8& lo, float& nrm)
{
    const float4 u = *reinterpret_cast<const float4*>(p);
    const float4 v = *reinterpret_cast<const float4*>(p + 4);
    uint4 h, l;
    split2(u.x, u.y, h.x, l.x);
    split2(u.z, u.w, h.y, l.y);
    split2(v.x, v.y, h.z, l.z);
    split2(v.z, v.w, h.w, l.w);
    hi = __builtin_bit_cast(bf16x8, h);
    lo = __builtin_bit_cast(bf16x8, l);
    nrm = __builtin_fmaf(u.x, u.x, nrm); nrm = __builtin_fmaf(u.y, u.y, nrm);
    nrm = __builtin_fmaf(u.z, u.z, nrm); nrm = __builtin_fmaf(u.w, u.w, nrm);
    nrm = __builtin_fmaf(v.x, v.x, nrm); nrm = __builtin_fmaf(v.y, v.y, nrm);
    nrm = __builtin_fmaf(v.z, v.z, nrm); nrm = __builtin_fmaf(v.w, v.w, nrm);
}

// Coefficient c of the bound |d~ - d| <= c S, S = |a|^2 + |b|^2, d~ = |a|^2 + |b|^2 - 2 G with G from the three
// products above over D16 (= D rounded up to 16) dimensions: dropped products <= 3 * 2^-16 |x||y| <= 1.5 * 2^-16 S;
// 3 D16 exact products per entry accumulated in fp32, every addition within 2^-23 of the sum of absolute values
// whatever the order or rounding mode; the norms; the two roundings of the final expression.
inline float split_gram_error_coefficient(int D16)
{
    const float dp = (float)D16;
    return 3.1f / 65536.0f + (3.1f * dp + 8.0f) / 8388608.0f + (dp + 2.0f) / 16777216.0f;
}

}  // namespace rsfk
