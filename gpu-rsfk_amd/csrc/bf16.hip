#include "bf16.hpp"
#include "wave64.hpp"
#include <algorithm>

namespace rsfk {

namespace {

// one wavefront per row: convert, pad, and sum the squares of the rounded values
__global__ __launch_bounds__(256) void k_to_bf16(const float* __restrict__ points, uint16_t* __restrict__ out,
                                                 float* __restrict__ norms, const float* __restrict__ mu, int N, int D,
                                                 int Db)
{
    const int lane = threadIdx.x & 63;
    const int wave_global = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int n_waves = (gridDim.x * blockDim.x) >> 6;
    for (int r = wave_global; r < N; r += n_waves) {
        const float* src = points + (size_t)r * (size_t)D;
        uint16_t* dst = out + (size_t)r * (size_t)Db;
        float q = 0.0f;
        for (int d = lane; d < Db; d += 64) {
            uint32_t u = d < D ? __float_as_uint(mu ? src[d] - mu[d] : src[d]) : 0u;
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

// column sums: a workgroup adds up its share of the rows, 256 columns at a time, and adds the result to sum[]
__global__ __launch_bounds__(256) void k_col_sum(const float* __restrict__ points, int N, int D, float* __restrict__ sum)
{
    const int rows_per = (N + gridDim.x - 1) / gridDim.x;
    const int r0 = blockIdx.x * rows_per, r1 = min(N, r0 + rows_per);
    for (int d = threadIdx.x; d < D; d += 256) {
        float acc = 0.0f;
        for (int r = r0; r < r1; ++r) acc += points[(size_t)r * (size_t)D + d];
        atomicAdd(&sum[d], acc);
    }
}

// The same for D <= 128: the workgroup reads m = 256 / D whole rows per step (thread t: row t / D of the step, column
// t % D, so its column never changes), eight steps in flight; the threads of a column are added up in LDS.
__global__ __launch_bounds__(256) void k_col_sum_narrow(const float* __restrict__ points, int N, int D, float* __restrict__ sum)
{
    __shared__ float part[256];
    const int m = 256 / D;
    const int rows_per = (N + gridDim.x - 1) / gridDim.x;
    const int r0 = blockIdx.x * rows_per, r1 = min(N, r0 + rows_per);
    const int sub = threadIdx.x / D, col = threadIdx.x - sub * D;
    float acc = 0.0f;
    if (sub < m) {
        const float* src = points + col;
        int r = r0 + sub;
        for (; r + 7 * m < r1; r += 8 * m) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(r + u * m) * (size_t)D];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; r < r1; r += m) acc += src[(size_t)r * (size_t)D];
    }
    part[threadIdx.x] = acc;
    __syncthreads();
    if ((int)threadIdx.x < D) {
        float t = 0.0f;
        for (int u = 0; u < m; ++u) t += part[u * D + threadIdx.x];
        atomicAdd(&sum[threadIdx.x], t);
    }
}

// sums -> means; a mean that is not finite is replaced by 0 (any shift is a valid one)
__global__ void k_col_mean(float* __restrict__ mu, int D, float inv_n)
{
    const int d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d < D) {
        const float m = mu[d] * inv_n;
        mu[d] = fabsf(m) <= 3.0e38f ? m : 0.0f;
    }
}

// one wavefront per row of the 8-bit copy
__global__ __launch_bounds__(256) void k_to_q8(const float* __restrict__ points, uint8_t* __restrict__ out,
                                               float* __restrict__ rho_sum, int N, int D, int pitch, float c_d)
{
    const int lane = threadIdx.x & 63;
    const int wave_global = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int n_waves = (gridDim.x * blockDim.x) >> 6;
    float rho_acc = 0.0f;
    for (int r = wave_global; r < N; r += n_waves) {
        const float* src = points + (size_t)r * (size_t)D;
        uint8_t* dst = out + (size_t)r * (size_t)pitch;
        float lo = INFINITY, hi = -INFINITY, sabs = 0.0f;
        bool bad = false;
        for (int d = lane; d < D; d += 64) {
            const float x = src[d];
            bad |= !(fabsf(x) <= 3.0e38f);                 // NaN or infinite
            lo = fminf(lo, x);
            hi = fmaxf(hi, x);
            sabs += fabsf(x);
        }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            lo = fminf(lo, __shfl_xor(lo, o, 64));
            hi = fmaxf(hi, __shfl_xor(hi, o, 64));
            sabs += __shfl_xor(sabs, o, 64);
        }
        bad = __ballot(bad) != 0;
        const float range = hi - lo;
        const float scale = range * (1.0f / 255.0f);
        const float inv = range > 0.0f ? 255.0f / range : 0.0f;
        float err = 0.0f;
        // four coordinates per lane and step: one 4-byte store instead of four 1-byte stores
        for (int d0 = 4 * lane; d0 < pitch - 16; d0 += 256) {
            uint32_t packed = 0u;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int d = d0 + k;
                if (d < D) {
                    const float x = src[d];
                    float t = __builtin_rintf((x - lo) * inv);
                    t = fminf(fmaxf(t, 0.0f), 255.0f);
                    packed |= (uint32_t)t << (8 * k);
                    err = fmaxf(err, fabsf(x - __builtin_fmaf(scale, t, lo)));
                }
            }
            *reinterpret_cast<uint32_t*>(dst + 16 + d0) = packed;
        }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) err = fmaxf(err, __shfl_xor(err, o, 64));
        // err was measured against fl(lo + scale q); the screen evaluates lo sum n + scale sum n q in fp32 and is
        // compared with an fp32 evaluation of n.x: all of that stays below c_d (|lo| + 255 scale) per unit of ||n||_1
        const float mag = fabsf(lo) + 255.0f * scale;
        float e1 = 1.01f * err + c_d * mag + 1e-37f;
        if (bad || !(range <= 3.0e38f)) e1 = __builtin_nanf("");      // the screen never decides for such a row
        if (lane == 0) {
            float* head = reinterpret_cast<float*>(dst);
            head[0] = 0.0f;
            head[1] = lo;
            head[2] = scale;
            head[3] = e1;
            const float bf = sabs / (float)D * (1.0f / 256.0f);
            rho_acc += (e1 == e1 && bf > 0.0f) ? fminf(e1 / bf, 1000.0f) : 1000.0f;
        }
    }
    // one atomic per workgroup (they all hit the same address)
    __shared__ float part[4];
    if (lane == 0) part[threadIdx.x >> 6] = rho_acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        const float t = part[0] + part[1] + part[2] + part[3];
        if (t != 0.0f) atomicAdd(rho_sum, t);
    }
}

// The same copy for rows whose 4-byte words of the 8-bit row (pitch - 16 bytes, the padding included) fit LPR lanes
// with at most PPL words each: LPR lanes per row (64 / LPR rows per wavefront), the coordinates are read once, as
// 16-byte pieces, and stay in registers between the pass that finds the range and the pass that rounds.  Produces the
// bytes and headers of k_to_q8 (minimum, maximum and rounding do not depend on the order; the sum of the absolute
// values, which only feeds the average that chooses between the screens, is added up in another order).
// Needs D % 4 == 0 and 16-byte aligned points.
template <int LPR, int PPL>
__global__ __launch_bounds__(256) void k_to_q8_regs(const float* __restrict__ points, uint8_t* __restrict__ out,
                                                    float* __restrict__ rho_sum, int N, int D, int pitch, float c_d)
{
    constexpr int kRowsPerWave = 64 / LPR;
    const int lane = threadIdx.x & 63, sub = lane / LPR, l = lane - sub * LPR;
    const int wave_global = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int n_waves = (gridDim.x * blockDim.x) >> 6;
    const int words = (pitch - 16) >> 2, pieces = D >> 2;
    float rho_acc = 0.0f;
    for (int rb = wave_global * kRowsPerWave; rb < N; rb += n_waves * kRowsPerWave) {
        const int r = rb + sub;
        const bool row_ok = r < N;
        const float* src = points + (size_t)(row_ok ? r : 0) * (size_t)D;
        float4 x[PPL];
        float lo = INFINITY, hi = -INFINITY, sabs = 0.0f;
        bool bad = false;
#pragma unroll
        for (int k = 0; k < PPL; ++k) {
            const int pc = l + k * LPR;
            x[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (row_ok && pc < pieces) {
                x[k] = *reinterpret_cast<const float4*>(src + 4 * pc);
                const float v[4] = {x[k].x, x[k].y, x[k].z, x[k].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    bad |= !(fabsf(v[c]) <= 3.0e38f);              // NaN or infinite
                    lo = fminf(lo, v[c]);
                    hi = fmaxf(hi, v[c]);
                    sabs += fabsf(v[c]);
                }
            }
        }
        int badi = bad ? 1 : 0;
#pragma unroll
        for (int o = 1; o < LPR; o <<= 1) {
            lo = fminf(lo, __shfl_xor(lo, o, 64));
            hi = fmaxf(hi, __shfl_xor(hi, o, 64));
            sabs += __shfl_xor(sabs, o, 64);
            badi |= __shfl_xor(badi, o, 64);
        }
        const float range = hi - lo;
        const float scale = range * (1.0f / 255.0f);
        const float inv = range > 0.0f ? 255.0f / range : 0.0f;
        float err = 0.0f;
        uint8_t* dst = out + (size_t)(row_ok ? r : 0) * (size_t)pitch;
#pragma unroll
        for (int k = 0; k < PPL; ++k) {
            const int pc = l + k * LPR;
            if (row_ok && pc < words) {
                uint32_t packed = 0u;
                if (pc < pieces) {
                    const float v[4] = {x[k].x, x[k].y, x[k].z, x[k].w};
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float t = __builtin_rintf((v[c] - lo) * inv);
                        t = fminf(fmaxf(t, 0.0f), 255.0f);
                        packed |= (uint32_t)t << (8 * c);
                        err = fmaxf(err, fabsf(v[c] - __builtin_fmaf(scale, t, lo)));
                    }
                }
                *reinterpret_cast<uint32_t*>(dst + 16 + 4 * pc) = packed;
            }
        }
#pragma unroll
        for (int o = 1; o < LPR; o <<= 1) err = fmaxf(err, __shfl_xor(err, o, 64));
        const float mag = fabsf(lo) + 255.0f * scale;
        float e1 = 1.01f * err + c_d * mag + 1e-37f;
        if (badi || !(range <= 3.0e38f)) e1 = __builtin_nanf("");      // the screen never decides for such a row
        if (row_ok && l == 0) {
            *reinterpret_cast<float4*>(dst) = make_float4(0.0f, lo, scale, e1);
            const float bf = sabs / (float)D * (1.0f / 256.0f);
            rho_acc += (e1 == e1 && bf > 0.0f) ? fminf(e1 / bf, 1000.0f) : 1000.0f;
        }
    }
    // one atomic per workgroup (they all hit the same address)
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) rho_acc += __shfl_xor(rho_acc, o, 64);
    __shared__ float part[4];
    if (lane == 0) part[threadIdx.x >> 6] = rho_acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        const float t = part[0] + part[1] + part[2] + part[3];
        if (t != 0.0f) atomicAdd(rho_sum, t);
    }
}

}  // namespace

int q8_copy_alloc(Q8Copy* c, int N, int D)
{
    if (ws_alloc(reinterpret_cast<void**>(&c->rows), std::max<size_t>((size_t)N * q8_pitch(D), 64))) return 1;
    if (ws_alloc(reinterpret_cast<void**>(&c->rho_sum), 16)) return 1;
    return 0;
}

void q8_copy_free(Q8Copy* c)
{
    ws_free(c->rows);
    ws_free(c->rho_sum);
    c->rows = nullptr;
    c->rho_sum = nullptr;
}

int q8_copy_fill(const Q8Copy& c, const float* points, int N, int D, hipStream_t stream)
{
    RSFK_HIP(hipMemsetAsync(c.rho_sum, 0, sizeof(float), stream));
    const int grid = std::min((N + 3) / 4, 4096);
    // (D/8 + D/32 + D + 32) 2^-24: chains of the screen and of the exact test, sum of the normal, rounding of lo + scale q
    const float c_d = (float)(D / 8 + D / 32 + D + 32) / 16777216.0f;
    const int pitch = q8_pitch(D), words = (pitch - 16) >> 2;
    const bool vec_ok = (D & 3) == 0 && (reinterpret_cast<uintptr_t>(points) & 15) == 0;
#define RSFK_Q8_REGS(L, P)                                                                                                 \
    hipLaunchKernelGGL((k_to_q8_regs<L, P>), dim3(std::min((N + 4 * (64 / L) - 1) / (4 * (64 / L)), 8192)), dim3(256), 0,   \
                       stream, points, c.rows, c.rho_sum, N, D, pitch, c_d)
    if (vec_ok && words <= 16) RSFK_Q8_REGS(16, 1);
    else if (vec_ok && words <= 32) RSFK_Q8_REGS(32, 1);
    else if (vec_ok && words <= 64) RSFK_Q8_REGS(64, 1);
    else if (vec_ok && words <= 128) RSFK_Q8_REGS(64, 2);
    else if (vec_ok && words <= 256) RSFK_Q8_REGS(64, 4);
    else hipLaunchKernelGGL(k_to_q8, dim3(grid), dim3(256), 0, stream, points, c.rows, c.rho_sum, N, D, pitch, c_d);
#undef RSFK_Q8_REGS
    RSFK_HIP(hipGetLastError());
    return 0;
}

int q8_copy_mean_rho(const Q8Copy& c, int N, float* mean_rho, hipStream_t stream)
{
    float sum = 0.0f;
    RSFK_HIP(hipMemcpyAsync(&sum, c.rho_sum, sizeof(float), hipMemcpyDeviceToHost, stream));
    RSFK_HIP(hipStreamSynchronize(stream));
    *mean_rho = N > 0 ? sum / (float)N : 0.0f;
    return 0;
}

size_t bf16_copy_bytes(int N, int D) { return (size_t)N * ((size_t)bf16_pitch(D) * 2 + 4); }

int bf16_copy_alloc(Bf16Copy* c, int N, int D, bool centred)
{
    if (centred && ws_alloc(reinterpret_cast<void**>(&c->mu), std::max<size_t>((size_t)D * 4, 16))) return 1;
    if (ws_alloc(reinterpret_cast<void**>(&c->rows), std::max<size_t>((size_t)N * bf16_pitch(D) * 2, 16))) return 1;
    if (ws_alloc(reinterpret_cast<void**>(&c->norms), std::max<size_t>((size_t)N * 4, 16))) return 1;
    return 0;
}

void bf16_copy_free(Bf16Copy* c)
{
    ws_free(c->rows);
    ws_free(c->norms);
    ws_free(c->mu);
    c->mu = nullptr;
    c->rows = nullptr;
    c->norms = nullptr;
}

int bf16_copy_fill(const Bf16Copy& c, const float* points, int N, int D, hipStream_t stream)
{
    if (c.mu) {
        RSFK_HIP(hipMemsetAsync(c.mu, 0, sizeof(float) * (size_t)D, stream));
        const int g = std::max(1, std::min(N / 64, 2048));
        if (D <= 128) hipLaunchKernelGGL(k_col_sum_narrow, dim3(g), dim3(256), 0, stream, points, N, D, c.mu);
        else hipLaunchKernelGGL(k_col_sum, dim3(g), dim3(256), 0, stream, points, N, D, c.mu);
        hipLaunchKernelGGL(k_col_mean, dim3((D + 255) / 256), dim3(256), 0, stream, c.mu, D, 1.0f / (float)N);
    }
    const int grid = std::min((N + 3) / 4, 65536);
    hipLaunchKernelGGL(k_to_bf16, dim3(grid), dim3(256), 0, stream, points, c.rows, c.norms, c.mu, N, D, bf16_pitch(D));
    RSFK_HIP(hipGetLastError());
    return 0;
}

}  // namespace rsfk
