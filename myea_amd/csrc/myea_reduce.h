// myea_reduce.h — launch helpers and the deterministic two-stage column reduction shared by the HBM-bound kernels.
#pragma once
#include <type_traits>

#include <hip/hip_runtime.h>
#include <stddef.h>

namespace myea {
namespace {

constexpr int kBlock = 256;

inline unsigned grid_for(size_t n, int per_block, unsigned cap = 65535u * 16u)
{
    size_t g = (n + per_block - 1) / per_block;
    if (g < 1) g = 1;
    if (g > cap) g = cap;
    return (unsigned)g;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// ---- two-stage column reductions -----------------------------------------------------------------
// Stage 1: grid (ceil(H/64), S); a workgroup is 64 columns x 4 row lanes and owns rows
// [y*chunk, (y+1)*chunk).  It writes NV partial sums per column to partial[(y*NV + v)*H + col].

// Per-lane accumulation is in fp64 (the kernels are HBM-bound, the adds are free): sums like
// E[x^2] - mean^2 lose most of their digits when |mean| >> sigma, and the fp32 result should then be the
// correctly rounded one rather than depend on the summation order.
// rows a lane keeps in flight at once: 4 unless the functor says otherwise (F::kUnroll)
template <class F, class = void> struct unroll_of { static constexpr int value = 4; };
template <class F> struct unroll_of<F, std::void_t<decltype(F::kUnroll)>> { static constexpr int value = F::kUnroll; };

template <int NV, typename F>
__global__ __launch_bounds__(kBlock) void column_partial_kernel(size_t rows, size_t H, size_t chunk, float *partial, F f)
{
    __shared__ double red[NV][4][64];
    const int c = threadIdx.x & 63, rl = threadIdx.x >> 6;
    const size_t col = (size_t)blockIdx.x * 64 + c;
    double acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.0;
    if (col < H) {
        const size_t r0 = (size_t)blockIdx.y * chunk, r1 = min(rows, r0 + chunk);
        // several rows' loads in flight per lane: a lane's rows are independent until the adds
#pragma unroll unroll_of<F>::value
        for (size_t r = r0 + rl; r < r1; r += 4) f(r, col, acc);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) red[v][rl][c] = acc[v];
    __syncthreads();
    if (rl == 0 && col < H) {
#pragma unroll
        for (int v = 0; v < NV; ++v)
            partial[((size_t)blockIdx.y * NV + v) * H + col] = (float)(red[v][0][c] + red[v][1][c] + red[v][2][c] + red[v][3][c]);
    }
}

inline void split_rows(size_t rows, size_t H, size_t &S, size_t &chunk)
{
    // aim at >= 1024 workgroups, at least 32 rows per chunk, at most 64 splits
    const size_t colblocks = (H + 63) / 64;
    S = (1024 + colblocks - 1) / colblocks;
    const size_t max_s = (rows + 31) / 32;
    if (S > max_s) S = max_s;
    if (S > 64) S = 64;
    if (S < 1) S = 1;
    chunk = (rows + S - 1) / S;
    S = (rows + chunk - 1) / chunk;
    if (S < 1) S = 1;
}

}  // namespace
}  // namespace myea
