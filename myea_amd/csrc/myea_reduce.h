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

// ---- column sums inside a workgroup of (row lane, column) lanes ---------------------------------
// For kernels in which a workgroup owns CW columns and all rows of a tensor: lane = CW * row lane + column, CW in {4, 16, 64},
// so a wavefront holds 64 / CW row lanes of every column.  What each lane summed over its rows becomes the column's sum in
// two stages.  Stage one runs in every wavefront and costs the LDS unit (which all wavefronts share) as little as possible:
// with CW < 16 the lanes of a 16-lane row that share a column add up by row rotations inside the vector unit and the row's
// first CW lanes write one partial each (four partials a wavefront); with CW == 16 the four 16-lane rows add up across the
// wavefront (one partial); with CW == 64 a lane's value is the partial.  Stage two runs in ONE wavefront per quantity: its
// lanes share out the column's partials, 64 / CW lanes a column, and add up inside their quad or 16-lane row.  Every sum is
// taken in a fixed order: the same bits in every run.
// the value of another lane of the 16-lane row, chosen by a data-parallel-primitive control word: a move inside the vector unit
template <int CTRL>
__device__ __forceinline__ double norm_dpp(double v)
{
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_mov_dpp(lo, CTRL, 0xf, 0xf, false);
    hi = __builtin_amdgcn_mov_dpp(hi, CTRL, 0xf, 0xf, false);
    return __hiloint2double(hi, lo);
}
// lane j of a 16-lane row takes the value of lane j - N (mod 16) of its row
template <int N> __device__ __forceinline__ double norm_row_rotate(double v) { return norm_dpp<0x120 + N>(v); }
// lane j takes the value of lane j ^ 1 resp. j ^ 2
__device__ __forceinline__ double norm_quad_xor1(double v) { return norm_dpp<0xB1>(v); }
__device__ __forceinline__ double norm_quad_xor2(double v) { return norm_dpp<0x4E>(v); }

template <int CW> constexpr int kNormPartials = CW < 16 ? 4 : 1;   // partials a wavefront leaves per column
template <int CW>
__device__ __forceinline__ double norm_fold_partial(double v)
{
    static_assert(CW == 1 || CW == 2 || CW == 4 || CW == 8 || CW == 16 || CW == 64, "columns per workgroup");
    if (CW <= 1) v += norm_row_rotate<1>(v);
    if (CW <= 2) v += norm_row_rotate<2>(v);
    if (CW <= 4) v += norm_row_rotate<4>(v);
    if (CW <= 8) v += norm_row_rotate<8>(v);
    if (CW == 16) { v += __shfl_xor(v, 16); v += __shfl_xor(v, 32); }
    return v;
}
// which lanes hold a partial, and where it goes among the workgroup's (wavefronts) * kNormPartials<CW>
template <int CW> __device__ __forceinline__ bool norm_partial_holder(int lane) { return CW < 16 ? (lane & 15) < CW : (CW == 16 ? lane < 16 : true); }
template <int CW> __device__ __forceinline__ int norm_partial_index(int wave, int lane) { return CW < 16 ? wave * 4 + (lane >> 4) : wave; }
// The finishing wavefront's lanes: lane -> the column it works for, and whether it is the one that keeps the column's total
template <int CW> __device__ __forceinline__ int norm_finish_column(int lane) { return CW >= 64 ? lane : lane / (64 / CW); }
template <int CW> __device__ __forceinline__ bool norm_finish_keeper(int lane) { return CW >= 64 ? true : lane % (64 / CW) == 0; }
// every lane of the finishing wavefront returns its column's total
template <int CW, int NP>
__device__ __forceinline__ double norm_sum_partials(const double (&p)[NP][CW], int lane)
{
    if (CW >= 64) {
        double v = 0.0;
#pragma unroll
        for (int w = 0; w < NP; ++w) v += p[w][lane % CW];
        return v;
    }
    constexpr int LPC = CW >= 64 ? 4 : 64 / CW;
    static_assert(CW >= 64 || LPC == 4 || LPC == 16, "a column's lanes are a quad or a 16-lane row");
    static_assert(CW >= 64 || NP % LPC == 0, "every lane of a column takes the same number of partials");
    const int column = lane / LPC, j = lane % LPC;
    double v = 0.0;
#pragma unroll
    for (int w = 0; w < NP / LPC; ++w) v += p[w * LPC + j][column % CW];
    v += norm_quad_xor1(v);
    v += norm_quad_xor2(v);
    if (LPC == 16) { v += norm_row_rotate<4>(v); v += norm_row_rotate<8>(v); }
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
