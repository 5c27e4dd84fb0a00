// myea_elementwise.hip — HBM-bound kernels of the training step for gfx950: activations and their
// derivatives, softmax, dropout column scaling, batch-(re)normalisation forward/backward, bias-gradient
// column sums, output-layer delta with loss/accuracy accumulation, global-norm clipping and the fused
// optimizer update.  All of them are coalesced along the unit (fastest) dimension; reductions over the
// batch are two-stage and deterministic (per-chunk partial sums in a fixed order, no float atomics).
//
// NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/.
#include <initializer_list>

#include "myea_device_af.h"
#include "myea_kernels.h"
#include "myea_reduce.h"

namespace myea {

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

// ---- plain elementwise -------------------------------------------------------------------------

__global__ __launch_bounds__(kBlock) void fill_kernel(float *p, size_t n, float v)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) p[i] = v;
}

// Forward_Pass__FC_AF (NN/Neural_Network__Forward_Pass__OpenMP.cpp:4839-4868) fused with the Bernoulli
// appliers (:4907-4990) through a per-column multiplier.
__global__ __launch_bounds__(kBlock) void activation_kernel(int act, const int *unit_act, size_t n, size_t H, const float *x, float *y, const float *colscale)
{
    auto all = [&](auto activation) {
        const int shared = activation;
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
            float v = af_fire(unit_act ? unit_act[i % H] : shared, x[i]);
            if (colscale) v *= colscale[i % H];
            y[i] = v;
        }
    };
    if (unit_act) all(act); else af_with(act, all);
}

__global__ __launch_bounds__(kBlock) void colscale_kernel(size_t n, size_t H, float *y, const float *colscale)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) y[i] *= colscale[i % H];
}

__global__ __launch_bounds__(kBlock) void mask_to_scale_kernel(size_t n, const uint8_t *mask, float on, float *colscale)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) colscale[i] = mask[i] ? on : 0.f;
}

// Backward_Pass__FC__DF (NN/Neural_Network__Backward_Pass__OpenMP.cpp:1225-1263)
__global__ __launch_bounds__(kBlock) void activation_derive_kernel(int act, float steep, const int *unit_act, const float *unit_steep, size_t H, size_t n,
                                                                   const float *pre, const float *val, const float *dy, float *dx)
{
    auto all = [&](auto activation) {
        const int shared = activation;
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
            dx[i] = dy[i] * af_derive(unit_act ? unit_act[i % H] : shared, pre[i], unit_steep ? unit_steep[i % H] : steep, val[i]);
    };
    if (unit_act) all(act); else af_with(act, all);
}

// Independently recurrent layer, the whole sequence in one launch: a thread owns one (example, unit) pair and walks the
// time steps with the previous activation in a register, so the T dependent steps cost one pass over the tensors.
// Forward_Pass__FC_Ind_RNN (NN/Neural_Network__Recurrent_Forward_Pass__Loop.cpp:813-866): pre_AF[t] = input[t] + u * AF[t-1]
// (a copy at t = 0), then Forward_Pass__FC_AF and, for an un-normalised layer, the Bernoulli applier in place on AF - the
// value the next time step reads.
// Two things bound such a launch: trips to memory inside the chain of dependent steps, and the code of the chain itself - a
// loop unrolled over the time steps is kilobytes of instructions that every wavefront fetches once and runs once, and that
// fetch was measured to cost more than the arithmetic.  So the operands of kIndRnnChunk time steps are requested together,
// ahead of the chain, straight into LDS (a lane's words of LDS are its own: no barrier), and the chain is a loop of a few dozen
// instructions that reads them from there, with the layer's activation as a compile-time constant where af_with knows it.
constexpr int kIndRnnChunk = 32;
constexpr int kIndRnnLanes = 128;
// operand number `which` of the lane's time step `s` of the chunk: [which][s][lane]
template <int N>
struct IndRnnStage {
    float w[N][kIndRnnChunk][kIndRnnLanes];
    // the load of every lane of the wavefront: global address of the lane's own element, LDS slot of the lane
    __device__ __forceinline__ void request(int which, int s, const float *from)
    {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)from,
                                         (__attribute__((address_space(3))) void *)&w[which][s][threadIdx.x & ~63u], 4, 0, 0);
    }
    __device__ __forceinline__ float at(int which, int s) const { return w[which][s][threadIdx.x]; }
};
// every request of this wavefront has written its LDS words: vmcnt(0), and nothing that reads them moves above the wait
__device__ __forceinline__ void ind_rnn_requests_landed()
{
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
}

__global__ __launch_bounds__(kIndRnnLanes) void ind_rnn_forward_kernel(IndRnnParams p)
{
    __shared__ IndRnnStage<1> stage;
    const size_t n = p.B * p.H, step = p.Bmax * p.H;
    for (size_t i0 = (size_t)blockIdx.x * kIndRnnLanes; i0 < n; i0 += (size_t)gridDim.x * kIndRnnLanes) {
        const size_t i = i0 + threadIdx.x;
        if (i >= n) continue;
        const size_t j = i % p.H;
        const float u = p.u[j];
        auto walk = [&](auto activation) {
            const int act = activation;
            float h = 0.f;
            for (size_t t0 = 0; t0 < p.T; t0 += kIndRnnChunk) {
                const size_t k0 = i + t0 * step;
                const int m = (int)(p.T - t0 < (size_t)kIndRnnChunk ? p.T - t0 : (size_t)kIndRnnChunk);
                for (int s = 0; s < m; ++s) stage.request(0, s, p.in + k0 + s * step);
                ind_rnn_requests_landed();
                float x = stage.at(0, 0), cs = p.colscale ? p.colscale[t0 * p.H + j] : 1.f;
                for (int s = 0; s < m; ++s) {
                    const float x_next = s + 1 < m ? stage.at(0, s + 1) : 0.f;
                    const float cs_next = (p.colscale && s + 1 < m) ? p.colscale[(t0 + s + 1) * p.H + j] : 1.f;
                    float pre = x;
                    if (t0 + s) pre = __fadd_rn(pre, __fmul_rn(u, h));
                    p.pre_afs[k0 + s * step] = pre;
                    h = af_fire(act, pre);
                    if (p.colscale) h *= cs;
                    p.afs[k0 + s * step] = h;
                    x = x_next; cs = cs_next;
                }
            }
        };
        if (p.unit_act) walk(p.unit_act[j]); else af_with(p.act, walk);
    }
}

// Backward_Pass__FC__DF_Ind_RNN (NN/Neural_Network__Backward_Pass__Loop.cpp:1296-1390), time steps from the last to the
// first: errors = dY AF'(t); dAF(t) = errors + u AF'(t) dAF(t+1), without the second term at the last step.
__global__ __launch_bounds__(kIndRnnLanes) void ind_rnn_backward_kernel(IndRnnParams p)
{
    __shared__ IndRnnStage<3> stage;   // pre-activations, activations, the deltas from above
    const size_t n = p.B * p.H, step = p.Bmax * p.H;
    for (size_t i0 = (size_t)blockIdx.x * kIndRnnLanes; i0 < n; i0 += (size_t)gridDim.x * kIndRnnLanes) {
        const size_t i = i0 + threadIdx.x;
        if (i >= n) continue;
        const size_t j = i % p.H;
        const float u = p.u[j], steep = p.unit_steep ? p.unit_steep[j] : p.steep;
        auto walk = [&](auto activation) {
            const int act = activation;
            float next = 0.f;
            double du = 0.0;   // this (example, unit)'s share of the self weight's gradient: the sum over t >= 1 of AF[t-1] dAF[t]
            for (size_t done = 0; done < p.T; done += kIndRnnChunk) {   // time steps T-1-done, T-2-done, ...
                const int m = (int)(p.T - done < (size_t)kIndRnnChunk ? p.T - done : (size_t)kIndRnnChunk);
                const size_t top = p.T - 1 - done;
                for (int s = 0; s < m; ++s) {
                    const size_t k = i + (top - s) * step;
                    stage.request(0, s, p.pre_afs + k); stage.request(1, s, p.afs + k); stage.request(2, s, p.dy + k);
                }
                ind_rnn_requests_landed();
                float pre = stage.at(0, 0), val = stage.at(1, 0), dy = stage.at(2, 0);
                for (int s = 0; s < m; ++s) {
                    const int sn = s + 1 < m ? s + 1 : s;
                    const float pre_next = stage.at(0, sn), val_next = stage.at(1, sn), dy_next = stage.at(2, sn);
                    const size_t t = top - s;
                    if (t + 1 != p.T) du += (double)val * (double)next;   // next: dAF[t+1]
                    const float daf = af_derive(act, pre, steep, val);
                    const float e = __fmul_rn(dy, daf);
                    const float r = (t + 1 == p.T) ? e : __fadd_rn(e, __fmul_rn(__fmul_rn(u, daf), next));
                    p.dafs[i + t * step] = r;
                    next = r;
                    pre = pre_next; val = val_next; dy = dy_next;
                }
            }
            if (p.du_rows) p.du_rows[i] = (float)du;
        };
        if (p.unit_act) walk(p.unit_act[j]); else af_with(p.act, walk);
    }
}

// Update_Derivative_Weight__FC_Ind_RNN (NN/Neural_Network__Recurrent_Update_Derivative_Weight__Loop.cpp:461-483) summed over
// the time steps 1 .. T-1: du[j] += sum_{t, b} AF[t-1][b][j] dAF[t][b][j].  Row r of the reduction is (t = r / B, b = r % B).
struct IndRnnDotF {
    const float *afs, *dafs; size_t H, B, Bmax;
    __device__ void operator()(size_t r, size_t col, double *acc) const
    {
        const size_t t = r / B, b = r % B;
        acc[0] += (double)afs[(t * Bmax + b) * H + col] * (double)dafs[((t + 1) * Bmax + b) * H + col];
    }
};

// Update_Weight_Regularization__Constraint_Recurrent_Weight__FC_Ind_RNN
// (NN/Neural_Network__Regularization__Constraint_Recurrent_Weight.cpp:317-333)
__global__ __launch_bounds__(kBlock) void clip_range_kernel(size_t n, float *w, float lo, float hi)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const float v = w[i];
        w[i] = v < lo ? lo : (v > hi ? hi : v);
    }
}

// Gaussian / Uout dropout (Forward_Pass__Dropout__Gaussian / __Uout, NN/Neural_Network__Forward_Pass__Loop.cpp:4993-5014,
// 5047-5068).  The draws come from a tensor: either the caller's own or the output of the counter-based generator below.
// Philox 4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11): counter = (element index / 4 lo, hi,
// stream lo, stream hi), key = the seed's two halves; four 32-bit outputs per counter value.
__device__ __forceinline__ void philox4x32_10(unsigned c0, unsigned c1, unsigned c2, unsigned c3, unsigned k0, unsigned k1, unsigned out[4])
{
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const unsigned long long p0 = 0xD2511F53ull * c0, p1 = 0xCD9E8D57ull * c2;
        const unsigned n0 = (unsigned)(p1 >> 32) ^ c1 ^ k0, n1 = (unsigned)p1, n2 = (unsigned)(p0 >> 32) ^ c3 ^ k1, n3 = (unsigned)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// normal: mean + sd * N(0,1) by Box-Muller on two uniforms in (0, 1]; uniform: lo + (hi - lo) * U[0, 1)
__global__ __launch_bounds__(kBlock) void dropout_noise_kernel(size_t n, float *noise, int normal, float a, float b, unsigned long long seed, unsigned long long stream)
{
    const size_t quads = (n + 3) / 4;
    for (size_t q = (size_t)blockIdx.x * kBlock + threadIdx.x; q < quads; q += (size_t)gridDim.x * kBlock) {
        unsigned r[4];
        philox4x32_10((unsigned)q, (unsigned)(q >> 32), (unsigned)stream, (unsigned)(stream >> 32), (unsigned)seed, (unsigned)(seed >> 32), r);
        float v[4];
        if (normal) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float u1 = ((float)(r[2 * h] >> 8) + 1.f) * (1.f / 16777216.f);   // (0, 1]
                const float u2 = (float)(r[2 * h + 1] >> 8) * (1.f / 16777216.f);       // [0, 1)
                const float rad = sqrtf(-2.f * logf(u1));
                float sn, cs;
                sincosf(6.283185307179586f * u2, &sn, &cs);
                v[2 * h] = a + b * rad * cs;
                v[2 * h + 1] = a + b * rad * sn;
            }
        } else {
#pragma unroll
            for (int h = 0; h < 4; ++h) v[h] = a + (b - a) * ((float)(r[h] >> 8) * (1.f / 16777216.f));
        }
#pragma unroll
        for (int h = 0; h < 4; ++h)
            if (q * 4 + h < n) noise[q * 4 + h] = v[h];
    }
}

// gaussian: y *= noise; uout: y += y * noise
__global__ __launch_bounds__(kBlock) void dropout_noise_apply_kernel(size_t n, float *y, const float *noise, int uout)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const float v = y[i], g = noise[i];
        y[i] = uout ? __fadd_rn(v, __fmul_rn(v, g)) : v * g;
    }
}

// ShakeDrop (Forward_Pass__Dropout__ShakeDrop NN/Neural_Network__Forward_Pass__Loop.cpp:5016-5045, Backward_Pass__Dropout__ShakeDrop
// NN/Neural_Network__Backward_Pass__Loop.cpp:1050-1078): rows whose mask is set are multiplied value by value by their draws;
// without a mask every value is multiplied by `constant` (the inference scaling).
__global__ __launch_bounds__(kBlock) void shakedrop_apply_kernel(size_t rows, size_t W, float *x, const float *mask, const float *draws, float constant)
{
    const size_t n = rows * W;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        if (!mask) x[i] *= constant;
        else if (mask[i / W] != 0.f) x[i] *= draws[i];
    }
}

// uniform draws in [0, 1) to a Bernoulli(p) mask held as 0 / 1
__global__ __launch_bounds__(kBlock) void threshold_kernel(size_t n, float *x, float p)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) x[i] = x[i] < p ? 1.f : 0.f;
}

// Sparse_K_Filter (NN/Neural_Network__K_Sparse.cpp:268-339): per row the k largest values stay, the others become 0; among
// equal values at the cut the lower indices stay.  One workgroup per row: a 4-pass radix select over order-preserving keys
// finds the k-th largest key and how many entries equal to it stay, then one ordered pass writes the zeros.
__device__ __forceinline__ unsigned k_sparse_key(float f)
{
    const unsigned u = __float_as_uint(f + 0.f);   // -0 and +0 are one value
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(kBlock) void k_sparse_kernel(size_t rows, size_t H, unsigned k, float *x)
{
    __shared__ unsigned hist[256];
    __shared__ unsigned s_bin, s_need, wave_cnt[kBlock / 64];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    for (size_t row = blockIdx.x; row < rows; row += gridDim.x) {
        float *r = x + row * H;
        unsigned prefix = 0, mask = 0, need = k;
        for (int shift = 24; shift >= 0; shift -= 8) {
            hist[tid] = 0;
            __syncthreads();
            for (size_t j = tid; j < H; j += kBlock) {
                const unsigned key = k_sparse_key(r[j]);
                if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (tid == 0) {
                unsigned acc = 0;
                int b = 255;
                for (; b > 0; --b) {
                    if (acc + hist[b] >= need) break;
                    acc += hist[b];
                }
                s_bin = (unsigned)b; s_need = need - acc;
            }
            __syncthreads();
            prefix |= s_bin << shift; mask |= 255u << shift; need = s_need;
            __syncthreads();
        }
        // prefix is the k-th largest key; `need` entries equal to it stay, in index order
        unsigned base = 0;
        for (size_t j0 = 0; j0 < H; j0 += kBlock) {
            const size_t j = j0 + tid;
            const bool valid = j < H;
            const unsigned key = valid ? k_sparse_key(r[j]) : 0u;
            const bool eq = valid && key == prefix;
            const unsigned long long ballot = __ballot(eq);
            const unsigned rank = (unsigned)__popcll(ballot & ((1ull << lane) - 1ull));
            if (lane == 0) wave_cnt[w] = (unsigned)__popcll(ballot);
            __syncthreads();
            unsigned before = 0, total = 0;
#pragma unroll
            for (int q = 0; q < kBlock / 64; ++q) { if (q < w) before += wave_cnt[q]; total += wave_cnt[q]; }
            const bool keep = key > prefix || (eq && base + before + rank < need);
            if (valid && !keep) r[j] = 0.f;
            base += total;
            __syncthreads();
        }
    }
}

// Forward_Pass__FC_AF__Softmax (:4870-4905): one wavefront per row.
__global__ __launch_bounds__(kBlock) void softmax_kernel(size_t rows, size_t H, const float *x, float *y, const float *colscale)
{
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *xr = x + row * H;
    float *yr = y + row * H;
    float mx = -3.402823466e+38f;
    for (size_t j = lane; j < H; j += 64) mx = fmaxf(mx, xr[j]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (size_t j = lane; j < H; j += 64) { float e = expf(xr[j] - mx); yr[j] = e; sum += e; }
    sum = 1.f / wave_sum(sum);
    for (size_t j = lane; j < H; j += 64) { float v = yr[j] * sum; if (colscale) v *= colscale[j]; yr[j] = v; }
}

// FF/RNN__Assign_Inputs (NN/Neural_Network__Assign_Inputs.cpp:20-204): example rows [T][W] -> [T][Bmax][W]
__global__ __launch_bounds__(kBlock) void scatter_time_major_kernel(size_t B, size_t T, size_t W, size_t Bmax, const float *src, float *dst)
{
    const size_t n = B * T * W;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const size_t w = i % W, bt = i / W, t = bt % T, b = bt / T;
        dst[(t * Bmax + b) * W + w] = src[i];
    }
}

struct SumF {
    const float *x; size_t H;
    __device__ void operator()(size_t r, size_t col, double *acc) const { acc[0] += x[r * H + col]; }
};

// grid: ceil(H / 64) workgroups; four row lanes per column (lane r: slabs r, r + 4, ...) whose sums meet in LDS and are added in
// lane order - the launch is a short chain of loads, shorter the more lanes share a column
__global__ __launch_bounds__(kBlock) void column_sum_final_kernel(size_t H, size_t S, const float *partial, float *out, int accumulate)
{
    __shared__ double red[kBlock / 64][64];
    const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
    const size_t col = (size_t)blockIdx.x * 64 + cl;
    double s = 0.0;
    if (col < H) {
#pragma unroll 8
        for (size_t y = rl; y < S; y += kBlock / 64) s += partial[y * H + col];
    }
    red[rl][cl] = s;
    __syncthreads();
    if (rl != 0 || col >= H) return;
#pragma unroll
    for (int r = 1; r < kBlock / 64; ++r) s += red[r][cl];
    out[col] = accumulate ? out[col] + (float)s : (float)s;
}

// ---- batch normalisation ----------------------------------------------------------------------------

struct BnStatF {
    const float *x; size_t H;
    __device__ void operator()(size_t r, size_t col, double *acc) const { const double s = x[r * H + col]; acc[0] += s; acc[1] += s * s; }
};

// Forward_Pass__Batch_Normalization__Training / __Batch_Renormalization__Training, "Average" loop
// (NN/Neural_Network__Forward_Pass__OpenMP.cpp:4639-4675 and :4756-4813)
__global__ __launch_bounds__(kBlock) void bn_forward_final_kernel(size_t H, size_t S, size_t rows, const float *partial, BnForwardParams p)
{
    const size_t j = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= H) return;
    double smd = 0.0, svd = 0.0;
#pragma unroll 8
    for (size_t y = 0; y < S; ++y) { smd += partial[(y * 2 + 0) * H + j]; svd += partial[(y * 2 + 1) * H + j]; }
    const float sm = (float)smd, sv = (float)svd;
    const float bscale = 1.f / (float)rows;
    const float mean = sm * bscale;
    float mavg = p.mean_avg[j];
    mavg += p.momentum * (mean - mavg);
    p.mean_avg[j] = mavg;
    const float var = sqrtf(sv * bscale - mean * mean + p.epsilon);
    float vavg = p.var_avg[j];
    vavg += p.momentum * (var - vavg);
    p.var_avg[j] = vavg;
    p.mean[j] = mean;
    p.var[j] = var;
    if (p.renorm) {
        const float g = var / vavg, lo = 1.f / p.r_max;
        p.r_corr[j] = g < lo ? lo : (g > p.r_max ? p.r_max : g);
        const float d = (mean - mavg) / vavg;
        p.d_corr[j] = d < -p.d_max ? -p.d_max : (d > p.d_max ? p.d_max : d);
    }
}

// "Activation function" loop of the same functions (:4677-4700, :4815-4836)
__global__ __launch_bounds__(kBlock) void bn_forward_apply_kernel(size_t n, BnForwardParams p)
{
    af_with(p.act, [&](auto activation) {
        const int act = activation;
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
            const size_t j = i % p.H;
            float s = (p.x[i] - p.mean[j]) / p.var[j];
            if (p.renorm) s = s * p.r_corr[j] + p.d_corr[j];
            p.hats[i] = s;
            const float y = p.scale[j] * s + p.shift[j];
            p.normalizes[i] = y;
            if (p.act_out) {   // Forward_Pass__FC_AF and the Bernoulli applier, as activation_kernel does them
                float v = af_fire(act, y);
                if (p.colscale) v *= p.colscale[j];
                p.act_out[i] = v;
            }
        }
    });
}

// The "Average" and "Activation function" loops in one launch, from the sums the producing contraction left per block
// of 32 rows: sums[blk][0][j] = sum of x, sums[blk][1][j] = sum of x * x.  A workgroup owns 64 x V columns (a lane V
// consecutive ones: V = 4 when H is a multiple of 4) and a slice of the rows; every workgroup finishes the statistics of
// its columns for itself (a few dozen loads), the workgroups of the first slice store them and move the running averages.
template <int V>
__global__ __launch_bounds__(kBlock) void bn_forward_from_sums_kernel(size_t blocks, size_t rows_per_slice, const float *sums, BnForwardParams p)
{
    const size_t j0 = ((size_t)blockIdx.x * 64 + (threadIdx.x & 63)) * V;
    const bool live = j0 < p.H;
    // every wavefront sums a quarter of the row blocks of the workgroup's columns; the four meet in LDS
    constexpr int kWaves = kBlock / 64;
    __shared__ double s_sum[kWaves][64 * V], s_sq[kWaves][64 * V];
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    {
        double smd[V], svd[V];
#pragma unroll
        for (int v = 0; v < V; ++v) { smd[v] = 0.0; svd[v] = 0.0; }
        if (live) {
            for (size_t y = w; y < blocks; y += kWaves) {
                float a[V], b[V];
                if (V == 4) { *reinterpret_cast<float4 *>(a) = *reinterpret_cast<const float4 *>(sums + (y * 2 + 0) * p.H + j0); *reinterpret_cast<float4 *>(b) = *reinterpret_cast<const float4 *>(sums + (y * 2 + 1) * p.H + j0); }
                else { a[0] = sums[(y * 2 + 0) * p.H + j0]; b[0] = sums[(y * 2 + 1) * p.H + j0]; }
#pragma unroll
                for (int v = 0; v < V; ++v) { smd[v] += a[v]; svd[v] += b[v]; }
            }
        }
#pragma unroll
        for (int v = 0; v < V; ++v) { s_sum[w][l * V + v] = smd[v]; s_sq[w][l * V + v] = svd[v]; }
    }
    __syncthreads();
    if (!live) return;
    float mean[V], var[V], scale[V], shift[V], cs[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const size_t j = j0 + v;
        double smd = 0.0, svd = 0.0;
#pragma unroll
        for (int k = 0; k < kWaves; ++k) { smd += s_sum[k][l * V + v]; svd += s_sq[k][l * V + v]; }   // in wavefront order: every lane gets the same bits
        const float sm = (float)smd, sv = (float)svd;
        const float bscale = 1.f / (float)p.rows;
        mean[v] = sm * bscale;
        var[v] = sqrtf(sv * bscale - mean[v] * mean[v] + p.epsilon);
        if (blockIdx.y == 0 && w == 0) {
            float mavg = p.mean_avg[j];
            mavg += p.momentum * (mean[v] - mavg);
            p.mean_avg[j] = mavg;
            float vavg = p.var_avg[j];
            vavg += p.momentum * (var[v] - vavg);
            p.var_avg[j] = vavg;
            p.mean[j] = mean[v];
            p.var[j] = var[v];
        }
        scale[v] = p.scale[j]; shift[v] = p.shift[j];
        cs[v] = (p.act_out && p.colscale) ? p.colscale[j] : 1.f;
    }
    const size_t r0 = (size_t)blockIdx.y * rows_per_slice, r1 = r0 + rows_per_slice < p.rows ? r0 + rows_per_slice : p.rows;
    af_with(p.act, [&](auto activation) {
        const int act = activation;
        for (size_t r = r0 + (threadIdx.x >> 6); r < r1; r += kBlock / 64) {
            const size_t i = r * p.H + j0;
            float x[V], hat[V], y[V], a[V];
            if (V == 4) *reinterpret_cast<float4 *>(x) = *reinterpret_cast<const float4 *>(p.x + i); else x[0] = p.x[i];
#pragma unroll
            for (int v = 0; v < V; ++v) {
                hat[v] = (x[v] - mean[v]) / var[v];
                y[v] = scale[v] * hat[v] + shift[v];
                a[v] = p.act_out ? af_fire(act, y[v]) * cs[v] : 0.f;
            }
            if (V == 4) {
                *reinterpret_cast<float4 *>(p.hats + i) = *reinterpret_cast<const float4 *>(hat);
                *reinterpret_cast<float4 *>(p.normalizes + i) = *reinterpret_cast<const float4 *>(y);
                if (p.act_out) *reinterpret_cast<float4 *>(p.act_out + i) = *reinterpret_cast<const float4 *>(a);
            } else {
                p.hats[i] = hat[0]; p.normalizes[i] = y[0];
                if (p.act_out) p.act_out[i] = a[0];
            }
        }
    });
}

// The backward pass's three loops in one launch, from sums[blk][0][j] = sum of dy * hats and sums[blk][1][j] = sum of dy:
// with hats = (x - mean) / sigma the two other sums of the first loop are these two times -scale / sigma.
// The launch is a chain - the blocks' sums, the column terms, the rows - and each link that asks memory for something only when
// its turn comes adds a round trip: a lane asks for its share of the sums, its columns' statistics and its first kBnHeld rows
// before it waits for anything; rows beyond those are read in the loop.  (The forward kernel measured no faster that way: it
// writes three tensors for each one it reads and is bound by those.)
constexpr int kBnHeld = 4;
template <int V>
__global__ __launch_bounds__(kBlock) void bn_backward_from_sums_kernel(size_t blocks, size_t rows_per_slice, const float *sums, BnBackwardParams p)
{
    const size_t j0 = ((size_t)blockIdx.x * 64 + (threadIdx.x & 63)) * V;
    const bool live = j0 < p.H;
    constexpr int kWaves = kBlock / 64;
    __shared__ double s_a0[kWaves][64 * V], s_a1[kWaves][64 * V];
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    const bool keeper = blockIdx.y == 0 && w == 0;   // adds the column sums to the scale's and the shift's derivatives
    const size_t r0 = (size_t)blockIdx.y * rows_per_slice, r1 = r0 + rows_per_slice < p.rows ? r0 + rows_per_slice : p.rows;
    float held_dy[kBnHeld][V], held_x[kBnHeld][V], vb[V], scale[V], mean[V], dscale_old[V], dshift_old[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { vb[v] = 1.f; scale[v] = 0.f; mean[v] = 0.f; dscale_old[v] = 0.f; dshift_old[v] = 0.f; }
    {
        double a0[V], a1[V];
#pragma unroll
        for (int v = 0; v < V; ++v) { a0[v] = 0.0; a1[v] = 0.0; }
        if (live) {
#pragma unroll
            for (int h = 0; h < kBnHeld; ++h) {
                const size_t r = r0 + w + (size_t)h * kWaves;
#pragma unroll
                for (int v = 0; v < V; ++v) { held_dy[h][v] = 0.f; held_x[h][v] = 0.f; }
                if (r < r1) {
                    if (V == 4) { *reinterpret_cast<float4 *>(held_dy[h]) = *reinterpret_cast<const float4 *>(p.dy + r * p.H + j0); *reinterpret_cast<float4 *>(held_x[h]) = *reinterpret_cast<const float4 *>(p.x + r * p.H + j0); }
                    else { held_dy[h][0] = p.dy[r * p.H + j0]; held_x[h][0] = p.x[r * p.H + j0]; }
                }
            }
#pragma unroll
            for (int v = 0; v < V; ++v) {
                vb[v] = p.var[j0 + v]; scale[v] = p.scale[j0 + v]; mean[v] = p.mean[j0 + v];
                if (keeper) { dscale_old[v] = p.dscale[j0 + v]; dshift_old[v] = p.dshift[j0 + v]; }
            }
            constexpr int kAhead = 4;   // blocks a wavefront asks for at once
            for (size_t y0 = w; y0 < blocks; y0 += kAhead * kWaves) {
                float a[kAhead][V], b[kAhead][V];
#pragma unroll
                for (int u = 0; u < kAhead; ++u) {
                    const size_t y = y0 + (size_t)u * kWaves;
#pragma unroll
                    for (int v = 0; v < V; ++v) { a[u][v] = 0.f; b[u][v] = 0.f; }
                    if (y < blocks) {
                        if (V == 4) { *reinterpret_cast<float4 *>(a[u]) = *reinterpret_cast<const float4 *>(sums + (y * 2 + 0) * p.H + j0); *reinterpret_cast<float4 *>(b[u]) = *reinterpret_cast<const float4 *>(sums + (y * 2 + 1) * p.H + j0); }
                        else { a[u][0] = sums[(y * 2 + 0) * p.H + j0]; b[u][0] = sums[(y * 2 + 1) * p.H + j0]; }
                    }
                }
#pragma unroll
                for (int u = 0; u < kAhead; ++u)
                    if (y0 + (size_t)u * kWaves < blocks) {
#pragma unroll
                        for (int v = 0; v < V; ++v) { a0[v] += a[u][v]; a1[v] += b[u][v]; }
                    }
            }
        }
#pragma unroll
        for (int v = 0; v < V; ++v) { s_a0[w][l * V + v] = a0[v]; s_a1[w][l * V + v] = a1[v]; }
    }
    __syncthreads();
    if (!live) return;
    float dmean[V], dvar[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const size_t j = j0 + v;
        double a0 = 0.0, a1 = 0.0;
#pragma unroll
        for (int k = 0; k < kWaves; ++k) { a0 += s_a0[k][l * V + v]; a1 += s_a1[k][l * V + v]; }
        if (keeper) { p.dscale[j] = dscale_old[v] + (float)a0; p.dshift[j] = dshift_old[v] + (float)a1; }
        dmean[v] = (float)a1 * scale[v] * (-1.f / vb[v]);
        dvar[v] = (float)a0 * scale[v] * (-1.f / vb[v]);
    }
    const float bsz = (float)p.rows, bscale = 1.f / (float)p.rows;
    int h = 0;
    for (size_t r = r0 + (threadIdx.x >> 6); r < r1; r += kBlock / 64, ++h) {
        const size_t i = r * p.H + j0;
        float dy[V], x[V], dx[V];
        if (h < kBnHeld) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                dy[v] = held_dy[0][v]; x[v] = held_x[0][v];
#pragma unroll
                for (int u = 1; u < kBnHeld; ++u) if (h == u) { dy[v] = held_dy[u][v]; x[v] = held_x[u][v]; }
            }
        } else if (V == 4) { *reinterpret_cast<float4 *>(dy) = *reinterpret_cast<const float4 *>(p.dy + i); *reinterpret_cast<float4 *>(x) = *reinterpret_cast<const float4 *>(p.x + i); }
        else { dy[0] = p.dy[i]; x[0] = p.x[i]; }
#pragma unroll
        for (int v = 0; v < V; ++v) {
            float e = dy[v] * scale[v];
            e *= 1.f / vb[v];
            e += dvar[v] * ((x[v] - mean[v]) / (bsz * vb[v]));
            e += dmean[v] * bscale;
            dx[v] = e;
        }
        if (V == 4) *reinterpret_cast<float4 *>(p.dx + i) = *reinterpret_cast<const float4 *>(dx); else p.dx[i] = dx[0];
    }
}

// Forward_Pass__Batch_Normalization__Inference (:4559-4589)
__global__ __launch_bounds__(kBlock) void bn_forward_inference_kernel(size_t n, size_t H, const float *x, const float *scale, const float *shift,
                                                                      const float *mavg, const float *vavg, float *out)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const size_t j = i % H;
        out[i] = scale[j] * ((x[i] - mavg[j]) / vavg[j]) + shift[j];
    }
}

// Backward_Pass__Batch_Normalization / __Batch_Renormalization, first loop
// (NN/Neural_Network__Backward_Pass__OpenMP.cpp:1385-1413, :1627-1655)
struct BnBackF {
    BnBackwardParams p;
    __device__ void operator()(size_t r, size_t col, double *acc) const
    {
        const size_t k = r * p.H + col;
        float e = p.dy[k];
        const float vb = p.var[col], rc = p.renorm ? p.r_corr[col] : 1.f;
        acc[0] += e * p.hats[k];
        acc[1] += e;
        e *= p.scale[col];
        acc[2] += e * (-rc / vb);
        acc[3] += e * (p.x[k] - p.mean[col]) * (-rc / (vb * vb));
    }
};

// reduction of the partials: dscale/dshift accumulate into the gradient vector, dmean/dvar go to scratch
__global__ __launch_bounds__(kBlock) void bn_backward_final_kernel(size_t H, size_t S, const float *partial, float *dscale, float *dshift, float *dmean_dvar)
{
    const size_t j = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= H) return;
    double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
#pragma unroll 8
    for (size_t y = 0; y < S; ++y) {
        a0 += partial[(y * 4 + 0) * H + j];
        a1 += partial[(y * 4 + 1) * H + j];
        a2 += partial[(y * 4 + 2) * H + j];
        a3 += partial[(y * 4 + 3) * H + j];
    }
    dscale[j] += (float)a0;
    dshift[j] += (float)a1;
    dmean_dvar[j] = (float)a2;
    dmean_dvar[H + j] = (float)a3;
}

// last loop (:1437-1466, :1679-1708)
__global__ __launch_bounds__(kBlock) void bn_backward_apply_kernel(size_t n, BnBackwardParams p, const float *dmean_dvar)
{
    const float bsz = (float)p.rows, bscale = 1.f / (float)p.rows;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const size_t j = i % p.H;
        const float vb = p.var[j], rc = p.renorm ? p.r_corr[j] : 1.f;
        float e = p.dy[i] * p.scale[j];
        e *= rc / vb;
        e += dmean_dvar[p.H + j] * ((p.x[i] - p.mean[j]) / (bsz * vb));
        e += dmean_dvar[j] * bscale;
        p.dx[i] = e;
    }
}

// ---- output-layer delta, loss and accuracy -------------------------------------------------------------
// FF__Compute__Error (NN/Neural_Network__Compute__Error__OpenMP.cpp:22-141), RNN__Compute__Error
// (NN/Neural_Network__Recurrent_Compute__Error__OpenMP.cpp:22-159), Update_Error
// (NN/Neural_Network__Compute__Error__Loop.cpp:20-77).  One wavefront per (t, example) row.

__device__ __forceinline__ float sign_f(float v) { return v > 0.f ? 1.f : (v < 0.f ? -1.f : 0.f); }

// V: elements per lane and trip (4: rows whose width is a multiple of 4, 16-byte loads and stores; 1 otherwise)
template <int V>
__global__ __launch_bounds__(kBlock) void compute_error_kernel(ErrorParams p)
{
    __shared__ float red[5][kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t nrows = (p.T - p.first_t) * p.B;
    float loss = 0.f, cnt = 0.f, acc = 0.f, bits = 0.f, sum_y = 0.f;
    // wavefronts stride over the rows and keep their sums in registers: one set of fp64 atomics per workgroup
    for (size_t rid = (size_t)blockIdx.x * (kBlock / 64) + wave; rid < nrows; rid += (size_t)gridDim.x * (kBlock / 64)) {
        const size_t t = p.first_t + rid / p.B, b = rid % p.B;
        const size_t off = (t * p.Bmax + b) * p.H;
        const float *y = p.values + off, *pre = p.pre + off;
        const float *d = p.desired + (b * p.T + t) * p.H;
        float *err = p.errors + off;
        // cross-entropy accuracy: first index whose target is 1, last index reaching the maximum (">=")
        if (p.accuracy == MYEA_ACCURACY_CROSS_ENTROPY) {
            unsigned want = 0xffffffffu; float mx = -3.402823466e+38f; unsigned got = 0;
            for (size_t j = lane; j < p.H; j += 64) {
                if (d[j] == 1.f && (unsigned)j < want) want = (unsigned)j;
                if (y[j] >= mx) { mx = y[j]; got = (unsigned)j; }
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const unsigned w2 = __shfl_xor(want, o, 64);
                const float m2 = __shfl_xor(mx, o, 64);
                const unsigned g2 = __shfl_xor(got, o, 64);
                want = min(want, w2);
                if (m2 > mx || (m2 == mx && g2 > got)) { mx = m2; got = g2; }
            }
            if (want == 0xffffffffu) want = (unsigned)p.H;
            if (lane == 0) acc += (want == got) ? 1.f : 0.f;
        }
        for (size_t j0 = (size_t)lane * V; j0 < p.H; j0 += 64 * V) {
            float y_v[V], d_v[V], pre_v[V], err_v[V];
            if (V == 4) {
                const f32x4 y4 = *reinterpret_cast<const f32x4 *>(y + j0), d4 = *reinterpret_cast<const f32x4 *>(d + j0);
                f32x4 q4 = {0.f, 0.f, 0.f, 0.f};
                if (p.write_delta && !p.rnn_pre_quirk) q4 = *reinterpret_cast<const f32x4 *>(pre + j0);
#pragma unroll
                for (int e = 0; e < V; ++e) { y_v[e] = y4[e]; d_v[e] = d4[e]; pre_v[e] = q4[e]; }
            } else {
                y_v[0] = y[j0]; d_v[0] = d[j0]; pre_v[0] = (p.write_delta && !p.rnn_pre_quirk) ? pre[j0] : 0.f;
            }
#pragma unroll
            for (int v = 0; v < V; ++v) {
            const size_t j = j0 + v;
            const float yo = y_v[v], de = d_v[v], diff = yo - de;
            err_v[v] = 0.f;
            float e = 0.f; bool counted = true;
            switch (p.loss) {
            case MYEA_LOSS_ME:
            case MYEA_LOSS_L1: e = diff; break;
            case MYEA_LOSS_MAE: e = fabsf(diff); break;
            case MYEA_LOSS_L2:
            case MYEA_LOSS_MSE:
            case MYEA_LOSS_RMSE: e = diff * diff; break;
            case MYEA_LOSS_MAPE: { float q = yo != 0.f ? yo : fmaxf(yo, 1e-6f); e = fabsf(diff / q); break; }
            case MYEA_LOSS_SMAPE: e = fabsf(diff) / (fabsf(de) + fabsf(yo)); break;
            case MYEA_LOSS_CROSS_ENTROPY: {
                float q = yo != 0.f ? yo : fmaxf(yo, 1e-6f);
                e = (p.H == 1) ? -(de * logf(q) + (1.f - de) * logf(1.f - q)) : -(de * logf(q));
                break;
            }
            case MYEA_LOSS_BIT: counted = false; if (fabsf(diff) >= p.bit_fail_limit) bits += 1.f; break;
            default: counted = false; break;
            }
            if (counted) { loss += e; cnt += 1.f; }
            switch (p.accuracy) {
            case MYEA_ACCURACY_DISTANCE: if (fabsf(diff) <= p.accuracy_variance) acc += 1.f; break;
            case MYEA_ACCURACY_DIRECTIONAL:
                // RNN: direction of change against the previous target (Recurrent_Compute__Error__OpenMP.cpp:115-120)
                if (!p.rnn_pre_quirk || t == 0 || sign_f(de - d[(long)j - (long)p.H]) == sign_f(yo - d[(long)j - (long)p.H])) acc += 1.f;
                break;
            case MYEA_ACCURACY_SIGN:
                if (sign_f(de) == sign_f(yo) || (sign_f(de) == 0.f && yo >= -1.192092896e-07f && yo <= 1.192092896e-07f)) acc += 1.f;
                break;
            case MYEA_ACCURACY_R: acc += de; sum_y += yo; break;  // running sums of the desired and the predicted values
            default: break;
            }
            if (!p.write_delta) continue;  // Compute__Loss: the same accumulation, no delta
            const float q = p.rnn_pre_quirk ? pre[0] : pre_v[v];
            err_v[v] = af_derive(p.unit_act ? p.unit_act[j] : p.act, q, p.unit_steep ? p.unit_steep[j] : p.steep, yo) * diff;
            }
            if (p.write_delta) {
                if (V == 4) *reinterpret_cast<f32x4 *>(err + j0) = f32x4{err_v[0], err_v[1], err_v[2], err_v[3]};
                else err[j0] = err_v[0];
            }
        }
    }
    loss = wave_sum(loss); cnt = wave_sum(cnt); acc = wave_sum(acc); bits = wave_sum(bits); sum_y = wave_sum(sum_y);
    if (lane == 0) { red[0][wave] = loss; red[1][wave] = cnt; red[2][wave] = acc; red[3][wave] = bits; red[4][wave] = sum_y; }
    __syncthreads();
    if (threadIdx.x < 5) {
        const float v = red[threadIdx.x][0] + red[threadIdx.x][1] + red[threadIdx.x][2] + red[threadIdx.x][3];
        if (v != 0.f) atomicAdd(&p.loss_acc[threadIdx.x], (double)v);
    }
}

// FF / RNN__Compute__Accuracy__R (NN/Neural_Network__Compute__R__Loop.cpp:38-90, NN/Neural_Network__Recurrent_Compute__R__Loop.cpp:20-75):
// numerator and the two denominators of the Pearson correlation into loss_acc[5..7]
__global__ __launch_bounds__(kBlock) void accuracy_r_kernel(ErrorParams p, float mean_d, float mean_y)
{
    __shared__ float red[3][kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t nrows = (p.T - p.first_t) * p.B;
    float num = 0.f, den_d = 0.f, den_y = 0.f;
    for (size_t rid = (size_t)blockIdx.x * (kBlock / 64) + wave; rid < nrows; rid += (size_t)gridDim.x * (kBlock / 64)) {
        const size_t t = p.first_t + rid / p.B, b = rid % p.B;
        const float *y = p.values + (t * p.Bmax + b) * p.H, *d = p.desired + (b * p.T + t) * p.H;
        for (size_t j = lane; j < p.H; j += 64) {
            const float dd = d[j] - mean_d, dy = y[j] - mean_y;
            num += dd * dy; den_d += dd * dd; den_y += dy * dy;
        }
    }
    num = wave_sum(num); den_d = wave_sum(den_d); den_y = wave_sum(den_y);
    if (lane == 0) { red[0][wave] = num; red[1][wave] = den_d; red[2][wave] = den_y; }
    __syncthreads();
    if (threadIdx.x < 3) {
        const float v = red[threadIdx.x][0] + red[threadIdx.x][1] + red[threadIdx.x][2] + red[threadIdx.x][3];
        if (v != 0.f) atomicAdd(&p.loss_acc[5 + threadIdx.x], (double)v);
    }
}

// rows index[0..B) of a resident dataset -> one contiguous batch (Dataset_Mini_Batch::Increment_Mini_Batch,
// NN/Dataset__Mini_Batch.cpp:290-314, re-points row pointers; here the rows are copied on the device)
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(size_t B, size_t row_floats, const unsigned long long *__restrict__ index,
                                                             const float *__restrict__ src, float *__restrict__ dst)
{
    const bool vec = (row_floats & 3) == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
    if (vec) {
        const size_t r4 = row_floats / 4, n = B * r4;
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
            const size_t b = i / r4, j = i - b * r4;
            reinterpret_cast<f32x4 *>(dst)[i] = reinterpret_cast<const f32x4 *>(src + index[b] * row_floats)[j];
        }
    } else {
        const size_t n = B * row_floats;
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
            const size_t b = i / row_floats, j = i - b * row_floats;
            dst[i] = src[index[b] * row_floats + j];
        }
    }
}

// ---- global-norm clipping and the fused optimizer update -------------------------------------------------

// Euclidean_Norm (NN/Neural_Network__Regularization__Max_Norm_Constraints.cpp:48-140), sum-of-squares part
__global__ __launch_bounds__(kBlock) void sum_squares_partial_kernel(size_t n, const float *g, float *partials)
{
    __shared__ float red[kBlock / 64];
    float s = 0.f;
    const size_t n4 = n / 4;
    const f32x4 *g4 = reinterpret_cast<const f32x4 *>(g);
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += (size_t)gridDim.x * kBlock) {
        const f32x4 v = g4[i];
        s += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) { const float v = g[n4 * 4 + threadIdx.x]; s += v * v; }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) partials[blockIdx.x] = red[0] + red[1] + red[2] + red[3];
}

__global__ __launch_bounds__(kBlock) void sum_squares_final_kernel(unsigned nparts, const float *partials, float *out)
{
    __shared__ float red[kBlock / 64];
    float s = 0.f;
    for (unsigned i = threadIdx.x; i < nparts; i += kBlock) s += partials[i];
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) out[0] = red[0] + red[1] + red[2] + red[3];
}

struct UpdateDev {
    size_t n, n_weights;
    float *w, *g, *s0, *s1, *s2;
    float lr, mu, lr_t, beta1, beta2, eps, lower, upper, wd;
    const float *norm_sq;
    float clip, grad_scale;
    const unsigned *fault;
    unsigned long long *applied;
};

// One element of Update_Parameters__Adam (NN/Neural_Network__Adam.cpp:43-97), __AMSGrad
// (NN/Neural_Network__AMSGrad.cpp:43-105), __AdaBound (NN/Neural_Network__AdaBound.cpp:43-110),
// Update_Parameter__Gradient_Descent (NN/Neural_Network__Gradient_Descent.cpp:84-120), __Momentum
// (NN/Neural_Network__Gradient_Descent_Momentum.cpp:22-62), Nesterov
// (NN/Neural_Network__Nesterov_Accelerated_Gradient.cpp:22-64; sign of the lr*g term as written there).
// __AMSBound (NN/Neural_Network__AMSBound.cpp:43-110), iRPROP+ (NN/Neural_Network__iRPROP_plus.cpp:28-117).
// NosAdam (NN/Neural_Network__NosAdam.cpp:43-100) is KIND 3 with the host's beta2 at time t.
// KIND: 0 GD, 1 momentum, 2 Nesterov, 3 Adam, 4 AMSGrad, 5 AdaBound, 6 AMSBound,
//       7 iRPROP+ (a = previous delta, b = previous step, c = previous slope; lr / mu = increase / decrease factor,
//         lower / upper = smallest / largest step, beta1 != 0 when the loss got worse),
//       8 iRPROP- (NN/Neural_Network__iRPROP_minus.cpp:21-67; b, c and the scalars as for iRPROP+; a slope that changed sign
//         is forgotten and, the sign of zero being zero, leaves the weight where it is).
template <int KIND, bool WD>
__device__ __forceinline__ void update_one(const UpdateDev &p, float gs, float &w, float g, float &a, float &b, float &c, bool is_weight)
{
    g *= gs;
    float step;
    if (KIND == 8) {
        const float same = c * g;
        float d = b;
        if (same > 0.f) b = d = fminf(b * p.lr, p.upper);
        else if (same < 0.f) { b = d = fmaxf(b * p.mu, p.lower); g = 0.f; }
        w += -(g > 0.f ? 1.f : (g < 0.f ? -1.f : 0.f)) * d;
        c = g;
        return;
    }
    if (KIND == 7) {
        const float sg = g > 0.f ? 1.f : (g < 0.f ? -1.f : 0.f), same = c * g;
        if (same > 0.f) {
            b = fminf(b * p.lr, p.upper);
            a = -sg * b;
            w += a;
            c = g;
        } else if (same < 0.f) {
            b = fmaxf(b * p.mu, p.lower);
            if (p.beta1 != 0.f) w -= a;
            c = 0.f;
        } else {
            a = -sg * b;
            w += a;
            c = g;
        }
        return;
    }
    if (KIND == 0) {
        step = p.lr * g;
    } else if (KIND == 1) {
        a = p.lr * g + p.mu * a;
        step = a;
    } else if (KIND == 2) {
        a = p.lr * g + p.mu * a;
        step = p.mu * a - p.lr * g;
    } else {
        a = p.beta1 * a + (1.f - p.beta1) * g;
        b = p.beta2 * b + (1.f - p.beta2) * g * g;
        if (KIND == 3) step = p.lr_t * a / (sqrtf(b) + p.eps);
        else if (KIND == 4) { c = fmaxf(c, b); step = p.lr_t * a / (sqrtf(c) + p.eps); }
        else {
            if (KIND == 6) c = fmaxf(c, b);
            float r = p.lr_t / (sqrtf(KIND == 6 ? c : b) + p.eps);
            r = r < p.lower ? p.lower : (r > p.upper ? p.upper : r);
            step = r * a;
        }
    }
    if (WD) step += (is_weight ? 1.f : 0.f) * p.wd * w;
    w -= step;
}

template <int KIND, bool WD>
__global__ __launch_bounds__(kBlock) void update_kernel(UpdateDev p)
{
    // A kernel of an earlier pass whose bounded wait gave up has left that pass incomplete and raised this word (earlier in
    // stream order: a plain load sees it): the update then changes nothing - weights, optimizer vectors and gradient stay as
    // they are - until the host has dealt with it.  The word is fetched with the operands and looked at in front of the stores,
    // so that no wavefront waits for it before it has its own loads in flight.
    const unsigned faulted = p.fault ? *p.fault : 0u;
    float gs = p.grad_scale;
    if (p.norm_sq) {  // Clip_Gradient: scale when norm >= clip (NN/Neural_Network__Clip_Gradient.cpp:81-94)
        const float norm = sqrtf(p.norm_sq[0]);
        if (norm >= p.clip) gs = p.clip / norm;
    }
    constexpr bool kA = KIND >= 1 && KIND != 8, kB = KIND >= 3, kC = KIND == 4 || KIND >= 6;
    const size_t n4 = p.n / 4;
    f32x4 *w4 = reinterpret_cast<f32x4 *>(p.w), *g4 = reinterpret_cast<f32x4 *>(p.g);
    f32x4 *a4 = reinterpret_cast<f32x4 *>(p.s0), *b4 = reinterpret_cast<f32x4 *>(p.s1), *c4 = reinterpret_cast<f32x4 *>(p.s2);
    // One 128-bit element per lane and no loop: every vector is streamed exactly once, so the stores bypass the caches
    // (non-temporal; the same hint on the loads was measured to cost the update a tenth of its rate) and a grid of n/1024
    // workgroups keeps enough requests in flight for HBM.
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n4) {
        const f32x4 wv = w4[i], gv = g4[i];
        f32x4 av = {0.f, 0.f, 0.f, 0.f}, bv = av, cv = av;
        if (kA) av = a4[i];
        if (kB) bv = b4[i];
        if (kC) cv = c4[i];
        if (faulted) return;
        float w[4], a[4], b[4], c[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            w[e] = wv[e]; a[e] = av[e]; b[e] = bv[e]; c[e] = cv[e];
            update_one<KIND, WD>(p, gs, w[e], gv[e], a[e], b[e], c[e], i * 4 + e < p.n_weights);
        }
        __builtin_nontemporal_store(f32x4{w[0], w[1], w[2], w[3]}, &w4[i]);
        if (kA) __builtin_nontemporal_store(f32x4{a[0], a[1], a[2], a[3]}, &a4[i]);
        if (kB) __builtin_nontemporal_store(f32x4{b[0], b[1], b[2], b[3]}, &b4[i]);
        if (kC) __builtin_nontemporal_store(f32x4{c[0], c[1], c[2], c[3]}, &c4[i]);
        __builtin_nontemporal_store(f32x4{0.f, 0.f, 0.f, 0.f}, &g4[i]);
    }
    if (faulted) return;
    if (p.applied && blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(p.applied, 1ull);   // the launch that completes a whole update counts it
    if (blockIdx.x == 0 && threadIdx.x < (p.n & 3)) {
        const size_t i = n4 * 4 + threadIdx.x;
        float w = p.w[i], a = kA ? p.s0[i] : 0.f, b = kB ? p.s1[i] : 0.f, c = kC ? p.s2[i] : 0.f;
        update_one<KIND, WD>(p, gs, w, p.g[i], a, b, c, i < p.n_weights);
        p.w[i] = w;
        if (kA) p.s0[i] = a;
        if (kB) p.s1[i] = b;
        if (kC) p.s2[i] = c;
        p.g[i] = 0.f;
    }
}

// Euclidean_Norm (NN/Neural_Network__Regularization__Max_Norm_Constraints.cpp:48-137): a weight segment whose norm is at
// or above max_norm is rescaled to max_norm.  GROUP threads (one wave, or the whole workgroup) own one segment.
template <int GROUP>
__global__ __launch_bounds__(kBlock) void max_norm_kernel(size_t nseg, const unsigned long long *__restrict__ first, const unsigned *__restrict__ len,
                                                          float max_norm, float *w)
{
    constexpr int kPerBlock = kBlock / GROUP;
    __shared__ float red[kBlock / 64];
    const size_t seg = (size_t)blockIdx.x * kPerBlock + threadIdx.x / GROUP;
    const unsigned lane = threadIdx.x % GROUP;
    const bool live = seg < nseg;
    float *v = live ? w + first[seg] : nullptr;
    const unsigned L = live ? len[seg] : 0u;
    const bool vec = ((reinterpret_cast<uintptr_t>(v) | ((uintptr_t)L * 4u)) & 15u) == 0;
    float s = 0.f;
    if (vec) {
        const f32x4 *v4 = reinterpret_cast<const f32x4 *>(v);
        for (unsigned i = lane; i < L / 4; i += GROUP) { const f32x4 x = v4[i]; s += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3]; }
    } else {
        for (unsigned i = lane; i < L; i += GROUP) s += v[i] * v[i];
    }
    s = wave_sum(s);
    if (GROUP > 64) {
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
        __syncthreads();
        s = red[0] + red[1] + red[2] + red[3];
    }
    const float norm = sqrtf(s);
    if (norm >= max_norm) {
        const float r = max_norm / norm;
        if (vec) {
            f32x4 *v4 = reinterpret_cast<f32x4 *>(v);
            for (unsigned i = lane; i < L / 4; i += GROUP) { f32x4 x = v4[i]; x[0] *= r; x[1] *= r; x[2] *= r; x[3] *= r; v4[i] = x; }
        } else {
            for (unsigned i = lane; i < L; i += GROUP) v[i] *= r;
        }
    }
}

template <int KIND>
int launch_update_kind(hipStream_t s, const UpdateDev &d, bool wd)
{
    const unsigned grid = grid_for(d.n / 4 + 1, kBlock, 0x7fffffffu);   // at least one workgroup, also for an empty range that only counts
    if (wd) hipLaunchKernelGGL((update_kernel<KIND, true>), dim3(grid), dim3(kBlock), 0, s, d);
    else hipLaunchKernelGGL((update_kernel<KIND, false>), dim3(grid), dim3(kBlock), 0, s, d);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

}  // namespace

// ---- launchers ----------------------------------------------------------------------------------------

int launch_fill(hipStream_t s, float *p, size_t n, float v)
{
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(fill_kernel, dim3(grid_for(n, kBlock, 4096)), dim3(kBlock), 0, s, p, n, v);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_activation(hipStream_t s, int act, size_t rows, size_t H, const float *x, float *y, const float *colscale, const int *unit_act)
{
    const size_t n = rows * H;
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(activation_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, act, unit_act, n, H, x, y, colscale);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_softmax(hipStream_t s, size_t rows, size_t H, const float *x, float *y, const float *colscale)
{
    if (rows == 0 || H == 0) return MYEA_OK;
    hipLaunchKernelGGL(softmax_kernel, dim3(grid_for(rows, kBlock / 64)), dim3(kBlock), 0, s, rows, H, x, y, colscale);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_activation_derive(hipStream_t s, int act, float steep, size_t n, const float *pre, const float *val, const float *dy, float *dx,
                             const int *unit_act, const float *unit_steep, size_t H)
{
    if (n == 0) return MYEA_OK;
    if ((unit_act || unit_steep) && H == 0) { set_last_error("activation derive: per-unit arrays need the row width"); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(activation_derive_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, act, steep, unit_act, unit_steep, H ? H : 1, n, pre, val, dy, dx);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// Forward_Pass__Zero_Padded_Identity (NN/Neural_Network__Forward_Pass__OpenMP.cpp:5158-5240) and
// Backward_Pass__Residual (NN/Neural_Network__Backward_Pass__OpenMP.cpp:1155-1215) as one shifted add.
__global__ void padded_add_kernel(size_t n, size_t wo, const float *__restrict__ a, size_t wa, long sa,
                                  const float *__restrict__ b, size_t wb, long sb, float *__restrict__ out)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / wo;
        const long j = (long)(i - r * wo);
        float v = 0.f;
        const long ja = j + sa;
        if (ja >= 0 && ja < (long)wa) v = a[r * wa + (size_t)ja];
        if (b) {
            const long jb = j + sb;
            if (jb >= 0 && jb < (long)wb) v += b[r * wb + (size_t)jb];
        }
        out[i] = v;
    }
}

int launch_padded_add(hipStream_t s, size_t rows, size_t wo, const float *a, size_t wa, long sa,
                      const float *b, size_t wb, long sb, float *out)
{
    const size_t n = rows * wo;
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(padded_add_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, n, wo, a, wa, sa, b, wb, sb, out);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_colscale(hipStream_t s, size_t rows, size_t H, float *y, const float *colscale)
{
    const size_t n = rows * H;
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(colscale_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, n, H, y, colscale);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_mask_to_scale(hipStream_t s, size_t n, const uint8_t *mask, float on, float *colscale)
{
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(mask_to_scale_kernel, dim3(grid_for(n, kBlock, 4096)), dim3(kBlock), 0, s, n, mask, on, colscale);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// scratch: 64 * H floats at most (S <= 64 row splits)
int launch_column_sum(hipStream_t s, size_t rows, size_t H, const float *x, float *out, int accumulate, float *scratch)
{
    if (H == 0) return MYEA_OK;
    if (rows == 0) { if (!accumulate) return launch_fill(s, out, H, 0.f); return MYEA_OK; }
    size_t S, chunk;
    split_rows(rows, H, S, chunk);
    SumF f{x, H};
    hipLaunchKernelGGL((column_partial_kernel<1, SumF>), dim3((unsigned)((H + 63) / 64), (unsigned)S), dim3(kBlock), 0, s, rows, H, chunk, scratch, f);
    MYEA_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(column_sum_final_kernel, dim3(grid_for(H, 64)), dim3(kBlock), 0, s, H, S, scratch, out, accumulate);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_column_sum_final(hipStream_t s, size_t H, size_t S, const float *partial, float *out, int accumulate)
{
    if (H == 0) return MYEA_OK;
    hipLaunchKernelGGL(column_sum_final_kernel, dim3(grid_for(H, 64)), dim3(kBlock), 0, s, H, S, partial, out, accumulate);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_dropout_noise(hipStream_t s, size_t n, float *noise, int normal, float a, float b, unsigned long long seed, unsigned long long stream_id)
{
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(dropout_noise_kernel, dim3(grid_for((n + 3) / 4, kBlock)), dim3(kBlock), 0, s, n, noise, normal, a, b, seed, stream_id);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_dropout_noise_apply(hipStream_t s, size_t n, float *y, const float *noise, int uout)
{
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(dropout_noise_apply_kernel, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, s, n, y, noise, uout);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_shakedrop_apply(hipStream_t s, size_t rows, size_t W, float *x, const float *mask, const float *draws, float constant)
{
    if (rows * W == 0) return MYEA_OK;
    hipLaunchKernelGGL(shakedrop_apply_kernel, dim3(grid_for(rows * W, kBlock)), dim3(kBlock), 0, s, rows, W, x, mask, draws, constant);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_threshold(hipStream_t s, size_t n, float *x, float p)
{
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(threshold_kernel, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, s, n, x, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_k_sparse(hipStream_t s, size_t rows, size_t H, size_t k, float *x)
{
    if (rows == 0 || k >= H) return MYEA_OK;   // k == width: nothing to filter (:288)
    if (k == 0) { set_last_error("k-sparse filter: k is 0"); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(k_sparse_kernel, dim3(grid_for(rows, 1)), dim3(kBlock), 0, s, rows, H, (unsigned)k, x);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_ind_rnn_forward(hipStream_t s, const IndRnnParams &p)
{
    if (p.B * p.H == 0 || p.T == 0) return MYEA_OK;
    hipLaunchKernelGGL(ind_rnn_forward_kernel, dim3(grid_for(p.B * p.H, kIndRnnLanes)), dim3(kIndRnnLanes), 0, s, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_ind_rnn_backward(hipStream_t s, const IndRnnParams &p)
{
    if (p.B * p.H == 0 || p.T == 0) return MYEA_OK;
    hipLaunchKernelGGL(ind_rnn_backward_kernel, dim3(grid_for(p.B * p.H, kIndRnnLanes)), dim3(kIndRnnLanes), 0, s, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// scratch: 64 * H floats at most
int launch_ind_rnn_self_weight_gradient(hipStream_t s, size_t T, size_t B, size_t Bmax, size_t H, const float *afs, const float *dafs, float *du, float *scratch)
{
    if (H == 0 || B == 0 || T < 2) return MYEA_OK;
    const size_t rows = (T - 1) * B;
    size_t S, chunk;
    split_rows(rows, H, S, chunk);
    IndRnnDotF f{afs, dafs, H, B, Bmax};
    hipLaunchKernelGGL((column_partial_kernel<1, IndRnnDotF>), dim3((unsigned)((H + 63) / 64), (unsigned)S), dim3(kBlock), 0, s, rows, H, chunk, scratch, f);
    MYEA_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(column_sum_final_kernel, dim3(grid_for(H, 64)), dim3(kBlock), 0, s, H, S, scratch, du, 1);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// grid (ceil(longest / 256), ranges)
__global__ __launch_bounds__(kBlock) void clip_ranges_kernel(const ClipRange *__restrict__ ranges, float *w)
{
    const ClipRange r = ranges[blockIdx.y];
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= r.count) return;
    const float v = w[r.first + i];
    w[r.first + i] = v < r.lo ? r.lo : (v > r.hi ? r.hi : v);
}

int launch_clip_ranges(hipStream_t s, const ClipRange *ranges, size_t count, size_t longest, float *w)
{
    if (count == 0 || longest == 0) return MYEA_OK;
    if (count > 65535) { set_last_error("clip_ranges: %zu ranges in one launch", count); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(clip_ranges_kernel, dim3(grid_for(longest, kBlock), (unsigned)count), dim3(kBlock), 0, s, ranges, w);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_clip_range(hipStream_t s, size_t n, float *w, float lo, float hi)
{
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(clip_range_kernel, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, s, n, w, lo, hi);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_bn_forward_training(hipStream_t s, const BnForwardParams &p, float *scratch)
{
    if (p.H == 0 || p.rows == 0) return MYEA_OK;
    size_t S, chunk;
    split_rows(p.rows, p.H, S, chunk);
    BnStatF f{p.x, p.H};
    hipLaunchKernelGGL((column_partial_kernel<2, BnStatF>), dim3((unsigned)((p.H + 63) / 64), (unsigned)S), dim3(kBlock), 0, s, p.rows, p.H, chunk, scratch, f);
    MYEA_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(bn_forward_final_kernel, dim3(grid_for(p.H, kBlock)), dim3(kBlock), 0, s, p.H, S, p.rows, scratch, p);
    MYEA_HIP_TRY(hipGetLastError());
    const size_t n = p.rows * p.H;
    hipLaunchKernelGGL(bn_forward_apply_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, n, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// rows per slice so that the grid has about a thousand workgroups, at least `least` rows each
static size_t bn_rows_per_slice(size_t rows, size_t colblocks, size_t least)
{
    size_t slices = (1024 + colblocks - 1) / colblocks;
    if (slices > (rows + least - 1) / least) slices = (rows + least - 1) / least;
    if (slices < 1) slices = 1;
    return (rows + slices - 1) / slices;
}
static bool rows_of_float4(size_t H, std::initializer_list<const void *> tensors)
{
    if (H % 4) return false;
    for (const void *t : tensors) if (t && (reinterpret_cast<uintptr_t>(t) & 15u)) return false;
    return true;
}

int launch_bn_forward_training_from_sums(hipStream_t s, const BnForwardParams &p, const float *sums, size_t blocks)
{
    if (p.H == 0 || p.rows == 0) return MYEA_OK;
    if (p.renorm || !sums || blocks == 0) { set_last_error("bn_forward_training_from_sums: plain batch normalisation with its column sums only"); return MYEA_E_INVALID; }
    static_assert(kBlock % 64 == 0, "64 lanes of columns per workgroup");
    const bool wide = rows_of_float4(p.H, {p.x, p.hats, p.normalizes, p.act_out});
    // a row a wavefront where the batch allows: the launch's time is its row loop, a memory round trip an iteration (512 x 2048:
    // 10.1 us at 4 rows a slice, 10.5 at 8, 12.1 at 16)
    const size_t colblocks = (p.H + (wide ? 255 : 63)) / (wide ? 256 : 64), per = bn_rows_per_slice(p.rows, colblocks, 4);
    const dim3 grid((unsigned)colblocks, (unsigned)((p.rows + per - 1) / per));
    if (wide) hipLaunchKernelGGL(bn_forward_from_sums_kernel<4>, grid, dim3(kBlock), 0, s, blocks, per, sums, p);
    else hipLaunchKernelGGL(bn_forward_from_sums_kernel<1>, grid, dim3(kBlock), 0, s, blocks, per, sums, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_bn_backward_from_sums(hipStream_t s, const BnBackwardParams &p, const float *sums, size_t blocks)
{
    if (p.H == 0 || p.rows == 0) return MYEA_OK;
    if (p.renorm || !sums || blocks == 0) { set_last_error("bn_backward_from_sums: plain batch normalisation with its column sums only"); return MYEA_E_INVALID; }
    const bool wide = rows_of_float4(p.H, {p.x, p.dy, p.dx});
    const size_t colblocks = (p.H + (wide ? 255 : 63)) / (wide ? 256 : 64), per = bn_rows_per_slice(p.rows, colblocks, 4 * kBnHeld);
    const dim3 grid((unsigned)colblocks, (unsigned)((p.rows + per - 1) / per));
    if (wide) hipLaunchKernelGGL(bn_backward_from_sums_kernel<4>, grid, dim3(kBlock), 0, s, blocks, per, sums, p);
    else hipLaunchKernelGGL(bn_backward_from_sums_kernel<1>, grid, dim3(kBlock), 0, s, blocks, per, sums, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// Every time step of a [T][Bmax][H] tensor in one launch.  Each time step has statistics of its own (the reference runs the
// layer's normalisation once per time step); workgroup (column block, t) owns CW columns of time step t over all of its rows:
// the column sums meet in LDS, one lane per column finishes the statistics with bn_forward_final_kernel's arithmetic, then the
// workgroup applies them as bn_forward_apply_kernel does.  p's per-time-step vectors (mean, var, averages,
// corrections, colscale) are those of time step 0, H apart from one step to the next; its tensors those of time step 0,
// Bmax * H apart.  training == 0: the running averages of each time step, nothing written but the output.
// A launch is a chain of passes that wait for each other, so a lane asks for its first kSeqHeld rows and its column's parameters
// before anything waits and keeps those rows in registers for the second pass; the column sums take the two-stage form of
// norm_fold_partial / norm_sum_partials.
constexpr int kSeqHeld = 4;
template <int CW>   // columns per workgroup: 64, or 16 / 4 for narrow layers (more row lanes, shorter loops)
__global__ __launch_bounds__(kBlock) void bn_forward_sequence_kernel(BnForwardParams p, size_t Bmax, int training)
{
    constexpr int kLanes = kBlock / CW, NW = kBlock / 64, NP = NW * kNormPartials<CW>;
    __shared__ double red[2][NP][CW];
    __shared__ float s_stat[4][CW];
    const int c = threadIdx.x % CW, rl = threadIdx.x / CW, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const size_t t = blockIdx.y, j = (size_t)blockIdx.x * CW + c;
    const bool live = j < p.H;
    const size_t base = t * Bmax * p.H, sj = t * p.H + j;
    // the lanes of wavefront 0 that finish the statistics: column fc of the workgroup
    const int fc = norm_finish_column<CW>(lane);
    const size_t fj = (size_t)blockIdx.x * CW + fc, sfj = t * p.H + fj;
    const bool keeper = wave == 0 && norm_finish_keeper<CW>(lane) && fj < p.H;
    float held[kSeqHeld], scale = 0.f, shift = 0.f, cs = 1.f, mavg = 0.f, vavg = 1.f;
#pragma unroll
    for (int h = 0; h < kSeqHeld; ++h) held[h] = 0.f;
    if (live) {
#pragma unroll
        for (int h = 0; h < kSeqHeld; ++h) {
            const size_t r = rl + (size_t)h * kLanes;
            if (r < p.rows) held[h] = p.x[base + r * p.H + j];
        }
        scale = p.scale[j]; shift = p.shift[j];
        if (p.colscale) cs = p.colscale[sj];
        if (!training) { mavg = p.mean_avg[sj]; vavg = p.var_avg[sj]; }
    }
    if (training && keeper) { mavg = p.mean_avg[sfj]; vavg = p.var_avg[sfj]; }
    if (training) {
        double sm = 0.0, sv = 0.0;
        if (live) {
#pragma unroll
            for (int h = 0; h < kSeqHeld; ++h)
                if (rl + (size_t)h * kLanes < p.rows) { const double v = held[h]; sm += v; sv += v * v; }
            for (size_t r = rl + (size_t)kSeqHeld * kLanes; r < p.rows; r += kLanes) { const double v = p.x[base + r * p.H + j]; sm += v; sv += v * v; }
        }
        sm = norm_fold_partial<CW>(sm); sv = norm_fold_partial<CW>(sv);
        if (norm_partial_holder<CW>(lane)) { const int slot = norm_partial_index<CW>(wave, lane); red[0][slot][c] = sm; red[1][slot][c] = sv; }
        __syncthreads();
        if (wave == 0) {
            const double smd = norm_sum_partials<CW, NP>(red[0], lane), svd = norm_sum_partials<CW, NP>(red[1], lane);
            if (keeper) {
                const float bscale = 1.f / (float)p.rows;
                const float mean = (float)smd * bscale;
                mavg += p.momentum * (mean - mavg);
                p.mean_avg[sfj] = mavg;
                const float var = sqrtf((float)svd * bscale - mean * mean + p.epsilon);
                vavg += p.momentum * (var - vavg);
                p.var_avg[sfj] = vavg;
                p.mean[sfj] = mean;
                p.var[sfj] = var;
                float rc = 1.f, dc = 0.f;
                if (p.renorm) {
                    const float g = var / vavg, lo = 1.f / p.r_max;
                    rc = g < lo ? lo : (g > p.r_max ? p.r_max : g);
                    const float d = (mean - mavg) / vavg;
                    dc = d < -p.d_max ? -p.d_max : (d > p.d_max ? p.d_max : d);
                    p.r_corr[sfj] = rc; p.d_corr[sfj] = dc;
                }
                s_stat[0][fc] = mean; s_stat[1][fc] = var; s_stat[2][fc] = rc; s_stat[3][fc] = dc;
            }
        }
        __syncthreads();
    }
    if (!live) return;
    if (!training) {
        for (size_t r = rl; r < p.rows; r += kLanes) {
            const size_t i = base + r * p.H + j;
            p.normalizes[i] = scale * ((p.x[i] - mavg) / vavg) + shift;
        }
        return;
    }
    const float mean = s_stat[0][c], var = s_stat[1][c], rc = s_stat[2][c], dc = s_stat[3][c];
    af_with(p.act, [&](auto activation) {
        const int act = activation;
        auto row = [&](size_t r, float x) {
            const size_t i = base + r * p.H + j;
            float h = (x - mean) / var;
            if (p.renorm) h = h * rc + dc;
            p.hats[i] = h;
            const float y = scale * h + shift;
            p.normalizes[i] = y;
            if (p.act_out) {
                float v = af_fire(act, y);
                if (p.colscale) v *= cs;
                p.act_out[i] = v;
            }
        };
#pragma unroll
        for (int h = 0; h < kSeqHeld; ++h)
            if (rl + (size_t)h * kLanes < p.rows) row(rl + (size_t)h * kLanes, held[h]);
        for (size_t r = rl + (size_t)kSeqHeld * kLanes; r < p.rows; r += kLanes) row(r, p.x[base + r * p.H + j]);
    });
}

static int sequence_columns(size_t H, size_t T)
{
    for (int cw : {64, 16})
        if ((H + cw - 1) / cw * T >= 256) return cw;
    return 4;
}

int launch_bn_forward_sequence(hipStream_t s, const BnForwardParams &p, size_t T, size_t Bmax, int training)
{
    if (p.H == 0 || p.rows == 0 || T == 0) return MYEA_OK;
    if (p.rows > Bmax || T > 65535) { set_last_error("bn_forward_sequence: %zu rows of %zu, %zu time steps", p.rows, Bmax, T); return MYEA_E_INVALID; }
    // the widest column block that still gives the device a workgroup per compute unit: a launch is a chain of memory round trips,
    // shorter the more row lanes share a column
    const int cw = sequence_columns(p.H, T);
    if (cw == 4) hipLaunchKernelGGL(bn_forward_sequence_kernel<4>, dim3((unsigned)((p.H + 3) / 4), (unsigned)T), dim3(kBlock), 0, s, p, Bmax, training);
    else if (cw == 16) hipLaunchKernelGGL(bn_forward_sequence_kernel<16>, dim3((unsigned)((p.H + 15) / 16), (unsigned)T), dim3(kBlock), 0, s, p, Bmax, training);
    else hipLaunchKernelGGL(bn_forward_sequence_kernel<64>, dim3((unsigned)((p.H + 63) / 64), (unsigned)T), dim3(kBlock), 0, s, p, Bmax, training);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// The backward pass of the same, every time step in one launch: the four column sums of BnBackF in LDS, the last loop of
// bn_backward_apply_kernel behind them.  The shares of the scale's and the shift's gradient - one per time step, all onto the
// same two vectors - go to `partial` ([T][2][H]) and are added by bn_backward_sequence_final_kernel in a fixed order.
template <int CW>
__global__ __launch_bounds__(kBlock) void bn_backward_sequence_kernel(BnBackwardParams p, size_t Bmax, float *__restrict__ partial)
{
    constexpr int kLanes = kBlock / CW, NW = kBlock / 64, NP = NW * kNormPartials<CW>;
    static_assert(NW == 4, "a wavefront finishes each of the four column sums");
    __shared__ double red[4][NP][CW];
    __shared__ float s_d[2][CW];
    const int c = threadIdx.x % CW, rl = threadIdx.x / CW, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const size_t t = blockIdx.y, j = (size_t)blockIdx.x * CW + c;
    const bool live = j < p.H;
    const size_t base = t * Bmax * p.H, sj = t * p.H + j;
    const int fc = norm_finish_column<CW>(lane);
    const size_t fj = (size_t)blockIdx.x * CW + fc;
    const bool keeper = norm_finish_keeper<CW>(lane) && fj < p.H;
    float vb = 1.f, rc = 1.f, mean = 0.f, scale = 0.f;
    float held_dy[kSeqHeld], held_x[kSeqHeld], held_hat[kSeqHeld];
#pragma unroll
    for (int h = 0; h < kSeqHeld; ++h) { held_dy[h] = 0.f; held_x[h] = 0.f; held_hat[h] = 0.f; }
    if (live) {
#pragma unroll
        for (int h = 0; h < kSeqHeld; ++h) {
            const size_t r = rl + (size_t)h * kLanes;
            if (r < p.rows) { const size_t k = base + r * p.H + j; held_dy[h] = p.dy[k]; held_hat[h] = p.hats[k]; held_x[h] = p.x[k]; }
        }
        vb = p.var[sj]; rc = p.renorm ? p.r_corr[sj] : 1.f; mean = p.mean[sj]; scale = p.scale[j];
    }
    double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
    if (live) {
        auto row = [&](float e, float hat, float x) {
            a0 += e * hat;
            a1 += e;
            e *= scale;
            a2 += e * (-rc / vb);
            a3 += e * (x - mean) * (-rc / (vb * vb));
        };
#pragma unroll
        for (int h = 0; h < kSeqHeld; ++h)
            if (rl + (size_t)h * kLanes < p.rows) row(held_dy[h], held_hat[h], held_x[h]);
        for (size_t r = rl + (size_t)kSeqHeld * kLanes; r < p.rows; r += kLanes) {
            const size_t k = base + r * p.H + j;
            row(p.dy[k], p.hats[k], p.x[k]);
        }
    }
    a0 = norm_fold_partial<CW>(a0); a1 = norm_fold_partial<CW>(a1); a2 = norm_fold_partial<CW>(a2); a3 = norm_fold_partial<CW>(a3);
    if (norm_partial_holder<CW>(lane)) {
        const int slot = norm_partial_index<CW>(wave, lane);
        red[0][slot][c] = a0; red[1][slot][c] = a1; red[2][slot][c] = a2; red[3][slot][c] = a3;
    }
    __syncthreads();
    {   // wavefront q finishes sum q: the scale's and the shift's shares of this time step go out, the two others to the second pass
        const double total = norm_sum_partials<CW, NP>(red[wave], lane);
        if (keeper) {
            if (wave < 2) partial[(t * 2 + wave) * p.H + fj] = (float)total;
            else s_d[wave - 2][fc] = (float)total;
        }
    }
    __syncthreads();
    if (!live) return;
    const float dmean = s_d[0][c], dvar = s_d[1][c];
    const float bsz = (float)p.rows, bscale = 1.f / (float)p.rows;
    auto apply = [&](size_t r, float dy, float x) {
        float e = dy * scale;
        e *= rc / vb;
        e += dvar * ((x - mean) / (bsz * vb));
        e += dmean * bscale;
        p.dx[base + r * p.H + j] = e;
    };
#pragma unroll
    for (int h = 0; h < kSeqHeld; ++h)
        if (rl + (size_t)h * kLanes < p.rows) apply(rl + (size_t)h * kLanes, held_dy[h], held_x[h]);
    for (size_t r = rl + (size_t)kSeqHeld * kLanes; r < p.rows; r += kLanes) {
        const size_t i = base + r * p.H + j;
        apply(r, p.dy[i], p.x[i]);
    }
}

// grid: ceil(H / 64); four lanes per column (lane q: time steps T-1-q, T-5-q, ...), their sums added in lane order onto the gradient
__global__ __launch_bounds__(kBlock) void bn_backward_sequence_final_kernel(size_t H, size_t T, const float *__restrict__ partial, float *dscale, float *dshift)
{
    __shared__ float red[2][kBlock / 64][64];
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6;
    const size_t j = (size_t)blockIdx.x * 64 + cl;
    float a = 0.f, b = 0.f;
    if (j < H) {
#pragma unroll 8
        for (size_t k = q; k < T; k += kBlock / 64) {
            const size_t t = T - 1 - k;
            a += partial[(t * 2 + 0) * H + j]; b += partial[(t * 2 + 1) * H + j];
        }
    }
    red[0][q][cl] = a; red[1][q][cl] = b;
    __syncthreads();
    if (q != 0 || j >= H) return;
#pragma unroll
    for (int r = 1; r < kBlock / 64; ++r) { a += red[0][r][cl]; b += red[1][r][cl]; }
    dscale[j] += a; dshift[j] += b;
}

// the same for one layer of a table of them: grid (ceil(widest H / 64), layers)
__global__ __launch_bounds__(kBlock) void bn_share_fold_kernel(const BnFoldJob *__restrict__ jobs)
{
    __shared__ float red[2][kBlock / 64][64];
    const BnFoldJob job = jobs[blockIdx.y];
    if ((size_t)blockIdx.x * 64 >= job.H) return;
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6;
    const size_t j = (size_t)blockIdx.x * 64 + cl, H = job.H, T = job.T;
    float a = 0.f, b = 0.f;
    if (j < H) {
#pragma unroll 8
        for (size_t k = q; k < T; k += kBlock / 64) {
            const size_t t = T - 1 - k;
            a += job.shares[(t * 2 + 0) * H + j]; b += job.shares[(t * 2 + 1) * H + j];
        }
    }
    red[0][q][cl] = a; red[1][q][cl] = b;
    __syncthreads();
    if (q != 0 || j >= H) return;
#pragma unroll
    for (int r = 1; r < kBlock / 64; ++r) { a += red[0][r][cl]; b += red[1][r][cl]; }
    job.dscale[j] += a; job.dshift[j] += b;
}

int launch_bn_share_folds(hipStream_t s, const BnFoldJob *jobs, size_t count, size_t widest)
{
    if (count == 0 || widest == 0) return MYEA_OK;
    if (count > 65535) { set_last_error("bn_share_folds: %zu layers in one launch", count); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(bn_share_fold_kernel, dim3(grid_for(widest, 64), (unsigned)count), dim3(kBlock), 0, s, jobs);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_bn_backward_sequence(hipStream_t s, const BnBackwardParams &p, size_t T, size_t Bmax, float *scratch, bool fold_now)
{
    if (p.H == 0 || p.rows == 0 || T == 0) return MYEA_OK;
    if (p.rows > Bmax || T > 65535) { set_last_error("bn_backward_sequence: %zu rows of %zu, %zu time steps", p.rows, Bmax, T); return MYEA_E_INVALID; }
    const int cw = sequence_columns(p.H, T);
    const size_t blocks = (p.H + cw - 1) / cw;
    if (cw == 4) hipLaunchKernelGGL(bn_backward_sequence_kernel<4>, dim3((unsigned)blocks, (unsigned)T), dim3(kBlock), 0, s, p, Bmax, scratch);
    else if (cw == 16) hipLaunchKernelGGL(bn_backward_sequence_kernel<16>, dim3((unsigned)blocks, (unsigned)T), dim3(kBlock), 0, s, p, Bmax, scratch);
    else hipLaunchKernelGGL(bn_backward_sequence_kernel<64>, dim3((unsigned)blocks, (unsigned)T), dim3(kBlock), 0, s, p, Bmax, scratch);
    MYEA_HIP_TRY(hipGetLastError());
    // (the shares are added by a launch of their own: a column block's last workgroup could add them itself, but the release of its
    // stores to the other XCDs' workgroups costs more than the launch - 38 against 9 + 8 us measured)
    if (!fold_now) return MYEA_OK;
    hipLaunchKernelGGL(bn_backward_sequence_final_kernel, dim3(grid_for(p.H, 64)), dim3(kBlock), 0, s, p.H, T, scratch, p.dscale, p.dshift);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_bn_forward_inference(hipStream_t s, size_t rows, size_t H, const float *x, const float *scale, const float *shift,
                                const float *mean_avg, const float *var_avg, float *normalizes)
{
    const size_t n = rows * H;
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(bn_forward_inference_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, n, H, x, scale, shift, mean_avg, var_avg, normalizes);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_bn_backward(hipStream_t s, const BnBackwardParams &p, float *scratch)
{
    if (p.H == 0 || p.rows == 0) return MYEA_OK;
    size_t S, chunk;
    split_rows(p.rows, p.H, S, chunk);
    BnBackF f{p};
    float *dmean_dvar = scratch;            // 2 * H
    float *partial = scratch + 2 * p.H;     // S * 4 * H
    hipLaunchKernelGGL((column_partial_kernel<4, BnBackF>), dim3((unsigned)((p.H + 63) / 64), (unsigned)S), dim3(kBlock), 0, s, p.rows, p.H, chunk, partial, f);
    MYEA_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(bn_backward_final_kernel, dim3(grid_for(p.H, kBlock)), dim3(kBlock), 0, s, p.H, S, partial, p.dscale, p.dshift, dmean_dvar);
    MYEA_HIP_TRY(hipGetLastError());
    const size_t n = p.rows * p.H;
    hipLaunchKernelGGL(bn_backward_apply_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, n, p, dmean_dvar);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_compute_error(hipStream_t s, const ErrorParams &p)
{
    if (p.T <= p.first_t || p.B == 0 || p.H == 0) return MYEA_OK;
    const size_t nrows = (p.T - p.first_t) * p.B;
    auto aligned = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const bool vec = (p.H & 3) == 0 && aligned(p.values) && aligned(p.desired) && aligned(p.pre) && aligned(p.errors);
    // 2048 workgroups: fewer leave long queues of rows behind each wavefront (512: 66 us for 16 384 rows of 512 against 54),
    // more lengthen the queue of fp64 atomics every workgroup ends with (8192: 69 us, and 113 against 52 on 32 768 rows of 32)
    if (vec) hipLaunchKernelGGL(compute_error_kernel<4>, dim3(grid_for(nrows, kBlock / 64, 2048)), dim3(kBlock), 0, s, p);
    else hipLaunchKernelGGL(compute_error_kernel<1>, dim3(grid_for(nrows, kBlock / 64, 1024)), dim3(kBlock), 0, s, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_accuracy_r(hipStream_t s, const ErrorParams &p, float desired_mean, float predicted_mean)
{
    if (p.T <= p.first_t || p.B == 0 || p.H == 0) return MYEA_OK;
    const size_t nrows = (p.T - p.first_t) * p.B;
    hipLaunchKernelGGL(accuracy_r_kernel, dim3(grid_for(nrows, kBlock / 64, 1024)), dim3(kBlock), 0, s, p, desired_mean, predicted_mean);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_gather_rows(hipStream_t s, size_t B, size_t row_floats, const unsigned long long *index, const float *src, float *dst)
{
    if (B == 0 || row_floats == 0) return MYEA_OK;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(grid_for(B * row_floats / 4 + 1, kBlock, 8192)), dim3(kBlock), 0, s, B, row_floats, index, src, dst);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_scatter_time_major(hipStream_t s, size_t B, size_t T, size_t W, size_t Bmax, const float *src, float *dst)
{
    const size_t n = B * T * W;
    if (n == 0) return MYEA_OK;
    hipLaunchKernelGGL(scatter_time_major_kernel, dim3(grid_for(n, kBlock, 8192)), dim3(kBlock), 0, s, B, T, W, Bmax, src, dst);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_sum_squares(hipStream_t s, size_t n, const float *g, float *partials, float *out_sum)
{
    const unsigned nparts = grid_for(n / 4 + 1, kBlock, 1024);
    hipLaunchKernelGGL(sum_squares_partial_kernel, dim3(nparts), dim3(kBlock), 0, s, n, g, partials);
    MYEA_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(sum_squares_final_kernel, dim3(1), dim3(kBlock), 0, s, nparts, partials, out_sum);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// Forward_Pass__Average_Pooling / __Max_Pooling (NN/Neural_Network__Forward_Pass__Loop.cpp:4537-4583, 5070-5135).  Window positions
// are padded coordinates p = j stride + k dilation; the input occupies [padding, padding + In).  Average: padding adds 0, the
// divisor is always the kernel size.  Max: a padded position stands for 0; the first maximum's position is kept.
__global__ __launch_bounds__(kBlock) void pool_forward_kernel(PoolParams p, const float *__restrict__ x, float *__restrict__ y, unsigned *__restrict__ index)
{
    const size_t n = p.rows * p.H;
    const float scale = 1.f / (float)p.kernel;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const size_t r = i / p.H, j = i - r * p.H;
        const float *xr = x + r * p.In;
        if (!p.is_max) {
            float s = 0.f;
            for (unsigned k = 0; k < p.kernel; ++k) {
                const size_t pos = j * p.stride + (size_t)k * p.dilation;
                if (pos < p.padding || pos >= p.In + p.padding) continue;
                s += xr[pos - p.padding];
            }
            y[i] = s * scale;
        } else {
            size_t at = 0; float mx = -3.402823466e+38f;
            for (unsigned k = 0; k < p.kernel; ++k) {
                const size_t pos = j * p.stride + (size_t)k * p.dilation;
                if (pos < p.padding || pos >= p.In + p.padding) { if (mx < 0.f) { at = pos; mx = 0.f; } }
                else { const float v = xr[pos - p.padding]; if (mx < v) { at = pos; mx = v; } }
            }
            index[i] = (unsigned)at;
            y[i] = mx;
        }
    }
}

// Backward_Pass__Average_Pooling / __Max_Pooling (NN/Neural_Network__Backward_Pass__Loop.cpp:1004-1049, 1139-1181) as a gather: an input
// position collects from the windows that contain it, in ascending window order (the order the reference's scatter adds them).
__global__ __launch_bounds__(kBlock) void pool_backward_kernel(PoolParams p, const float *__restrict__ dy, const unsigned *__restrict__ index, float *__restrict__ dx)
{
    const size_t n = p.rows * p.In;
    const float scale = 1.f / (float)p.kernel;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const size_t r = i / p.In, c = i - r * p.In;
        const size_t pos = c + p.padding;
        float v = 0.f;
        for (unsigned kk = p.kernel; kk-- > 0;) {
            const size_t off = (size_t)kk * p.dilation;
            if (off > pos) continue;
            if (p.is_max && p.dilation == 0 && kk != 0) continue;   // every tap of such a window is the one position: its window hands down once
            const size_t q = pos - off;
            if (q % p.stride) continue;
            const size_t j = q / p.stride;
            if (j >= p.H) continue;
            if (!p.is_max) v += dy[r * p.H + j] * scale;
            else if (index[r * p.H + j] == (unsigned)pos) v += dy[r * p.H + j];
        }
        dx[i] = v;
    }
}

int launch_pool_forward(hipStream_t s, const PoolParams &p, const float *x, float *y, unsigned *index)
{
    if (p.rows == 0 || p.H == 0) return MYEA_OK;
    if (p.kernel == 0 || p.stride == 0 || !x || !y || (p.is_max && !index)) { set_last_error("pooling forward: bad parameters"); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(pool_forward_kernel, dim3(grid_for(p.rows * p.H, kBlock, 8192)), dim3(kBlock), 0, s, p, x, y, index);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_pool_backward(hipStream_t s, const PoolParams &p, const float *dy, const unsigned *index, float *dx)
{
    if (p.rows == 0 || p.In == 0) return MYEA_OK;
    if (p.kernel == 0 || p.stride == 0 || !dy || !dx || (p.is_max && !index)) { set_last_error("pooling backward: bad parameters"); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(pool_backward_kernel, dim3(grid_for(p.rows * p.In, kBlock, 8192)), dim3(kBlock), 0, s, p, dy, index, dx);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// dst[i] += slab 0 [i] + slab 1 [i] + ... (in slab order): the second half of a deterministic split-K contraction
__global__ __launch_bounds__(kBlock) void slab_sum_add_kernel(size_t n, int nslab, const float *__restrict__ slabs, float *__restrict__ dst)
{
    const size_t n4 = n / 4;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += (size_t)gridDim.x * kBlock) {
        f32x4 v = reinterpret_cast<const f32x4 *>(slabs)[i];
#pragma unroll 8
        for (int s = 1; s < nslab; ++s) {
            const f32x4 w = reinterpret_cast<const f32x4 *>(slabs + (size_t)s * n)[i];
            v[0] += w[0]; v[1] += w[1]; v[2] += w[2]; v[3] += w[3];
        }
        f32x4 d = reinterpret_cast<f32x4 *>(dst)[i];
        d[0] += v[0]; d[1] += v[1]; d[2] += v[2]; d[3] += v[3];
        reinterpret_cast<f32x4 *>(dst)[i] = d;
    }
}

// the same value by value, for slices that are no aligned multiple of four floats; 64 values a workgroup, four lanes per value
// (lane q: slabs q, q + 4, ...), their sums added in lane order: few values and many slabs make the launch a chain of loads,
// shorter the more lanes share a value
__global__ __launch_bounds__(kBlock) void slab_sum_add_scalar_kernel(size_t n, int nslab, const float *__restrict__ slabs, float *__restrict__ dst)
{
    __shared__ float red[kBlock / 64][64];
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6;
    const size_t i = (size_t)blockIdx.x * 64 + cl;
    float v = 0.f;
    if (i < n) {
#pragma unroll 8
        for (int s = q; s < nslab; s += kBlock / 64) v += slabs[(size_t)s * n + i];
    }
    red[q][cl] = v;
    __syncthreads();
    if (q != 0 || i >= n) return;
#pragma unroll
    for (int r = 1; r < kBlock / 64; ++r) v += red[r][cl];
    dst[i] += v;
}

// grid (ceil(widest n / 64), jobs)
__global__ __launch_bounds__(kBlock) void slab_fold_jobs_kernel(const SlabFoldJob *__restrict__ jobs)
{
    __shared__ float red[kBlock / 64][64];
    const SlabFoldJob job = jobs[blockIdx.y];
    if ((size_t)blockIdx.x * 64 >= job.n) return;
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6;
    const size_t i = (size_t)blockIdx.x * 64 + cl, n = job.n;
    float v = 0.f;
    if (i < n) {
#pragma unroll 8
        for (unsigned s = q; s < job.nslab; s += kBlock / 64) v += job.slabs[(size_t)s * n + i];
    }
    red[q][cl] = v;
    __syncthreads();
    if (q != 0 || i >= n) return;
#pragma unroll
    for (int r = 1; r < kBlock / 64; ++r) v += red[r][cl];
    job.dst[i] += v;
}

int launch_slab_fold_jobs(hipStream_t s, const SlabFoldJob *jobs, size_t count, size_t widest)
{
    if (count == 0 || widest == 0) return MYEA_OK;
    if (count > 65535) { set_last_error("slab_fold_jobs: %zu sums in one launch", count); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(slab_fold_jobs_kernel, dim3(grid_for(widest, 64), (unsigned)count), dim3(kBlock), 0, s, jobs);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// value_by_value: the value-by-value form (and its order of additions) whatever the alignment
int launch_slab_sum_add(hipStream_t s, size_t n, int nslab, const float *slabs, float *dst, bool value_by_value)
{
    if (n == 0 || nslab <= 0) return MYEA_OK;
    if (value_by_value || (n & 3) || (reinterpret_cast<uintptr_t>(slabs) & 15u) || (reinterpret_cast<uintptr_t>(dst) & 15u))
        hipLaunchKernelGGL(slab_sum_add_scalar_kernel, dim3(grid_for(n, 64)), dim3(kBlock), 0, s, n, nslab, slabs, dst);
    else
        hipLaunchKernelGGL(slab_sum_add_kernel, dim3(grid_for(n / 4, kBlock, 8192)), dim3(kBlock), 0, s, n, nslab, slabs, dst);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_max_norm(hipStream_t s, size_t nseg, const unsigned long long *first, const unsigned *len, unsigned longest, float max_norm, float *w)
{
    if (nseg == 0) return MYEA_OK;
    if (!first || !len || !w) { set_last_error("max-norm: null segment table"); return MYEA_E_INVALID; }
    if (longest > 1024) hipLaunchKernelGGL((max_norm_kernel<kBlock>), dim3(grid_for(nseg, 1, 0x7fffffffu)), dim3(kBlock), 0, s, nseg, first, len, max_norm, w);
    else hipLaunchKernelGGL((max_norm_kernel<64>), dim3(grid_for(nseg, kBlock / 64, 0x7fffffffu)), dim3(kBlock), 0, s, nseg, first, len, max_norm, w);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_update(hipStream_t s, const UpdateParams &p)
{
    if (p.n == 0 && !p.applied) return MYEA_OK;
    UpdateDev d;
    d.n = p.n; d.n_weights = p.n_weights;
    d.w = p.w; d.g = p.g; d.s0 = p.s0; d.s1 = p.s1; d.s2 = p.s2;
    d.lr = p.lr; d.mu = p.mu; d.lr_t = p.lr_t; d.beta1 = p.beta1; d.beta2 = p.beta2; d.eps = p.eps;
    d.lower = p.lower; d.upper = p.upper; d.wd = p.wd;
    d.norm_sq = p.norm_sq; d.clip = p.clip; d.grad_scale = p.grad_scale;
    d.fault = p.fault; d.applied = p.applied;
    const bool wd = p.wd != 0.f;
    auto need = [&](float *ptr, const char *name) { if (!ptr) { set_last_error("optimizer update: %s state is null", name); return false; } return true; };
    // the vector path needs 16-byte aligned bases
    auto al = [](const void *q) { return q == nullptr || (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (!al(p.w) || !al(p.g) || !al(p.s0) || !al(p.s1) || !al(p.s2)) { set_last_error("optimizer update: vectors must be 16-byte aligned"); return MYEA_E_INVALID; }
    switch (p.optimizer) {
    case MYEA_OPTIMIZER_GD:
        if (p.variant == 0) return launch_update_kind<0>(s, d, wd);
        if (!need(p.s0, "previous delta")) return MYEA_E_INVALID;
        return p.variant == 1 ? launch_update_kind<1>(s, d, wd) : launch_update_kind<2>(s, d, wd);
    case MYEA_OPTIMIZER_ADAM:
        if (!need(p.s0, "first moment") || !need(p.s1, "second moment")) return MYEA_E_INVALID;
        return launch_update_kind<3>(s, d, wd);
    case MYEA_OPTIMIZER_AMSGRAD:
        if (!need(p.s0, "first moment") || !need(p.s1, "second moment") || !need(p.s2, "second moment hat")) return MYEA_E_INVALID;
        return launch_update_kind<4>(s, d, wd);
    case MYEA_OPTIMIZER_ADABOUND:
        if (!need(p.s0, "first moment") || !need(p.s1, "second moment")) return MYEA_E_INVALID;
        return launch_update_kind<5>(s, d, wd);
    case MYEA_OPTIMIZER_AMSBOUND:
        if (!need(p.s0, "first moment") || !need(p.s1, "second moment") || !need(p.s2, "second moment hat")) return MYEA_E_INVALID;
        return launch_update_kind<6>(s, d, wd);
    case MYEA_OPTIMIZER_NOSADAM:
        if (!need(p.s0, "first moment") || !need(p.s1, "second moment")) return MYEA_E_INVALID;
        return launch_update_kind<3>(s, d, wd);
    case MYEA_OPTIMIZER_IRPROP_PLUS:
        if (!need(p.s0, "previous delta") || !need(p.s1, "previous steps") || !need(p.s2, "previous slopes")) return MYEA_E_INVALID;
        return launch_update_kind<7>(s, d, false);
    case MYEA_OPTIMIZER_IRPROP_MINUS:
        if (!need(p.s1, "previous steps") || !need(p.s2, "previous slopes")) return MYEA_E_INVALID;
        return launch_update_kind<8>(s, d, false);
    default:
        set_last_error("optimizer %d is not on this path", p.optimizer);
        return MYEA_E_UNSUPPORTED;
    }
}

}  // namespace myea
