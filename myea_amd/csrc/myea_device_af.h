// myea_device_af.h — activation functions and their derivatives on the device.
//
// Forward: the AF_FIRE switch of Header_Files/Neural_Network/Activation_Functions.hpp:120-184 (the
// steepness is NOT applied in the forward direction).  Derivative: Neural_Network::
// Activation_Function_Derive, Source_Files/Neural_Network/Neural_Network.cpp:3157-3201, with the *_derive
// macros of Activation_Functions.hpp:36-119.  tanh is 2/(1+exp(-2x))-1 as in the reference, and its
// derivative (like sigmoid's) is taken on the stored — possibly dropped-out — value.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/myea_hip.h"

namespace myea {

__device__ __forceinline__ float af_seg(float v1, float r1, float v2, float r2, float s) { return (((r2 - r1) * (s - v1)) / (v2 - v1)) + r1; }

__device__ __forceinline__ float af_stepwise(float v1, float v2, float v3, float v4, float v5, float v6, float r1, float r2, float r3,
                                             float r4, float r5, float r6, float mn, float mx, float s)
{
    return s < v5 ? (s < v3 ? (s < v2 ? (s < v1 ? mn : af_seg(v1, r1, v2, r2, s)) : af_seg(v2, r2, v3, r3, s))
                            : (s < v4 ? af_seg(v3, r3, v4, r4, s) : af_seg(v4, r4, v5, r5, s)))
                  : (s < v6 ? af_seg(v5, r5, v6, r6, s) : mx);
}

#define MYEA_SELU_ALPHA 1.6732632423543772848170429916717f
#define MYEA_SELU_SCALE 1.0507009873554804934193349852946f

__device__ __forceinline__ float af_fire(int type, float s)
{
    switch (type) {
    case MYEA_AF_LINEAR: return s;
    case MYEA_AF_LINEAR_PIECE: return s < 0.f ? 0.f : (s > 1.f ? 1.f : s);
    case MYEA_AF_LINEAR_PIECE_SYMMETRIC: return s < -1.f ? -1.f : (s > 1.f ? 1.f : s);
    case MYEA_AF_SIGMOID: return 1.f / (1.f + expf(-s));
    case MYEA_AF_TANH: return 2.f / (1.f + expf(-2.f * s)) - 1.f;
    case MYEA_AF_SIGMOID_STEPWISE:
        return af_stepwise(-2.64665246009826660156f, -1.47221946716308593750f, -5.49306154251098632812e-01f,
                           5.49306154251098632812e-01f, 1.47221934795379638672f, 2.64665293693542480469f,
                           4.99999988824129104614e-03f, 5.00000007450580596924e-02f, 2.5e-01f, 7.5e-01f,
                           9.49999988079071044922e-01f, 9.95000004768371582031e-01f, 0.f, 1.f, s);
    case MYEA_AF_TANH_STEPWISE:
        return af_stepwise(-2.64665293693542480469f, -1.47221934795379638672f, -5.49306154251098632812e-01f,
                           5.49306154251098632812e-01f, 1.47221934795379638672f, 2.64665293693542480469f,
                           -9.90000009536743164062e-01f, -8.99999976158142089844e-01f, -5.0e-01f, 5.0e-01f,
                           8.99999976158142089844e-01f, 9.90000009536743164062e-01f, -1.f, 1.f, s);
    case MYEA_AF_THRESHOLD: return s < 0.f ? 0.f : 1.f;
    case MYEA_AF_THRESHOLD_SYMMETRIC: return s < 0.f ? -1.f : 1.f;
    case MYEA_AF_GAUSSIAN: return expf(-s * s);
    case MYEA_AF_GAUSSIAN_SYMMETRIC: return expf(-s * s) * 2.f - 1.f;
    case MYEA_AF_GAUSSIAN_STEPWISE: return 0.f;
    case MYEA_AF_ELLIOT: return (s / 2.f) / (1.f + fabsf(s)) + 0.5f;
    case MYEA_AF_ELLIOT_SYMMETRIC: return s / (1.f + fabsf(s));
    case MYEA_AF_SINE: return sinf(s) / 2.f + 0.5f;
    case MYEA_AF_SINE_SYMMETRIC: return sinf(s);
    case MYEA_AF_COSINE: return cosf(s) / 2.f + 0.5f;
    case MYEA_AF_COSINE_SYMMETRIC: return cosf(s);
    case MYEA_AF_ISRU: return s * (1.f / sqrtf(1.f + s * s));
    case MYEA_AF_ISRLU: return s < 0.f ? s * (1.f / sqrtf(1.f + s * s)) : s;
    case MYEA_AF_ELU: return s < 0.f ? (expf(s) - 1.f) : s;
    case MYEA_AF_SELU: return MYEA_SELU_SCALE * (s <= 0.f ? MYEA_SELU_ALPHA * expf(s) - MYEA_SELU_ALPHA : s);
    case MYEA_AF_RELU: return s < 0.f ? 0.f : s;
    case MYEA_AF_LEAKY_RELU: return s < 0.f ? 0.01f * s : s;
    case MYEA_AF_PARAMETRIC_RELU: return s < 0.f ? 0.01f * s : s;
    case MYEA_AF_SOFTMAX: return expf(s);
    default: return s;
    }
}

__device__ __forceinline__ float af_derive(int type, float q, float st, float v)
{
    switch (type) {
    case MYEA_AF_COSINE: return st * -sinf(st * q) / 2.f;
    case MYEA_AF_COSINE_SYMMETRIC: return st * -sinf(st * q);
    case MYEA_AF_ELU: return q < 0.f ? st * v : st;
    case MYEA_AF_ELLIOT: return st / (2.f * (1.f + fabsf(q)) * (1.f + fabsf(q)));
    case MYEA_AF_ELLIOT_SYMMETRIC: return st / ((1.f + fabsf(q)) * (1.f + fabsf(q)));
    case MYEA_AF_GAUSSIAN: return -2.f * q * v * st * st;
    case MYEA_AF_GAUSSIAN_SYMMETRIC: return -2.f * q * (v + 1.f) * st * st;
    // pow(float, 3u) there promotes to double and the cube is rounded to float once (Activation_Functions.hpp:86, 90)
    case MYEA_AF_ISRU: { const double r = (double)(v / q); return st * (float)(r * r * r); }
    case MYEA_AF_ISRLU: { const double r = (double)(v / q); return q < 0.f ? st * (float)(r * r * r) : st; }
    case MYEA_AF_LINEAR:
    case MYEA_AF_LINEAR_PIECE:
    case MYEA_AF_LINEAR_PIECE_SYMMETRIC: return st;
    case MYEA_AF_LEAKY_RELU: return q < 0.f ? st * 0.01f : st;
    case MYEA_AF_PARAMETRIC_RELU: return q < 0.f ? st * 0.01f : st;
    case MYEA_AF_RELU: return q < 0.f ? 0.f : st;
    case MYEA_AF_SELU: return MYEA_SELU_SCALE * (q <= 0.f ? st * (v + MYEA_SELU_ALPHA) : st);
    case MYEA_AF_SIGMOID:
    case MYEA_AF_SIGMOID_STEPWISE: return st * v * (1.f - v);
    case MYEA_AF_SINE: return st * cosf(st * q) / 2.f;
    case MYEA_AF_SINE_SYMMETRIC: return st * cosf(st * q);
    case MYEA_AF_TANH:
    case MYEA_AF_TANH_STEPWISE: return st * (1.f - v * v);
    case MYEA_AF_SOFTMAX: return st;
    default: return v;
    }
}


// af_fire and af_derive take the layer's activation type as a run-time value.  Inlined into a loop body the whole switch - its
// sines, exponentials and tables - sits in that loop, and a chain unrolled over time steps carries a copy per step: the lanes
// then fetch and branch through kilobytes of code for a handful of instructions.  af_with(type, f) calls f with the type as a
// compile-time constant for the types the hot paths meet and with the run-time value for the others; inside f (a generic
// lambda that reads its argument as an int) the switch folds to its one case.
template <int TYPE> using AfConst = std::integral_constant<int, TYPE>;
template <class F>
__device__ __forceinline__ void af_with(int type, F &&f)
{
    switch (type) {
    case MYEA_AF_LINEAR: f(AfConst<MYEA_AF_LINEAR>{}); break;
    case MYEA_AF_SIGMOID: f(AfConst<MYEA_AF_SIGMOID>{}); break;
    case MYEA_AF_TANH: f(AfConst<MYEA_AF_TANH>{}); break;
    case MYEA_AF_RELU: f(AfConst<MYEA_AF_RELU>{}); break;
    case MYEA_AF_LEAKY_RELU: f(AfConst<MYEA_AF_LEAKY_RELU>{}); break;
    case MYEA_AF_ISRU: f(AfConst<MYEA_AF_ISRU>{}); break;
    case MYEA_AF_ISRLU: f(AfConst<MYEA_AF_ISRLU>{}); break;
    case MYEA_AF_ELU: f(AfConst<MYEA_AF_ELU>{}); break;
    case MYEA_AF_SELU: f(AfConst<MYEA_AF_SELU>{}); break;
    default: f(type); break;
    }
}

// Activations cheap enough to live in a contraction's epilogue (no table, at most one exp).
__device__ __forceinline__ bool af_is_fusable(int type)
{
    return type == MYEA_AF_LINEAR || type == MYEA_AF_RELU || type == MYEA_AF_LEAKY_RELU || type == MYEA_AF_PARAMETRIC_RELU ||
           type == MYEA_AF_TANH || type == MYEA_AF_SIGMOID;
}
__device__ __forceinline__ float af_fire_fused(int type, float s)
{
    if (type == MYEA_AF_TANH || type == MYEA_AF_SIGMOID) {
        const bool th = type == MYEA_AF_TANH;
        const float e = expf(th ? -2.f * s : -s);
        return th ? 2.f / (1.f + e) - 1.f : 1.f / (1.f + e);
    }
    if (type == MYEA_AF_RELU) return s < 0.f ? 0.f : s;
    if (type == MYEA_AF_LINEAR) return s;
    return s < 0.f ? 0.01f * s : s;  // leaky / parametric
}
__device__ __forceinline__ float af_derive_fused(int type, float q, float st, float v)
{
    if (type == MYEA_AF_TANH) return st * (1.f - v * v);
    if (type == MYEA_AF_SIGMOID) return st * v * (1.f - v);
    if (type == MYEA_AF_RELU) return q < 0.f ? 0.f : st;
    if (type == MYEA_AF_LINEAR) return st;
    return q < 0.f ? st * 0.01f : st;  // leaky / parametric
}

}  // namespace myea
