// The tanh-form GELU and its derivative, shared by every kernel that applies them (product
// epilogues, the few-column products, the element-wise kernels), so that all kernels of one
// arithmetic mode produce the same bits.  Two forms:
//  * nchip_gelu / nchip_gelu_grad: tanh from the math library - the fp32 path, whose results
//    are held to 1e-5 of the checker's over several optimiser steps;
//  * nchip_gelu_fast / nchip_gelu_grad_fast: tanh from one hardware exponential and one
//    hardware reciprocal,
//      tanh(u) = sign(u) (1 - e) / (1 + e),   e = 2^(-2 log2(e) |u|),
//    a dozen instructions against the library routine's fifty - the bf16-operand products,
//    where these run after the last MFMA with nothing to hide behind (the 2048 x 2048 x 512
//    products of a feed-forward block spent 10 of 25 microseconds there).  Absolute error of
//    tanh <= 1.5e-7: far inside what rounding the operands to bf16 leaves.
#ifndef NCHIP_K_ACT_H
#define NCHIP_K_ACT_H

#include <math.h>

__device__ __forceinline__ float nchip_tanh(float u)
{
    const float a = fabsf(u);
#if defined(__HIP_DEVICE_COMPILE__)
    const float e = __builtin_amdgcn_exp2f(-2.8853900817779268f * a); // v_exp_f32
    const float t = (1.0f - e) * __builtin_amdgcn_rcpf(1.0f + e);     // v_rcp_f32
#else
    const float e = exp2f(-2.8853900817779268f * a);
    const float t = (1.0f - e) * (1.0f / (1.0f + e));
#endif
    return copysignf(t, u);
}

__device__ __forceinline__ float nchip_gelu(float x)
{
    const float c0 = 0.7978845608f, c1 = 0.044715f;
    return 0.5f * x * (1.0f + tanhf(c0 * (x + c1 * x * x * x)));
}

__device__ __forceinline__ float nchip_gelu_grad(float x)
{
    const float c0 = 0.7978845608f, c1 = 0.044715f;
    const float t = tanhf(c0 * (x + c1 * x * x * x));
    return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * c0 * (1.0f + 3.0f * c1 * x * x);
}

__device__ __forceinline__ float nchip_gelu_fast(float x)
{
    const float c0 = 0.7978845608f, c1 = 0.044715f;
    return 0.5f * x * (1.0f + nchip_tanh(c0 * (x + c1 * x * x * x)));
}

__device__ __forceinline__ float nchip_gelu_grad_fast(float x)
{
    const float c0 = 0.7978845608f, c1 = 0.044715f;
    const float t = nchip_tanh(c0 * (x + c1 * x * x * x));
    return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * c0 * (1.0f + 3.0f * c1 * x * x);
}

#endif
