// The arithmetic of one normalised column held by one wavefront, lane l owning elements
// l + 64 v: shared by the norm kernel and by product kernels that normalise their operand
// on the way in, so that both write the same bits.
#ifndef K_NORM_INLINE_H
#define K_NORM_INLINE_H

#include <hip/hip_runtime.h>

__device__ __forceinline__ float norm_wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

// xv: the column (D = 64 NV elements).  h = (x - mean) * rstd (mean 0 for the RMS form,
// avg == 0), y = h * w + b when there is a gain / bias pair, else h.  Returns rstd.
template <int NV>
__device__ __forceinline__ float norm_column_reg(const float (&xv)[NV], const float (&wv)[NV], const float (&bv)[NV],
                                                 bool has_w, float eps, int avg, float (&h)[NV], float (&y)[NV])
{
    constexpr int D = 64 * NV;
    float s = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; v++) s += xv[v];
    const float mean = avg ? norm_wave_sum(s) / (float)D : 0.0f;
    float q = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; v++) { float t = xv[v] - mean; q += t * t; }
    const float r = 1.0f / sqrtf(norm_wave_sum(q) / (float)D + eps);
#pragma unroll
    for (int v = 0; v < NV; v++) {
        h[v] = (xv[v] - mean) * r;
        y[v] = has_w ? h[v] * wv[v] + bv[v] : h[v];
    }
    return r;
}

#endif
