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

// xv: NC columns (D = 64 NV elements each) held by one wavefront.  h = (x - mean) * rstd (mean 0
// for the RMS form, avg == 0), y = h * w + b when there is a gain / bias pair, else h; rstd per
// column in r.  The columns are independent and their reductions are written side by side: a
// shuffle takes about a hundred cycles to come back, and twelve of them in a row per column
// would otherwise be the whole cost of normalising a few columns.
template <int NV, int NC>
__device__ __forceinline__ void norm_columns_reg(const float (&xv)[NC][NV], const float (&wv)[NV], const float (&bv)[NV],
                                                 bool has_w, float eps, int avg, float (&h)[NC][NV], float (&y)[NC][NV],
                                                 float (&r)[NC])
{
    constexpr int D = 64 * NV;
    float s[NC], mean[NC], q[NC];
#pragma unroll
    for (int c = 0; c < NC; c++) {
        s[c] = 0.0f;
#pragma unroll
        for (int v = 0; v < NV; v++) s[c] += xv[c][v];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
#pragma unroll
        for (int c = 0; c < NC; c++) s[c] += __shfl_xor(s[c], o, 64);
#pragma unroll
    for (int c = 0; c < NC; c++) {
        mean[c] = avg ? s[c] / (float)D : 0.0f;
        q[c] = 0.0f;
#pragma unroll
        for (int v = 0; v < NV; v++) { float t = xv[c][v] - mean[c]; q[c] += t * t; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
#pragma unroll
        for (int c = 0; c < NC; c++) q[c] += __shfl_xor(q[c], o, 64);
#pragma unroll
    for (int c = 0; c < NC; c++) {
        r[c] = 1.0f / sqrtf(q[c] / (float)D + eps);
#pragma unroll
        for (int v = 0; v < NV; v++) {
            h[c][v] = (xv[c][v] - mean[c]) * r[c];
            y[c][v] = has_w ? h[c][v] * wv[v] + bv[v] : h[c][v];
        }
    }
}

// one column (the norm kernel's form)
template <int NV>
__device__ __forceinline__ float norm_column_reg(const float (&xv)[NV], const float (&wv)[NV], const float (&bv)[NV],
                                                 bool has_w, float eps, int avg, float (&h)[NV], float (&y)[NV])
{
    float r[1];
    norm_columns_reg<NV, 1>(reinterpret_cast<const float (&)[1][NV]>(xv), wv, bv, has_w, eps, avg,
                            reinterpret_cast<float (&)[1][NV]>(h), reinterpret_cast<float (&)[1][NV]>(y), r);
    return r[0];
}

#endif
