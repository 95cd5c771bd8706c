// Coder-side probability path: logits -> softmax -> 16-bit integer CDF, and the
// cumulative-frequency search a decoder performs.  The result must be
// bit-identical to the CPU checker, so the only floating-point steps are
// IEEE-exact ones (max, subtract, one multiply, fmaf chains, round-to-even,
// exponent-field scaling, float->uint truncation); every sum is an integer sum.
// This file is compiled with -ffp-contract=off.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/nchip_kernels.h"

namespace {

constexpr int TPB = 256;

// same operation sequence as nc_exp_det in the CPU checker (x <= 0)
__device__ __forceinline__ float exp_det(float x)
{
    const float log2e = 0x1.715476p+0f;
    const float ln2_hi = 0x1.63p-1f;
    const float ln2_lo = -0x1.bd0106p-13f;
    float n = rintf(x * log2e);
    float r = fmaf(-n, ln2_hi, x);
    r = fmaf(-n, ln2_lo, r);
    float p = 0x1.6c16c2p-10f;
    p = fmaf(p, r, 0x1.111112p-7f);
    p = fmaf(p, r, 0x1.555556p-5f);
    p = fmaf(p, r, 0x1.555556p-3f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    unsigned int u = __float_as_uint(p);
    u += (unsigned int)((int)n * (1 << 23));
    return __uint_as_float(u);
}

__device__ __forceinline__ unsigned int quant(float x, float mx)
{
    float d = x - mx;
    d = d < -30.0f ? -30.0f : d;
    return (unsigned int)(exp_det(d) * 16777216.0f);
}

// one block per column; thread t owns the contiguous chunk [t*per, (t+1)*per)
__global__ __launch_bounds__(TPB) void softmax_cdf16_kernel(const float *logits, uint16_t *cdf, int v)
{
    __shared__ float smax[TPB];
    __shared__ unsigned long long ssum[TPB];
    __shared__ unsigned long long stot;
    const float *x = logits + (int64_t)blockIdx.x * v;
    uint16_t *out = cdf + (int64_t)blockIdx.x * v;
    int t = threadIdx.x;

    float mx = -INFINITY;
    for (int i = t; i < v; i += TPB) mx = fmaxf(mx, x[i]);
    smax[t] = mx;
    __syncthreads();
    for (int s = TPB / 2; s > 0; s >>= 1) {
        if (t < s) smax[t] = fmaxf(smax[t], smax[t + s]);
        __syncthreads();
    }
    mx = smax[0];

    int per = (v + TPB - 1) / TPB;
    int i0 = t * per, i1 = min(v, i0 + per);
    unsigned long long local = 0;
    for (int i = i0; i < i1; i++) local += quant(x[i], mx);
    ssum[t] = local;
    __syncthreads();
    // exclusive scan of the 256 chunk totals (integers: order is irrelevant)
    if (t == 0) {
        unsigned long long run = 0;
        for (int k = 0; k < TPB; k++) {
            unsigned long long c = ssum[k];
            ssum[k] = run;
            run += c;
        }
        stot = run;
    }
    __syncthreads();
    unsigned long long tot = stot, run = ssum[t];
    unsigned long long scale = (unsigned long long)(65536 - v);
    for (int i = i0; i < i1; i++) {
        out[i] = (uint16_t)(run * scale / tot + (unsigned long long)i);
        run += quant(x[i], mx);
    }
}

__global__ __launch_bounds__(TPB) void cdf_lookup_kernel(const uint16_t *cdf, const uint16_t *target,
                                                         uint16_t *sym, int v, int64_t m, int use_lds)
{
    __shared__ uint16_t sc[16384];
    const uint16_t *c = cdf + (int64_t)blockIdx.y * v;
    if (use_lds) {
        for (int i = threadIdx.x; i < v; i += TPB) sc[i] = c[i];
        __syncthreads();
    }
    const uint16_t *tp = target + (int64_t)blockIdx.y * m;
    uint16_t *sp = sym + (int64_t)blockIdx.y * m;
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < m; i += (int64_t)gridDim.x * TPB) {
        unsigned int tv = tp[i];
        int lo = 0, hi = v; // cdf[lo] <= tv < cdf[hi], with cdf[v] = 65536
        while (hi - lo > 1) {
            int mid = (lo + hi) >> 1;
            unsigned int cv = use_lds ? sc[mid] : c[mid];
            if (cv <= tv) lo = mid; else hi = mid;
        }
        sp[i] = (uint16_t)lo;
    }
}

} // namespace

extern "C" int nchip_softmax_cdf16(void *stream, const float *logits, uint16_t *cdf, int v, int64_t n)
{
    if (n <= 0) return 0;
    if (v < 1 || v > 65535) { fprintf(stderr, "nchip_softmax_cdf16: vocabulary %d outside [1, 65535]\n", v); return -1; }
    hipLaunchKernelGGL(softmax_cdf16_kernel, dim3((unsigned)n), dim3(TPB), 0, (hipStream_t)stream, logits, cdf, v);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { fprintf(stderr, "nchip_softmax_cdf16: %s\n", hipGetErrorString(e)); return -2; }
    return 0;
}

extern "C" int nchip_cdf_lookup(void *stream, const uint16_t *cdf, const uint16_t *target,
                                uint16_t *sym, int v, int64_t m, int64_t n)
{
    if (n <= 0 || m <= 0) return 0;
    if (n > 65535) { fprintf(stderr, "nchip_cdf_lookup: too many columns\n"); return -1; }
    int64_t bx = (m + TPB * 4 - 1) / (TPB * 4);
    if (bx > 1024) bx = 1024;
    hipLaunchKernelGGL(cdf_lookup_kernel, dim3((unsigned)bx, (unsigned)n), dim3(TPB), 0, (hipStream_t)stream,
                       cdf, target, sym, v, m, v <= 16384 ? 1 : 0);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { fprintf(stderr, "nchip_cdf_lookup: %s\n", hipGetErrorString(e)); return -2; }
    return 0;
}
