// Bandwidth-bound column kernels: LayerNorm/RMSNorm, softmax, log-likelihood,
// embedding gather / scatter-add, optimiser step.  One 64-lane wavefront owns
// one column (libnc axis 0) and reduces with xor-shuffles, so every lane ends
// with the same, order-fixed sum; cross-column reductions (dw, db of the norm
// affine, embedding gradient) are two-stage or sequential and use no atomics.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <mutex>
#include "../../include/nchip_kernels.h"
#include "k_norm_inline.h"
#include "k_bf16.h"

// Scratch of nchip_norm_bwd_static: the partial dw / db rows of the norm backward, held by the
// library itself so that the call allocates nothing.  In host code this name is only a
// handle for hipGetSymbolAddress: every GPU holds its own copy at its own address, looked up
// once per device (static_scratch_of_current_device) and passed to the kernels as a pointer.
constexpr size_t NORM_STATIC_SCRATCH_FLOATS = (size_t)2 << 20; // 8 MiB
static __device__ __align__(256) float scratch[NORM_STATIC_SCRATCH_FLOATS];

namespace {

constexpr int TPB = 256;
constexpr int WPB = TPB / 64; // wavefronts (columns) per block

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

__global__ __launch_bounds__(TPB) void norm_fwd_kernel(const float *x, const float *w, const float *b,
                                                       float *y, float *xhat, float *rstd,
                                                       int d, int64_t n, float eps, int avg, uint16_t *y16)
{
    int lane = threadIdx.x & 63;
    int64_t c = (int64_t)blockIdx.x * WPB + (threadIdx.x >> 6);
    if (c >= n) return;
    const float *xc = x + c * d;
    float s = 0.0f;
    for (int i = lane; i < d; i += 64) s += xc[i];
    float mean = avg ? wave_sum(s) / (float)d : 0.0f;
    float v = 0.0f;
    for (int i = lane; i < d; i += 64) { float t = xc[i] - mean; v += t * t; }
    float r = 1.0f / sqrtf(wave_sum(v) / (float)d + eps);
    if (lane == 0) rstd[c] = r;
    for (int i = lane; i < d; i += 64) {
        float h = (xc[i] - mean) * r;
        if (xhat) xhat[c * d + i] = h;
        const float out = w ? h * w[i] + b[i] : h;
        y[c * d + i] = out;
        if (y16) y16[c * d + i] = f32_to_bf16_rne(out);
    }
}

// d = 64*NV: the column is read once and stays in registers (the generic kernel walks it
// three times, each pass waiting for memory: with a few thousand columns that latency is
// the whole run time).  Same per-lane summation order, so the results are the same.
template <int NV>
__global__ __launch_bounds__(TPB) void norm_fwd_reg(const float *x, const float *w, const float *b,
                                                    float *y, float *xhat, float *rstd,
                                                    int64_t n, float eps, int avg, uint16_t *y16)
{
    constexpr int D = 64 * NV;
    const int lane = threadIdx.x & 63;
    const int64_t c = (int64_t)blockIdx.x * WPB + (threadIdx.x >> 6);
    if (c >= n) return;
    const float *xc = x + c * D;
    float xv[NV], wv[NV], bv[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) xv[v] = xc[lane + 64 * v];
    if (w) {
#pragma unroll
        for (int v = 0; v < NV; v++) { wv[v] = w[lane + 64 * v]; bv[v] = b[lane + 64 * v]; }
    }
    float h[NV], yv[NV];
    const float r = norm_column_reg<NV>(xv, wv, bv, w != nullptr, eps, avg, h, yv);
    if (lane == 0) rstd[c] = r;
#pragma unroll
    for (int v = 0; v < NV; v++) {
        if (xhat) xhat[c * D + lane + 64 * v] = h[v];
        y[c * D + lane + 64 * v] = yv[v];
    }
    if (y16) { // the operand copy of the products that read y
#pragma unroll
        for (int v = 0; v < NV; v++) y16[c * D + lane + 64 * v] = f32_to_bf16_rne(yv[v]);
    }
}

// dx = rstd * (gh - mean(gh) - xhat * mean(gh * xhat)),  gh = g * w
__global__ __launch_bounds__(TPB) void norm_bwd_dx_kernel(const float *g, const float *xhat,
                                                          const float *rstd, const float *w,
                                                          float *dx, const float *dx_add, int d, int64_t n, int avg,
                                                          uint16_t *dx16)
{
    int lane = threadIdx.x & 63;
    int64_t c = (int64_t)blockIdx.x * WPB + (threadIdx.x >> 6);
    if (c >= n) return;
    const float *gc = g + c * d, *hc = xhat + c * d;
    float s1 = 0.0f, s2 = 0.0f;
    for (int i = lane; i < d; i += 64) {
        float gh = w ? gc[i] * w[i] : gc[i];
        s1 += gh;
        s2 += gh * hc[i];
    }
    s1 = avg ? wave_sum(s1) / (float)d : 0.0f;
    s2 = wave_sum(s2) / (float)d;
    float r = rstd[c];
    for (int i = lane; i < d; i += 64) {
        float gh = w ? gc[i] * w[i] : gc[i];
        float v = r * (gh - s1 - hc[i] * s2);
        v = dx_add ? dx_add[c * d + i] + v : v;
        dx[c * d + i] = v;
        if (dx16) dx16[c * d + i] = f32_to_bf16_rne(v);
    }
}

// partial[s][0][i] = sum_c g*xhat, partial[s][1][i] = sum_c g over slice s of the columns
__global__ __launch_bounds__(TPB) void norm_bwd_wb_stage1(const float *g, const float *xhat,
                                                          float *partial, int d, int64_t n, int rows)
{
    int i = blockIdx.x * TPB + threadIdx.x;
    int s = blockIdx.y;
    if (i >= d) return;
    int64_t per = (n + rows - 1) / rows, c0 = s * per, c1 = c0 + per < n ? c0 + per : n;
    float aw = 0.0f, ab = 0.0f;
    for (int64_t c = c0; c < c1; c++) {
        float gv = g[c * d + i];
        aw += gv * xhat[c * d + i];
        ab += gv;
    }
    partial[((int64_t)s * 2) * d + i] = aw;
    partial[((int64_t)s * 2 + 1) * d + i] = ab;
}

// d = 64*NV: dx and the per-block dw / db partials in ONE pass over g and xhat.
// A wavefront walks cw consecutive columns keeping them in registers; its
// per-lane dw / db sums are combined over the 4 wavefronts in wavefront order
// and written as partial row blockIdx.x.
template <int NV>
__global__ __launch_bounds__(TPB) void norm_bwd_fused(const float *g, const float *xhat, const float *rstd,
                                                      const float *w, float *dx, const float *dx_add,
                                                      float *partial, int64_t n, int avg, int cw,
                                                      float *dx_partial, uint16_t *dx16)
{
    constexpr int D = NV * 64;
    __shared__ float sh[WPB - 1][3][D];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    float wr[NV], aw[NV], ab[NV], ax[NV]; // ax: row sums of the dx written (dx_partial)
#pragma unroll
    for (int v = 0; v < NV; v++) { wr[v] = w ? w[lane + 64 * v] : 1.0f; aw[v] = 0.0f; ab[v] = 0.0f; ax[v] = 0.0f; }
    const int64_t c0 = ((int64_t)blockIdx.x * WPB + wv) * cw;
    for (int k = 0; k < cw; k++) {
        const int64_t c = c0 + k;
        if (c >= n) break;
        float gv[NV], hv[NV];
#pragma unroll
        for (int v = 0; v < NV; v++) { gv[v] = g[c * D + lane + 64 * v]; hv[v] = xhat[c * D + lane + 64 * v]; }
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int v = 0; v < NV; v++) {
            float gh = gv[v] * wr[v];
            s1 += gh;
            s2 += gh * hv[v];
            aw[v] += gv[v] * hv[v];
            ab[v] += gv[v];
        }
        if (dx) {
            s1 = avg ? wave_sum(s1) / (float)D : 0.0f;
            s2 = wave_sum(s2) / (float)D;
            const float r = rstd[c];
#pragma unroll
            for (int v = 0; v < NV; v++) {
                float val = r * (gv[v] * wr[v] - s1 - hv[v] * s2);
                val = dx_add ? dx_add[c * D + lane + 64 * v] + val : val;
                dx[c * D + lane + 64 * v] = val;
                if (dx16) dx16[c * D + lane + 64 * v] = f32_to_bf16_rne(val);
                ax[v] += val;
            }
        }
    }
    if (!partial && !dx_partial) return;
    if (wv > 0) {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            sh[wv - 1][0][lane + 64 * v] = aw[v]; sh[wv - 1][1][lane + 64 * v] = ab[v]; sh[wv - 1][2][lane + 64 * v] = ax[v];
        }
    }
    __syncthreads();
    if (wv == 0) {
        if (partial) {
            float *pw = partial + (int64_t)blockIdx.x * 2 * D, *pb = pw + D;
#pragma unroll
            for (int v = 0; v < NV; v++) {
                float a = aw[v], b = ab[v];
#pragma unroll
                for (int u = 0; u < WPB - 1; u++) { a += sh[u][0][lane + 64 * v]; b += sh[u][1][lane + 64 * v]; }
                pw[lane + 64 * v] = a;
                pb[lane + 64 * v] = b;
            }
        }
        if (dx_partial) { // row blockIdx.x of the partial row sums of dx, wavefronts in order
#pragma unroll
            for (int v = 0; v < NV; v++) {
                float a = ax[v];
#pragma unroll
                for (int u = 0; u < WPB - 1; u++) a += sh[u][2][lane + 64 * v];
                dx_partial[(int64_t)blockIdx.x * D + lane + 64 * v] = a;
            }
        }
    }
}

// dw[i], db[i] = sum of the partial rows: 4 interleaved row groups per element
// (sequential inside a group), combined in group order
__global__ __launch_bounds__(TPB) void norm_bwd_wb_stage2(const float *partial, float *dw, float *db, int d, int rows)
{
    __shared__ float sh[WPB - 1][2][64];
    const int ig = threadIdx.x & 63, rg = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + ig;
    float aw = 0.0f, ab = 0.0f;
    if (i < d) {
#pragma unroll 4
        for (int s = rg; s < rows; s += WPB) {
            aw += partial[((int64_t)s * 2) * d + i];
            ab += partial[((int64_t)s * 2 + 1) * d + i];
        }
    }
    if (rg > 0) { sh[rg - 1][0][ig] = aw; sh[rg - 1][1][ig] = ab; }
    __syncthreads();
    if (rg == 0 && i < d) {
#pragma unroll
        for (int u = 0; u < WPB - 1; u++) { aw += sh[u][0][ig]; ab += sh[u][1][ig]; }
        if (dw) dw[i] = aw;
        if (db) db[i] = ab;
    }
}

__global__ __launch_bounds__(TPB) void softmax_fwd_kernel(const float *x, float *y, int v, int64_t n)
{
    int lane = threadIdx.x & 63;
    int64_t c = (int64_t)blockIdx.x * WPB + (threadIdx.x >> 6);
    if (c >= n) return;
    const float *xc = x + c * v;
    float *yc = y + c * v;
    float mx = -INFINITY;
    for (int i = lane; i < v; i += 64) mx = fmaxf(mx, xc[i]);
    mx = wave_max(mx);
    float s = 0.0f;
    for (int i = lane; i < v; i += 64) {
        float e = expf(xc[i] - mx);
        yc[i] = e;
        s += e;
    }
    float inv = 1.0f / wave_sum(s);
    for (int i = lane; i < v; i += 64) yc[i] *= inv;
}

// Long columns (a vocabulary of thousands): one workgroup per column, the column read once
// into registers (thread t holds the float4 at 4 (r TPB + t), r < R), written once.
template <int R>
__global__ __launch_bounds__(TPB) void softmax_fwd_block_kernel(const float *x, float *y, int v)
{
    __shared__ float red[2][WPB];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const float *xc = x + (int64_t)blockIdx.x * v;
    float *yc = y + (int64_t)blockIdx.x * v;
    float4 f[R];
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i0 = (r * TPB + t) * 4;
        f[r] = i0 < v ? *reinterpret_cast<const float4 *>(xc + i0) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        mx = fmaxf(fmaxf(mx, fmaxf(f[r].x, f[r].y)), fmaxf(f[r].z, f[r].w));
    }
    mx = wave_max(mx);
    if (lane == 0) red[0][wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    float s = 0.0f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        f[r].x = expf(f[r].x - mx); f[r].y = expf(f[r].y - mx);
        f[r].z = expf(f[r].z - mx); f[r].w = expf(f[r].w - mx);
        s += (f[r].x + f[r].y) + (f[r].z + f[r].w);
    }
    s = wave_sum(s);
    if (lane == 0) red[1][wave] = s;
    __syncthreads();
    const float inv = 1.0f / ((red[1][0] + red[1][1]) + (red[1][2] + red[1][3]));
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i0 = (r * TPB + t) * 4;
        if (i0 < v)
            *reinterpret_cast<float4 *>(yc + i0) = make_float4(f[r].x * inv, f[r].y * inv, f[r].z * inv, f[r].w * inv);
    }
}

__global__ __launch_bounds__(TPB) void softmax_bwd_kernel(const float *y, const float *g, float *dx,
                                                          int v, int64_t n)
{
    int lane = threadIdx.x & 63;
    int64_t c = (int64_t)blockIdx.x * WPB + (threadIdx.x >> 6);
    if (c >= n) return;
    const float *yc = y + c * v, *gc = g + c * v;
    float s = 0.0f;
    for (int i = lane; i < v; i += 64) s += gc[i] * yc[i];
    s = wave_sum(s);
    for (int i = lane; i < v; i += 64) dx[c * v + i] = yc[i] * (gc[i] - s);
}

// Indices come from the caller's data: one outside [0, v) reads nothing (the result is 0)
// and raises the flag, a word of pinned host memory that the host looks at after a wait.
__global__ void indexed_log_kernel(const float *p, const int32_t *idx, float *y, int v, int64_t n, int *bad)
{
    int64_t c = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (c >= n) return;
    const int s = idx[c];
    const bool ok = (unsigned)s < (unsigned)v;
    y[c] = ok ? logf(p[c * v + s]) : 0.0f;
    if (!ok) *bad = 1;
}

__global__ void nll_bwd_kernel(const float *p, const int32_t *idx, const float *g, float *dl,
                               int v, int64_t total, int fused)
{
    for (int64_t e = (int64_t)blockIdx.x * TPB + threadIdx.x; e < total; e += (int64_t)gridDim.x * TPB) {
        int64_t c = e / v;
        int i = (int)(e % v);
        float gc = g[c];
        float r;
        if (fused) r = gc * ((i == idx[c] ? 1.0f : 0.0f) - p[e]);
        else r = (i == idx[c]) ? gc / p[e] : 0.0f;
        dl[e] = r;
    }
}

// the same for long columns: blockIdx.x the column, blockIdx.y a run of 4 TPB rows of it
__global__ __launch_bounds__(TPB) void nll_bwd_vec_kernel(const float *p, const int32_t *idx, const float *g, float *dl,
                                                          int v, int fused)
{
    const int64_t c = blockIdx.x;
    const int i0 = ((int)blockIdx.y * TPB + (int)threadIdx.x) * 4;
    if (i0 >= v) return;
    const float gc = g[c];
    const int s = idx[c];
    const float4 pv = *reinterpret_cast<const float4 *>(p + c * v + i0);
    const float in[4] = { pv.x, pv.y, pv.z, pv.w };
    float r[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (fused) r[j] = gc * ((i0 + j == s ? 1.0f : 0.0f) - in[j]);
        else r[j] = (i0 + j == s) ? gc / in[j] : 0.0f;
    }
    *reinterpret_cast<float4 *>(dl + c * v + i0) = make_float4(r[0], r[1], r[2], r[3]);
}

__global__ void get_col_kernel(const float *w, const int32_t *idx, float *y, int d, int v, int64_t total, int *bad,
                               float scale)
{
    for (int64_t e = (int64_t)blockIdx.x * TPB + threadIdx.x; e < total; e += (int64_t)gridDim.x * TPB) {
        int64_t c = e / d;
        int i = (int)(e % d);
        const int s = idx[c];
        const bool ok = (unsigned)s < (unsigned)v;
        y[e] = ok ? w[(int64_t)s * d + i] * scale : 0.0f; // (scale 1: the value itself)
        if (!ok && i == 0) *bad = 1;
    }
}

// Embedding gradient dw[:, sym] = sum of the columns whose token is sym, added
// in increasing token order.  One block per vocabulary entry: the block first
// lists its columns in order (each thread scans a contiguous slice of the
// tokens, an exclusive prefix over the threads places its hits), then every
// thread sums its feature rows down the list, so each column of g is read once.
constexpr int ADD_COL_MAX_N = 8192; // tokens whose indices fit the LDS list

__global__ __launch_bounds__(TPB) void add_col_kernel(const float *g, const int32_t *idx, float *dw,
                                                      int d, int64_t n)
{
    __shared__ int list[ADD_COL_MAX_N];
    __shared__ int wave_hits[WPB];
    const int sym = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int per = (int)((n + TPB - 1) / TPB); // <= 32: a thread's hits fit one mask
    const int c0 = t * per, c1 = (int)(c0 + per < n ? c0 + per : n);
    unsigned int mask = 0;
    if ((per & 3) == 0 && c0 + per <= n && ((uintptr_t)idx & 15) == 0) {
        for (int q = 0; q < per; q += 4) {
            const uint4 w = *reinterpret_cast<const uint4 *>(idx + c0 + q);
            mask |= ((unsigned int)((int)w.x == sym) | (unsigned int)((int)w.y == sym) << 1 |
                     (unsigned int)((int)w.z == sym) << 2 | (unsigned int)((int)w.w == sym) << 3) << q;
        }
    } else {
        for (int c = c0; c < c1; c++) mask |= (unsigned int)(idx[c] == sym) << (c - c0);
    }
    // exclusive prefix of the threads' hit counts: by shuffles inside a wave, through LDS across the four
    const int mine = __builtin_popcount(mask);
    int incl = mine;
#pragma unroll
    for (int dd = 1; dd < 64; dd <<= 1) {
        const int o = __shfl_up(incl, dd, 64);
        if (lane >= dd) incl += o;
    }
    if (lane == 63) wave_hits[wave] = incl;
    __syncthreads();
    int pos = incl - mine, total = 0;
#pragma unroll
    for (int w = 0; w < WPB; w++) {
        if (w < wave) pos += wave_hits[w];
        total += wave_hits[w];
    }
    while (mask) {
        list[pos++] = c0 + __builtin_ctz(mask);
        mask &= mask - 1;
    }
    __syncthreads();
    // A frequent symbol's list is hundreds of tokens long and its sums (each in token order) are
    // bound by the loads in flight: eight rows are requested before the first is added.
    if ((d & 3) == 0 && (((uintptr_t)g | (uintptr_t)dw) & 15) == 0) {
        for (int i0 = 4 * t; i0 < d; i0 += 4 * TPB) {
            float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            int k = 0;
            for (; k + 8 <= total; k += 8) {
                float4 r[8];
#pragma unroll
                for (int u = 0; u < 8; u++) r[u] = *reinterpret_cast<const float4 *>(g + (int64_t)list[k + u] * d + i0);
#pragma unroll
                for (int u = 0; u < 8; u++) { acc.x += r[u].x; acc.y += r[u].y; acc.z += r[u].z; acc.w += r[u].w; }
            }
            for (; k < total; k++) {
                const float4 r = *reinterpret_cast<const float4 *>(g + (int64_t)list[k] * d + i0);
                acc.x += r.x; acc.y += r.y; acc.z += r.z; acc.w += r.w;
            }
            *reinterpret_cast<float4 *>(dw + (int64_t)sym * d + i0) = acc;
        }
        return;
    }
    for (int i = t; i < d; i += TPB) {
        float acc = 0.0f;
        int k = 0;
        for (; k + 8 <= total; k += 8) {
            float r[8];
#pragma unroll
            for (int u = 0; u < 8; u++) r[u] = g[(int64_t)list[k + u] * d + i];
#pragma unroll
            for (int u = 0; u < 8; u++) acc += r[u];
        }
        for (; k < total; k++) acc += g[(int64_t)list[k] * d + i];
        dw[(int64_t)sym * d + i] = acc;
    }
}

// any n: every block scans all tokens for every feature slice
__global__ __launch_bounds__(TPB) void add_col_scan_kernel(const float *g, const int32_t *idx, float *dw,
                                                           int d, int64_t n)
{
    int sym = blockIdx.x;
    for (int i0 = 0; i0 < d; i0 += TPB) {
        int i = i0 + threadIdx.x;
        float acc = 0.0f;
        for (int64_t c = 0; c < n; c++)
            if (idx[c] == sym && i < d)
                acc += g[c * d + i];
        if (i < d) dw[(int64_t)sym * d + i] = acc;
    }
}

__global__ void opt_update_kernel(int algo, float *w, float *m, float *v, const float *g, int64_t n,
                                  float lr, float b1, float b2, float eps, float clip, float c1, float c2)
{
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
        float gi = g[i];
        if (algo == 0) {
            w[i] -= lr * gi;
        } else if (algo == 1) {
            if (clip != 0.0f) gi = fminf(fmaxf(gi, -clip), clip);
            float mi = b1 * m[i] + (1.0f - b1) * gi;
            float vi = b2 * v[i] + (1.0f - b2) * gi * gi;
            m[i] = mi;
            v[i] = vi;
            w[i] -= lr * (mi * c1) / (sqrtf(vi * c2) + eps);
        } else {
            float vi = b2 * v[i] + (1.0f - b2) * gi * gi;
            v[i] = vi;
            w[i] -= lr * gi / (sqrtf(vi) + eps);
        }
    }
}

__device__ __forceinline__ void opt_step(int algo, float &w, float *m, float &v, float gi, float lr,
                                         float b1, float b2, float eps, float clip, float c1, float c2)
{
    if (algo == 0) {
        w -= lr * gi;
    } else if (algo == 1) {
        if (clip != 0.0f) gi = fminf(fmaxf(gi, -clip), clip);
        float mi = gi;
        if (m) { mi = b1 * *m + (1.0f - b1) * gi; *m = mi; }
        float vi = b2 * v + (1.0f - b2) * gi * gi;
        v = vi;
        w -= lr * (mi * c1) / (sqrtf(vi * c2) + eps);
    } else {
        float vi = b2 * v + (1.0f - b2) * gi * gi;
        v = vi;
        w -= lr * gi / (sqrtf(vi) + eps);
    }
}

// One launch for every parameter: block -> (tensor, chunk) through a prefix
// table of chunk counts; element-wise, so the result equals the per-tensor kernel.
__global__ __launch_bounds__(TPB) void opt_update_multi_kernel(const NchipOptTensor *tab,
                                                               const int *chunk_prefix, int n_tensors,
                                                               int chunk, int algo, float b1, float b2,
                                                               float eps, float clip, float c1, float c2)
{
    int bid = blockIdx.x, lo = 0, hi = n_tensors; // chunk_prefix[lo] <= bid < chunk_prefix[hi]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (chunk_prefix[mid] <= bid) lo = mid; else hi = mid;
    }
    NchipOptTensor t = tab[lo];
    int64_t e0 = (int64_t)(bid - chunk_prefix[lo]) * chunk;
    int64_t e1 = e0 + chunk < t.n ? e0 + chunk : t.n;
    for (int64_t i = e0 + threadIdx.x; i < e1; i += TPB) {
        float w = t.w[i], v = t.v ? t.v[i] : 0.0f;
        opt_step(algo, w, t.m ? t.m + i : nullptr, v, t.g[i], t.lr, b1, b2, eps, clip, c1, c2);
        t.w[i] = w;
        if (t.v) t.v[i] = v;
        if (t.w16) {
            const uint16_t r = f32_to_bf16_rne(w);
            t.w16[i] = r;
            if (t.wide) t.wide[i] = __builtin_bit_cast(float, (uint32_t)r << 16);
        }
    }
}

inline int grid_for(int64_t n, int cap = 8192)
{
    int64_t b = (n + TPB - 1) / TPB;
    return (int)(b > cap ? cap : (b < 1 ? 1 : b));
}

inline int check(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fprintf(stderr, "%s: launch failed: %s\n", what, hipGetErrorString(e));
        return -2;
    }
    return 0;
}

} // namespace

extern "C" {

int nchip_norm_fwd(void *stream, const float *x, const float *w, const float *b, float *y,
                   float *xhat, float *rstd, int d, int64_t n, float eps, int avg)
{
    return nchip_norm_fwd_bf16copy(stream, x, w, b, y, xhat, rstd, d, n, eps, avg, nullptr);
}

int nchip_norm_fwd_bf16copy(void *stream, const float *x, const float *w, const float *b, float *y,
                            float *xhat, float *rstd, int d, int64_t n, float eps, int avg, uint16_t *y16)
{
    if (n <= 0 || d <= 0) return 0;
    if ((w == nullptr) != (b == nullptr)) { fprintf(stderr, "nchip_norm_fwd: w and b go together\n"); return -1; }
    const dim3 grid((unsigned)((n + WPB - 1) / WPB));
#define NORM_FWD(NV) hipLaunchKernelGGL(norm_fwd_reg<NV>, grid, dim3(TPB), 0, (hipStream_t)stream, x, w, b, y, xhat, rstd, n, eps, avg, y16)
    if (d == 128) NORM_FWD(2);
    else if (d == 256) NORM_FWD(4);
    else if (d == 512) NORM_FWD(8);
    else if (d == 1024) NORM_FWD(16);
    else
        hipLaunchKernelGGL(norm_fwd_kernel, grid, dim3(TPB), 0, (hipStream_t)stream, x, w, b, y, xhat, rstd, d, n, eps, avg, y16);
#undef NORM_FWD
    return check("nchip_norm_fwd");
}

// columns per wavefront of the fused backward: 2, more when that would give
// more than 1024 partial rows
static int norm_bwd_cw(int64_t n)
{
    int64_t cw = (n + (int64_t)WPB * 1024 - 1) / ((int64_t)WPB * 1024);
    return (int)(cw < 2 ? 2 : cw);
}

int nchip_norm_bwd_partial_rows(int64_t n)
{
    int cw = norm_bwd_cw(n);
    int64_t r = (n + (int64_t)WPB * cw - 1) / ((int64_t)WPB * cw);
    return (int)(r < 32 ? 32 : r); // the generic path uses up to 32 slices
}

// exact number of partial rows nchip_norm_bwd writes for (d, n)
int nchip_norm_bwd_rows(int d, int64_t n)
{
    if (d == 128 || d == 256 || d == 512 || d == 1024) {
        const int cw = norm_bwd_cw(n);
        return (int)((n + (int64_t)WPB * cw - 1) / ((int64_t)WPB * cw));
    }
    return (int)(n / 16 > 32 ? 32 : (n / 16 < 1 ? 1 : n / 16));
}

bool nchip_norm_bwd_has_dx_rowsum(int d) { return d == 128 || d == 256 || d == 512 || d == 1024; }

int nchip_norm_bwd(void *stream, const float *g, const float *xhat, const float *rstd, const float *w,
                   float *dx, const float *dx_add, float *dw, float *db, float *partial, int d, int64_t n,
                   int avg)
{
    return nchip_norm_bwd_rowsum(stream, g, xhat, rstd, w, dx, dx_add, dw, db, partial, d, n, avg, nullptr);
}

int nchip_norm_bwd_rowsum(void *stream, const float *g, const float *xhat, const float *rstd, const float *w,
                          float *dx, const float *dx_add, float *dw, float *db, float *partial, int d, int64_t n,
                          int avg, float *dx_partial)
{
    return nchip_norm_bwd_bf16copy(stream, g, xhat, rstd, w, dx, dx_add, dw, db, partial, d, n, avg, dx_partial, nullptr);
}

int nchip_norm_bwd_bf16copy(void *stream, const float *g, const float *xhat, const float *rstd, const float *w,
                            float *dx, const float *dx_add, float *dw, float *db, float *partial, int d, int64_t n,
                            int avg, float *dx_partial, uint16_t *dx16)
{
    if (n <= 0 || d <= 0) return 0;
    if (dx16 && !dx) { fprintf(stderr, "nchip_norm_bwd_bf16copy: a copy of dx needs dx\n"); return -1; }
    if (dx_partial && (!dx || !nchip_norm_bwd_has_dx_rowsum(d))) {
        fprintf(stderr, "nchip_norm_bwd_rowsum: row sums of dx need dx and d in {128, 256, 512, 1024}\n");
        return -1;
    }
    hipStream_t st = (hipStream_t)stream;
    const bool wb = dw || db;
    if (wb && !partial) { fprintf(stderr, "nchip_norm_bwd: partial buffer missing\n"); return -1; }
    // partial given without dw / db: the partial rows are left for the caller to sum
    if (d == 128 || d == 256 || d == 512 || d == 1024) {
        const int cw = norm_bwd_cw(n);
        const int rows = nchip_norm_bwd_rows(d, n);
        float *pp = partial;
#define NORM_BWD(NV) hipLaunchKernelGGL(norm_bwd_fused<NV>, dim3(rows), dim3(TPB), 0, st, g, xhat, rstd, w, dx, dx_add, pp, n, avg, cw, dx_partial, dx16)
        if (d == 128) NORM_BWD(2); else if (d == 256) NORM_BWD(4); else if (d == 512) NORM_BWD(8); else NORM_BWD(16);
#undef NORM_BWD
        if (wb)
            hipLaunchKernelGGL(norm_bwd_wb_stage2, dim3((d + 63) / 64), dim3(TPB), 0, st,
                               (const float *)partial, dw, db, d, rows);
        return check("nchip_norm_bwd");
    }
    if (dx)
        hipLaunchKernelGGL(norm_bwd_dx_kernel, dim3((unsigned)((n + WPB - 1) / WPB)), dim3(TPB), 0, st,
                           g, xhat, rstd, w, dx, dx_add, d, n, avg, dx16);
    if (partial) {
        int rows = nchip_norm_bwd_rows(d, n);
        hipLaunchKernelGGL(norm_bwd_wb_stage1, dim3((d + TPB - 1) / TPB, rows), dim3(TPB), 0, st,
                           g, xhat, partial, d, n, rows);
        if (wb)
            hipLaunchKernelGGL(norm_bwd_wb_stage2, dim3((d + 63) / 64), dim3(TPB), 0, st,
                               (const float *)partial, dw, db, d, rows);
    }
    return check("nchip_norm_bwd");
}

size_t nchip_norm_bwd_static_capacity(void) { return NORM_STATIC_SCRATCH_FLOATS; }

// device address of `scratch` on the current device, looked up once per device
static float *static_scratch_of_current_device()
{
    constexpr int MAX_DEVICES = 64;
    static float *ptr_of[MAX_DEVICES];
    static std::mutex mu;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        fprintf(stderr, "nchip_norm_bwd_static: no current device (%s)\n", hipGetErrorString(e));
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr_of[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            fprintf(stderr, "nchip_norm_bwd_static: hipGetSymbolAddress failed on device %d: %s\n", dev,
                    hipGetErrorString(e));
            return nullptr;
        }
        ptr_of[dev] = (float *)p;
    }
    return ptr_of[dev];
}

int nchip_norm_bwd_static(void *stream, const float *g, const float *xhat, const float *rstd, const float *w,
                          float *dx, const float *dx_add, float *dw, float *db, int d, int64_t n, int avg)
{
    if (n <= 0 || d <= 0) return 0;
    const size_t need = (size_t)nchip_norm_bwd_rows(d, n) * 2 * (size_t)d;
    if (need > NORM_STATIC_SCRATCH_FLOATS) {
        fprintf(stderr, "nchip_norm_bwd_static: (d = %d, n = %lld) needs %zu floats of scratch, the library's "
                        "buffer holds %zu; use nchip_norm_bwd with a buffer of the caller\n",
                d, (long long)n, need, (size_t)NORM_STATIC_SCRATCH_FLOATS);
        return -3;
    }
    float *partial = nullptr;
    if (dw || db) { // every partial row that is summed is written first: nothing has to start at zero
        partial = static_scratch_of_current_device();
        if (!partial) return -4;
    }
    return nchip_norm_bwd(stream, g, xhat, rstd, w, dx, dx_add, dw, db, partial, d, n, avg);
}

int nchip_softmax_fwd(void *stream, const float *x, float *y, int v, int64_t n)
{
    if (n <= 0 || v <= 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = v % 4 == 0 && (((uintptr_t)x | (uintptr_t)y) & 15) == 0 && n <= 0x7fffffff;
    if (vec && v >= 2048 && v <= 16 * 4 * TPB) { // a workgroup per column, the column in registers
        const dim3 grid((unsigned)n);
        if (v <= 2 * 4 * TPB) hipLaunchKernelGGL(softmax_fwd_block_kernel<2>, grid, dim3(TPB), 0, st, x, y, v);
        else if (v <= 4 * 4 * TPB) hipLaunchKernelGGL(softmax_fwd_block_kernel<4>, grid, dim3(TPB), 0, st, x, y, v);
        else if (v <= 8 * 4 * TPB) hipLaunchKernelGGL(softmax_fwd_block_kernel<8>, grid, dim3(TPB), 0, st, x, y, v);
        else hipLaunchKernelGGL(softmax_fwd_block_kernel<16>, grid, dim3(TPB), 0, st, x, y, v);
    } else
        hipLaunchKernelGGL(softmax_fwd_kernel, dim3((unsigned)((n + WPB - 1) / WPB)), dim3(TPB), 0, st, x, y, v, n);
    return check("nchip_softmax_fwd");
}

int nchip_softmax_bwd(void *stream, const float *y, const float *g, float *dx, int v, int64_t n)
{
    if (n <= 0 || v <= 0) return 0;
    hipLaunchKernelGGL(softmax_bwd_kernel, dim3((unsigned)((n + WPB - 1) / WPB)), dim3(TPB), 0, (hipStream_t)stream, y, g, dx, v, n);
    return check("nchip_softmax_bwd");
}

// The out-of-range flag: one int of pinned host memory per process, written by the kernels
// that index a table with caller data, read (and cleared) by nchip_index_error().
static int *index_flag()
{
    static int *flag = nullptr;
    static std::mutex mu;
    std::lock_guard<std::mutex> lock(mu);
    if (!flag) {
        void *p = nullptr;
        if (hipHostMalloc(&p, 64, hipHostMallocDefault) != hipSuccess || !p) {
            fprintf(stderr, "nchip: cannot allocate the index error flag\n");
            abort();
        }
        flag = (int *)p;
        *flag = 0;
    }
    return flag;
}

int nchip_index_error(void)
{
    int *f = index_flag();
    const int v = *(volatile int *)f;
    *(volatile int *)f = 0;
    return v;
}

int nchip_indexed_log(void *stream, const float *p, const int32_t *idx, float *y, int v, int64_t n)
{
    if (n <= 0) return 0;
    hipLaunchKernelGGL(indexed_log_kernel, dim3(grid_for(n, 1 << 20)), dim3(TPB), 0, (hipStream_t)stream, p, idx, y, v, n,
                       index_flag());
    return check("nchip_indexed_log");
}

int nchip_nll_bwd(void *stream, const float *p, const int32_t *idx, const float *g, float *dl,
                  int v, int64_t n, int fused)
{
    if (n <= 0) return 0;
    if (v >= 1024 && v % 4 == 0 && (((uintptr_t)p | (uintptr_t)dl) & 15) == 0 && n <= 0x7fffffff && v <= 65535 * 4 * TPB)
        hipLaunchKernelGGL(nll_bwd_vec_kernel, dim3((unsigned)n, (unsigned)((v + 4 * TPB - 1) / (4 * TPB))), dim3(TPB), 0,
                           (hipStream_t)stream, p, idx, g, dl, v, fused);
    else
        hipLaunchKernelGGL(nll_bwd_kernel, dim3(grid_for(n * v)), dim3(TPB), 0, (hipStream_t)stream, p, idx, g, dl, v, n * v, fused);
    return check("nchip_nll_bwd");
}

int nchip_get_col(void *stream, const float *w, const int32_t *idx, float *y, int d, int v, int64_t n)
{
    return nchip_get_col_scaled(stream, w, idx, y, d, v, n, 1.0f);
}

int nchip_get_col_scaled(void *stream, const float *w, const int32_t *idx, float *y, int d, int v, int64_t n, float scale)
{
    if (n <= 0) return 0;
    hipLaunchKernelGGL(get_col_kernel, dim3(grid_for(n * d)), dim3(TPB), 0, (hipStream_t)stream, w, idx, y, d, v, n * d,
                       index_flag(), scale);
    return check("nchip_get_col");
}

int nchip_add_col(void *stream, const float *g, const int32_t *idx, float *dw, int d, int v, int64_t n)
{
    if (v <= 0 || d <= 0) return 0;
    if (n <= ADD_COL_MAX_N)
        hipLaunchKernelGGL(add_col_kernel, dim3(v), dim3(TPB), 0, (hipStream_t)stream, g, idx, dw, d, n);
    else
        hipLaunchKernelGGL(add_col_scan_kernel, dim3(v), dim3(TPB), 0, (hipStream_t)stream, g, idx, dw, d, n);
    return check("nchip_add_col");
}

int nchip_opt_update_multi(void *stream, int algo, const NchipOptTensor *dev_table,
                            const int *dev_chunk_prefix, int n_tensors, int total_chunks, int chunk,
                            float beta1, float beta2, float eps, float clip, float c1, float c2)
{
    if (n_tensors <= 0 || total_chunks <= 0) return 0;
    if (algo != 0 && algo != 1 && algo != 16) { fprintf(stderr, "nchip_opt_update_multi: unknown algo %d\n", algo); return -1; }
    hipLaunchKernelGGL(opt_update_multi_kernel, dim3(total_chunks), dim3(TPB), 0, (hipStream_t)stream,
                       dev_table, dev_chunk_prefix, n_tensors, chunk, algo, beta1, beta2, eps, clip, c1, c2);
    return check("nchip_opt_update_multi");
}

int nchip_opt_update(void *stream, int algo, float *w, float *m, float *v, const float *g, int64_t n,
                     float lr, float beta1, float beta2, float eps, float clip, float c1, float c2)
{
    if (n <= 0) return 0;
    if (algo != 0 && algo != 1 && algo != 16) { fprintf(stderr, "nchip_opt_update: unknown algo %d\n", algo); return -1; }
    hipLaunchKernelGGL(opt_update_kernel, dim3(grid_for(n)), dim3(TPB), 0, (hipStream_t)stream,
                       algo, w, m, v, g, n, lr, beta1, beta2, eps, clip, c1, c2);
    return check("nchip_opt_update");
}

} // extern "C"
