// Data-movement and element-wise kernels behind the unfused libnc ops
// (nc_add, nc_mul, nc_slice, nc_concat, nc_permute_4d, nc_repeat_*, nc_pad,
// nc_rel_shift, nc_masked_fill, activations, reductions).  All are plain
// bandwidth-bound grid-stride kernels with coalesced accesses along libnc's
// axis 0; reductions use fixed-order two-stage sums (no atomics) so results
// are run-to-run identical.
#include "k_internal.h"
#include "k_act.h"

namespace {

constexpr int TPB = 256;

inline int nblocks(int64_t n, int per_block = TPB, int cap = 8192)
{
    int64_t b = (n + per_block - 1) / per_block;
    if (b > cap) b = cap;
    if (b < 1) b = 1;
    return (int)b;
}

#define GRID_STRIDE(i, n) \
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (n); i += (int64_t)gridDim.x * blockDim.x)

__device__ __forceinline__ void nd_offsets(const NdDesc &d, int64_t i, int64_t &oa, int64_t &ob)
{
    oa = 0; ob = 0;
#pragma unroll 1
    for (int a = 0; a < d.nd; a++) {
        int64_t c = i % d.dims[a];
        i /= d.dims[a];
        oa += c * d.sa[a];
        ob += c * d.sb[a];
    }
}

template <typename T>
__global__ void copy_nd_kernel(const T *src, T *dst, NdDesc d, int64_t n)
{
    GRID_STRIDE(i, n) {
        int64_t oa, ob;
        nd_offsets(d, i, oa, ob);
        dst[ob] = src[oa];
    }
}

__global__ void fill_f32_kernel(float *p, float v, int64_t n)
{
    GRID_STRIDE(i, n) p[i] = v;
}

__global__ void fill_bytes_kernel(uint8_t *p, uint8_t v, int64_t n)
{
    GRID_STRIDE(i, n) p[i] = v;
}

__global__ void binary_prefix_kernel(int op, const float *a, const float *b, float *y,
                                     int64_t n, int64_t nb)
{
    if (nb == n) {
        GRID_STRIDE(i, n) y[i] = op == KB_ADD ? a[i] + b[i] : a[i] * b[i];
    } else if (nb == 1) {
        float bv = b[0];
        GRID_STRIDE(i, n) y[i] = op == KB_ADD ? a[i] + bv : a[i] * bv;
    } else {
        GRID_STRIDE(i, n) {
            float bv = b[i % nb];
            y[i] = op == KB_ADD ? a[i] + bv : a[i] * bv;
        }
    }
}

__global__ void binary_nd_kernel(int op, const float *a, const float *b, float *y, NdDesc d, int64_t n)
{
    GRID_STRIDE(i, n) {
        int64_t oa, ob;
        nd_offsets(d, i, oa, ob);
        y[i] = op == KB_ADD ? a[oa] + b[ob] : a[oa] * b[ob];
    }
}

__global__ void masked_fill_kernel(const float *x, const int8_t *mask, float *y, int64_t n,
                                   int64_t nm, float c, int inv)
{
    GRID_STRIDE(i, n) {
        bool m = (mask[i % nm] != 0) != (inv != 0);
        y[i] = m ? c : x[i];
    }
}

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ float gelu_f(float x) { return nchip_gelu(x); }           // k_act.h
__device__ __forceinline__ float gelu_grad_f(float x) { return nchip_gelu_grad(x); }

__global__ void unary_fwd_kernel(int op, const float *x, float *y, int64_t n)
{
    GRID_STRIDE(i, n) {
        float v = x[i];
        switch (op) {
        case KU_SIGMOID: v = sigmoid_f(v); break;
        case KU_TANH: v = tanhf(v); break;
        case KU_RELU: v = v > 0.0f ? v : 0.0f; break;
        default: v = gelu_f(v); break;
        }
        y[i] = v;
    }
}

__global__ void unary_bwd_kernel(int op, const float *x, const float *g, float *dx, int64_t n)
{
    GRID_STRIDE(i, n) {
        float v = x[i], d;
        switch (op) {
        case KU_SIGMOID: { float s = sigmoid_f(v); d = s * (1.0f - s); break; }
        case KU_TANH: { float t = tanhf(v); d = 1.0f - t * t; break; }
        case KU_RELU: d = v > 0.0f ? 1.0f : 0.0f; break;
        default: d = gelu_grad_f(v); break;
        }
        dx[i] = g[i] * d;
    }
}

__global__ void gated_swish_fwd_kernel(const float *g, const float *x, float *y, int64_t n, float beta)
{
    GRID_STRIDE(i, n) y[i] = g[i] * x[i] * sigmoid_f(beta * x[i]);
}

__global__ void gated_swish_bwd_kernel(const float *g, const float *x, const float *gy,
                                       float *dg, float *dx, int64_t n, float beta)
{
    GRID_STRIDE(i, n) {
        float s = sigmoid_f(beta * x[i]);
        dg[i] = gy[i] * x[i] * s;
        dx[i] = gy[i] * g[i] * (s + beta * x[i] * s * (1.0f - s));
    }
}

__global__ void lerp_fwd_kernel(const float *a, const float *b, const float *t, float *y, int64_t n)
{
    GRID_STRIDE(i, n) y[i] = a[i] * (1.0f - t[i]) + b[i] * t[i];
}

__global__ void lerp_bwd_kernel(const float *a, const float *b, const float *t, const float *g,
                                float *da, float *db, float *dt, int64_t n)
{
    GRID_STRIDE(i, n) {
        da[i] = g[i] * (1.0f - t[i]);
        db[i] = g[i] * t[i];
        dt[i] = g[i] * (b[i] - a[i]);
    }
}

__global__ void lstm_clamped_fwd_kernel(const float *cp, const float *in, const float *fg,
                                        const float *ig, float *y, int64_t n)
{
    GRID_STRIDE(i, n) y[i] = cp[i] * fg[i] + fminf(1.0f - fg[i], ig[i]) * in[i];
}

__global__ void lstm_clamped_bwd_kernel(const float *cp, const float *in, const float *fg,
                                        const float *ig, const float *g, float *dcp, float *din,
                                        float *dfg, float *dig, int64_t n)
{
    GRID_STRIDE(i, n) {
        bool clamped = (1.0f - fg[i]) < ig[i];
        dcp[i] = g[i] * fg[i];
        din[i] = g[i] * fminf(1.0f - fg[i], ig[i]);
        dfg[i] = g[i] * cp[i] - (clamped ? g[i] * in[i] : 0.0f);
        dig[i] = clamped ? 0.0f : g[i] * in[i];
    }
}

// stage 1: tmp[s][i] = sum over the s-th slice of the outer axis.  Four
// interleaved chains (rows o0+u, o0+u+4, ...) keep four loads in flight; they
// are combined in chain order.
__global__ void reduce_trailing_stage1(const float *x, float *tmp, int64_t inner, int64_t outer,
                                       int nsplit)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int s = blockIdx.y;
    if (i >= inner) return;
    int64_t per = (outer + nsplit - 1) / nsplit;
    int64_t o0 = s * per, o1 = o0 + per < outer ? o0 + per : outer;
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
    int64_t o = o0;
    for (; o + 3 < o1; o += 4) {
        a0 += x[i + o * inner];
        a1 += x[i + (o + 1) * inner];
        a2 += x[i + (o + 2) * inner];
        a3 += x[i + (o + 3) * inner];
    }
    for (; o < o1; o++) a0 += x[i + o * inner];
    tmp[(int64_t)s * inner + i] = (a0 + a1) + (a2 + a3);
}

// stage 2: out[i] = y0[i] + sum_s tmp[s][i]; 4 interleaved slice groups per
// element (sequential inside a group), combined in group order
__global__ __launch_bounds__(256) void reduce_trailing_stage2(const float *tmp, const float *y0, float *out,
                                                              int64_t inner, int nsplit)
{
    __shared__ float sh[3][64];
    const int ig = threadIdx.x & 63, rg = threadIdx.x >> 6;
    const int64_t i = (int64_t)blockIdx.x * 64 + ig;
    float acc = 0.0f;
    if (i < inner) {
#pragma unroll 4
        for (int s = rg; s < nsplit; s += 4) acc += tmp[(int64_t)s * inner + i];
    }
    if (rg > 0) sh[rg - 1][ig] = acc;
    __syncthreads();
    if (rg == 0 && i < inner) {
        acc = (acc + sh[0][ig]) + (sh[1][ig] + sh[2][ig]);
        out[i] = y0 ? y0[i] + acc : acc;
    }
}

__global__ __launch_bounds__(256) void reduce_rows_multi_kernel(const KReduceRowsEntry *table)
{
    __shared__ float sh[3][64];
    const KReduceRowsEntry e = table[blockIdx.y];
    const int ig = threadIdx.x & 63, rg = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + ig;
    if (blockIdx.x * 64 >= e.n) return; // uniform per block
    float acc = 0.0f;
    if (i < e.n) {
#pragma unroll 4
        for (int r = rg; r < e.rows; r += 4) acc += e.src[(int64_t)r * e.stride + i];
    }
    if (rg > 0) sh[rg - 1][ig] = acc;
    __syncthreads();
    if (rg == 0 && i < e.n) e.dst[i] = (acc + sh[0][ig]) + (sh[1][ig] + sh[2][ig]);
}

// block-level fixed tree sum of 256 partials
__device__ __forceinline__ float block_tree_sum(float v, float *sh)
{
    sh[threadIdx.x] = v;
    __syncthreads();
    for (int s = TPB / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
        __syncthreads();
    }
    float r = sh[0];
    __syncthreads();
    return r;
}

__global__ void reduce_all_stage1(const float *x, float *tmp, int64_t n)
{
    __shared__ float sh[TPB];
    float acc = 0.0f;
    GRID_STRIDE(i, n) acc += x[i];
    float r = block_tree_sum(acc, sh);
    if (threadIdx.x == 0) tmp[blockIdx.x] = r;
}

__global__ void reduce_all_stage2(const float *tmp, float *out, int nb)
{
    __shared__ float sh[TPB];
    float acc = 0.0f;
    for (int i = threadIdx.x; i < nb; i += TPB) acc += tmp[i];
    float r = block_tree_sum(acc, sh);
    if (threadIdx.x == 0) out[0] = r;
}

__global__ void unbroadcast_nd_kernel(const float *g, float *out, NdDesc keep, NdDesc red,
                                      int64_t nout, int64_t nred)
{
    GRID_STRIDE(i, nout) {
        int64_t base, dummy;
        nd_offsets(keep, i, base, dummy);
        float acc = 0.0f;
        for (int64_t r = 0; r < nred; r++) {
            int64_t off, d2;
            nd_offsets(red, r, off, d2);
            acc += g[base + off];
        }
        out[i] = acc;
    }
}

__global__ void rel_shift_kernel(const float *x, float *y, int64_t n0, int64_t n1, int64_t total,
                                 int64_t pos, int64_t mult, int adjoint)
{
    GRID_STRIDE(e, total) {
        int64_t j = e % n0, i = (e / n0) % n1;
        int64_t s = pos + i * mult;
        int64_t src = adjoint ? j + s : j - s;
        y[e] = (src >= 0 && src < n0) ? x[e - j + src] : 0.0f;
    }
}

__global__ void pad_kernel(const float *x, float *y, int64_t n_in, int64_t n_out, int64_t cols,
                           int64_t left, int lop, int64_t right, int rop)
{
    GRID_STRIDE(e, n_out * cols) {
        int64_t i = e % n_out, c = e / n_out;
        const float *xc = x + c * n_in;
        int64_t s = i - left;
        float v = 0.0f;
        if (s < 0) { if (lop == 1) v = xc[0]; }
        else if (s >= n_in) { if (rop == 1) v = xc[n_in - 1]; }
        else v = xc[s];
        if (left < 0 && lop == 1 && i == 0)
            for (int64_t k = 0; k < -left; k++) v += xc[k];
        if (right < 0 && rop == 1 && i == n_out - 1)
            for (int64_t k = n_in + right; k < n_in; k++) v += xc[k];
        y[e] = v;
    }
}

// adjoint of pad_kernel: gx[s] = sum of the gy entries that read x[s]
__global__ void pad_bwd_kernel(const float *gy, float *gx, int64_t n_in, int64_t n_out,
                               int64_t cols, int64_t left, int lop, int64_t right, int rop)
{
    GRID_STRIDE(e, n_in * cols) {
        int64_t s = e % n_in, c = e / n_in;
        const float *gc = gy + c * n_out;
        float v = 0.0f;
        int64_t i = s + left;
        if (i >= 0 && i < n_out) v = gc[i];
        if (s == 0 && left > 0 && lop == 1)
            for (int64_t k = 0; k < left; k++) v += gc[k];
        if (s == n_in - 1 && right > 0 && rop == 1)
            for (int64_t k = n_out - right; k < n_out; k++) v += gc[k];
        if (left < 0 && lop == 1 && s < -left) v += gc[0];
        if (right < 0 && rop == 1 && s >= n_in + right) v += gc[n_out - 1];
        gx[e] = v;
    }
}

// dst (k-major copy) [i][kk] = src (m x k, rows contiguous) [kk][i]: 32 x 32 tiles through LDS,
// reads and writes both coalesced
__global__ __launch_bounds__(256) void transpose_f32_kernel(const float *src, float *dst, int m, int k)
{
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8
    const int i0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int kk = k0 + ty + 8 * r, i = i0 + tx;
        if (kk < k && i < m) tile[ty + 8 * r][tx] = src[(int64_t)kk * m + i];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int i = i0 + ty + 8 * r, kk = k0 + tx;
        if (i < m && kk < k) dst[(int64_t)i * k + kk] = tile[tx][ty + 8 * r];
    }
}

} // namespace

extern "C" {

void k_transpose_f32(hipStream_t st, const float *src, float *dst, int m, int k)
{
    if (m > 0 && k > 0)
        hipLaunchKernelGGL(transpose_f32_kernel, dim3((m + 31) / 32, (k + 31) / 32), dim3(256), 0, st, src, dst, m, k);
}

void k_copy_nd(hipStream_t st, const void *src, void *dst, const NdDesc *d, int esize)
{
    int64_t n = 1;
    for (int a = 0; a < d->nd; a++) n *= d->dims[a];
    if (n == 0) return;
    dim3 grid(nblocks(n)), block(TPB);
    if (esize == 4) hipLaunchKernelGGL(copy_nd_kernel<uint32_t>, grid, block, 0, st, (const uint32_t *)src, (uint32_t *)dst, *d, n);
    else if (esize == 2) hipLaunchKernelGGL(copy_nd_kernel<uint16_t>, grid, block, 0, st, (const uint16_t *)src, (uint16_t *)dst, *d, n);
    else hipLaunchKernelGGL(copy_nd_kernel<uint8_t>, grid, block, 0, st, (const uint8_t *)src, (uint8_t *)dst, *d, n);
}

void k_fill_f32(hipStream_t st, float *p, float v, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(fill_f32_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, p, v, n);
}

void k_fill_bytes(hipStream_t st, void *p, int v, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(fill_bytes_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, (uint8_t *)p, (uint8_t)v, n);
}

void k_binary_prefix(hipStream_t st, int op, const float *a, const float *b, float *y, int64_t n, int64_t nb)
{
    if (n > 0) hipLaunchKernelGGL(binary_prefix_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, op, a, b, y, n, nb);
}

void k_binary_nd(hipStream_t st, int op, const float *a, const float *b, float *y, const NdDesc *d, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(binary_nd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, op, a, b, y, *d, n);
}

void k_masked_fill(hipStream_t st, const float *x, const int8_t *mask, float *y, int64_t n, int64_t nm, float c, int inv)
{
    if (n > 0) hipLaunchKernelGGL(masked_fill_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, x, mask, y, n, nm, c, inv);
}

void k_unary_fwd(hipStream_t st, int op, const float *x, float *y, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(unary_fwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, op, x, y, n);
}

void k_unary_bwd(hipStream_t st, int op, const float *x, const float *g, float *dx, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(unary_bwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, op, x, g, dx, n);
}

void k_gated_swish_fwd(hipStream_t st, const float *g, const float *x, float *y, int64_t n, float beta)
{
    if (n > 0) hipLaunchKernelGGL(gated_swish_fwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, g, x, y, n, beta);
}

void k_gated_swish_bwd(hipStream_t st, const float *g, const float *x, const float *gy, float *dg, float *dx, int64_t n, float beta)
{
    if (n > 0) hipLaunchKernelGGL(gated_swish_bwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, g, x, gy, dg, dx, n, beta);
}

void k_lerp_fwd(hipStream_t st, const float *a, const float *b, const float *t, float *y, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(lerp_fwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, a, b, t, y, n);
}

void k_lerp_bwd(hipStream_t st, const float *a, const float *b, const float *t, const float *g, float *da, float *db, float *dt, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(lerp_bwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, a, b, t, g, da, db, dt, n);
}

void k_lstm_clamped_fwd(hipStream_t st, const float *cp, const float *in, const float *fg, const float *ig, float *y, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(lstm_clamped_fwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, cp, in, fg, ig, y, n);
}

void k_lstm_clamped_bwd(hipStream_t st, const float *cp, const float *in, const float *fg, const float *ig, const float *g, float *dcp, float *din, float *dfg, float *dig, int64_t n)
{
    if (n > 0) hipLaunchKernelGGL(lstm_clamped_bwd_kernel, dim3(nblocks(n)), dim3(TPB), 0, st, cp, in, fg, ig, g, dcp, din, dfg, dig, n);
}

int k_reduce_trailing_nsplit(int64_t inner, int64_t outer)
{
    // enough slices to occupy the chip while both stages stay short sequential
    // sums (stage 1: outer/nsplit terms per thread, stage 2: nsplit terms)
    int64_t blocks_x = (inner + TPB - 1) / TPB;
    int64_t s = 512 / (blocks_x > 0 ? blocks_x : 1);
    if (s > outer / 8) s = outer / 8;
    if (s > 64) s = 64;
    if (s < 1) s = 1;
    return (int)s;
}

void k_reduce_trailing(hipStream_t st, const float *x, const float *y0, float *out, float *tmp, int64_t inner, int64_t outer)
{
    if (inner <= 0) return;
    int ns = k_reduce_trailing_nsplit(inner, outer);
    dim3 grid((unsigned)((inner + TPB - 1) / TPB), ns);
    hipLaunchKernelGGL(reduce_trailing_stage1, grid, dim3(TPB), 0, st, x, tmp, inner, outer, ns);
    hipLaunchKernelGGL(reduce_trailing_stage2, dim3((unsigned)((inner + 63) / 64)), dim3(256), 0, st, (const float *)tmp, y0, out, inner, ns);
}

int k_reduce_trailing_partials(hipStream_t st, const float *x, float *tmp, int64_t inner, int64_t outer)
{
    if (inner <= 0) return 0;
    int ns = k_reduce_trailing_nsplit(inner, outer);
    dim3 grid((unsigned)((inner + TPB - 1) / TPB), ns);
    hipLaunchKernelGGL(reduce_trailing_stage1, grid, dim3(TPB), 0, st, x, tmp, inner, outer, ns);
    return ns;
}

void k_reduce_rows_multi(hipStream_t st, const KReduceRowsEntry *dev_table, int n_entries, int max_n)
{
    if (n_entries <= 0 || max_n <= 0) return;
    hipLaunchKernelGGL(reduce_rows_multi_kernel, dim3((unsigned)((max_n + 63) / 64), n_entries), dim3(256), 0, st, dev_table);
}

void k_reduce_all(hipStream_t st, const float *x, float *out, float *tmp, int64_t n)
{
    int nb = nblocks(n, TPB * 8, 1024);
    hipLaunchKernelGGL(reduce_all_stage1, dim3(nb), dim3(TPB), 0, st, x, tmp, n);
    hipLaunchKernelGGL(reduce_all_stage2, dim3(1), dim3(TPB), 0, st, (const float *)tmp, out, nb);
}

void k_unbroadcast_nd(hipStream_t st, const float *g, float *out, const NdDesc *keep, const NdDesc *red, int64_t nout, int64_t nred)
{
    if (nout > 0) hipLaunchKernelGGL(unbroadcast_nd_kernel, dim3(nblocks(nout)), dim3(TPB), 0, st, g, out, *keep, *red, nout, nred);
}

void k_rel_shift(hipStream_t st, const float *x, float *y, int64_t n0, int64_t n1, int64_t outer, int64_t pos, int64_t mult, int adjoint)
{
    int64_t total = n0 * n1 * outer;
    if (total > 0) hipLaunchKernelGGL(rel_shift_kernel, dim3(nblocks(total)), dim3(TPB), 0, st, x, y, n0, n1, total, pos, mult, adjoint);
}

void k_pad(hipStream_t st, const float *x, float *y, int64_t n_in, int64_t cols, int64_t left, int lop, int64_t right, int rop)
{
    int64_t n_out = n_in + left + right;
    hipLaunchKernelGGL(pad_kernel, dim3(nblocks(n_out * cols)), dim3(TPB), 0, st, x, y, n_in, n_out, cols, left, lop, right, rop);
}

void k_pad_bwd(hipStream_t st, const float *gy, float *gx, int64_t n_in, int64_t cols, int64_t left, int lop, int64_t right, int rop)
{
    int64_t n_out = n_in + left + right;
    hipLaunchKernelGGL(pad_bwd_kernel, dim3(nblocks(n_in * cols)), dim3(TPB), 0, st, gy, gx, n_in, n_out, cols, left, lop, right, rop);
}

} // extern "C"
