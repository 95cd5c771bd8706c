// Relative-position causal attention over memory + current segment
// (nncp.c:722-800 and its gradient), first generation: the per-(stream, head)
// products run as strided, two-level batched MFMA GEMMs that read the
// (features, streams, time) activations in place, and two fused column kernels
// do the score assembly (relative shift + bias + scale + causal mask + softmax)
// and its backward.  No head-split copies, no atomics; the gradients of the
// shared w_r / b_r are reduced over streams in a fixed order.
//
// Index conventions (K = M + T keys, query i, key j, distance delta = i+M-j):
//   score[j,i] = (k_j.q_i + rel[pi(delta), i] + b_r_scale*b_r[K-1-delta, h]) / sqrt(dk)
//   rel[p, i]  = w_r[:, p, h] . q_i ,  pi(delta) = max(d_pos-1-delta, 0)
//   valid iff 0 <= delta < attn_len
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include "../../include/nchip_kernels.h"
#include "k_internal.h"

namespace {

constexpr int TPB = 256;
constexpr int WPB = TPB / 64;
constexpr int MAXR = 8; // keys per lane: K <= 512

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

struct ScoreArgs {
    float *probs;       // (K, T, H, B) in: raw k.q ; out: probabilities
    const float *rel;   // (d_pos, T, H, B) or null
    const float *b_r;   // (K, H) or null
    int H, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
};

// one wavefront per score column (i, h, b)
__global__ __launch_bounds__(TPB) void score_softmax_fwd(ScoreArgs a)
{
    int lane = threadIdx.x & 63;
    int64_t col = (int64_t)blockIdx.x * WPB + (threadIdx.x >> 6);
    int64_t ncol = (int64_t)a.T * a.H * a.B;
    if (col >= ncol) return;
    int i = (int)(col % a.T), h = (int)((col / a.T) % a.H);
    float *p = a.probs + col * a.K;
    const float *rel = a.rel ? a.rel + col * a.d_pos : nullptr;
    const float *br = a.b_r ? a.b_r + (int64_t)h * a.K : nullptr;
    float s[MAXR];
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < MAXR; r++) {
        int j = lane + r * 64;
        s[r] = -INFINITY;
        if (j < a.K) {
            int delta = i + a.M - j;
            if (delta >= 0 && delta < a.attn_len) {
                float v = p[j];
                if (rel) { int pi = a.d_pos - 1 - delta; v += rel[pi > 0 ? pi : 0]; }
                if (br) v += a.b_r_scale * br[a.K - 1 - delta];
                s[r] = v * a.scale;
            }
        }
        mx = fmaxf(mx, s[r]);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int r = 0; r < MAXR; r++) {
        s[r] = (s[r] == -INFINITY) ? 0.0f : expf(s[r] - mx);
        sum += s[r];
    }
    float inv = 1.0f / wave_sum(sum);
#pragma unroll
    for (int r = 0; r < MAXR; r++) {
        int j = lane + r * 64;
        if (j < a.K) p[j] = s[r] * inv;
    }
}

struct ScoreBwdArgs {
    const float *probs; // (K, T, H, B)
    float *ds;          // in: dA = v_j.do_i ; out: dS
    float *drel;        // (d_pos, T, H, B) or null
    int H, B, T, M, K, d_pos, attn_len;
    float scale;
};

__global__ __launch_bounds__(TPB) void score_softmax_bwd(ScoreBwdArgs a)
{
    __shared__ float sh[WPB][64 * MAXR];
    int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int64_t col = (int64_t)blockIdx.x * WPB + w;
    int64_t ncol = (int64_t)a.T * a.H * a.B;
    if (col >= ncol) return;
    int i = (int)(col % a.T);
    const float *p = a.probs + col * a.K;
    float *ds = a.ds + col * a.K;
    float pv[MAXR], dv[MAXR], dot = 0.0f;
#pragma unroll
    for (int r = 0; r < MAXR; r++) {
        int j = lane + r * 64;
        pv[r] = j < a.K ? p[j] : 0.0f;
        dv[r] = j < a.K ? ds[j] : 0.0f;
        dot += pv[r] * dv[r];
    }
    dot = wave_sum(dot);
#pragma unroll
    for (int r = 0; r < MAXR; r++) {
        int j = lane + r * 64;
        float v = pv[r] * (dv[r] - dot) * a.scale; // masked entries have p = 0
        if (j < a.K) { ds[j] = v; sh[w][j] = v; }
    }
    if (!a.drel) return;
    // same-wavefront LDS exchange: make the writes visible before reading
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float *dr = a.drel + col * a.d_pos;
    // rows p >= 1 collect exactly one key: delta = d_pos-1-p
    for (int pp = lane; pp < a.d_pos; pp += 64) {
        if (pp == 0) continue;
        int delta = a.d_pos - 1 - pp;
        int j = i + a.M - delta;
        dr[pp] = (j >= 0 && j < a.K) ? sh[w][j] : 0.0f; // dS is already 0 where masked
    }
    // row 0 collects every key with delta >= d_pos-1, i.e. j <= i+M-(d_pos-1)
    int jmax = i + a.M - (a.d_pos - 1);
    float acc = 0.0f;
    for (int j = lane; j <= jmax && j < a.K; j += 64) acc += sh[w][j];
    acc = wave_sum(acc);
    if (lane == 0) dr[0] = acc;
}

// db_r[p, h] = b_r_scale * sum_{b,i} dS[j = p-(T-1-i), i, h, b]
__global__ __launch_bounds__(TPB) void bias_grad_kernel(const float *ds, float *db, int H, int B,
                                                        int T, int K, float b_r_scale)
{
    __shared__ float sh[TPB];
    int p = blockIdx.x, h = blockIdx.y;
    float acc = 0.0f;
    for (int e = threadIdx.x; e < B * T; e += TPB) {
        int i = e % T, b = e / T;
        int j = p - (T - 1 - i);
        if (j >= 0 && j < K)
            acc += ds[((int64_t)(b * H + h) * T + i) * K + j];
    }
    sh[threadIdx.x] = acc;
    __syncthreads();
    for (int s = TPB / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) db[(int64_t)h * K + p] = b_r_scale * sh[0];
}

// ---------------------------------------------------------------------------
// Second generation: ONE kernel per direction.  A workgroup (4 wavefronts) owns
// one (stream, head); Q, the relative-position vectors w_r[:, :, h], K and V of
// that head are staged once in LDS as [token][feature] rows of DK + 4 floats:
// with that stride both fragment shapes of v_mfma_f32_16x16x4_f32 read LDS at
// the 2-lanes-per-bank minimum ("row = token, k = feature": bank 4*il + g;
// "row = feature, k = token 4g + r": bank 16g + il).  Wavefront w owns query
// columns 16w..16w+15:
//   rel = w_r^T q -> per-wavefront LDS strip;  S = K^T q (+ shifted rel + bias,
//   scale, causal mask) entirely in registers;  softmax over the keys with two
//   xor-shuffles (a column lives in the 4 lanes l, l^16, l^32, l^48);
//   O = V P with P fed to the MFMA straight from the score registers.
// Key tiles beyond the causal frontier of the wavefront are skipped.
typedef float floatx4_t __attribute__((ext_vector_type(4)));

constexpr int FA_TMAX = 64, FA_KMAX = 128;
constexpr int FA_RSTRIDE = 131; // rel strip: shifted reads and tile writes both <= 4 lanes per bank
constexpr int FA_PSTRIDE = 65;  // transposed P / dS tiles of the backward

__device__ __forceinline__ floatx4_t mfma16(float a, float b, floatx4_t c)
{
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void wave_lds_sync()
{
    // same-wavefront LDS exchange: earlier writes of any lane before later reads
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// rows [0, rows_pad) of a [token][RS] LDS tile from global rows of DK floats;
// src(row) gives the address of the row, rows >= rows_valid become zero
template <int DK, typename F>
__device__ __forceinline__ void stage_rows(float *dst, int rows_pad, int rows_valid, F src)
{
    constexpr int RS = DK + 4, C4 = DK / 4;
    for (int idx = threadIdx.x; idx < rows_pad * C4; idx += 256) {
        int row = idx / C4, c = (idx % C4) * 4;
        floatx4_t v = { 0, 0, 0, 0 };
        if (row < rows_valid) v = *reinterpret_cast<const floatx4_t *>(src(row) + c);
        *reinterpret_cast<floatx4_t *>(dst + row * RS + c) = v;
    }
}

struct FusedFwdArgs {
    const float *q, *kv, *kvm, *w_r, *b_r;
    float *out, *probs;
    int64_t ldq, ldkv, ldo;
    int H, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
};

template <int DK>
constexpr size_t fused_fwd_lds_floats()
{
    return (size_t)FA_TMAX * (DK + 4) + 3 * (size_t)FA_KMAX * (DK + 4) + 4 * 16 * FA_RSTRIDE + FA_KMAX;
}

template <int DK>
__global__ __launch_bounds__(256) void relpos_attn_fwd_fused(FusedFwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int RS = DK + 4, NS = DK / 4, NT = FA_KMAX / 16;
    float *Qs = lds;                        // [64][RS]
    float *Ws = Qs + FA_TMAX * RS;          // [128][RS]
    float *Ks = Ws + FA_KMAX * RS;          // [128][RS]
    float *Vs = Ks + FA_KMAX * RS;          // [128][RS]
    float *Rs = Vs + FA_KMAX * RS;          // [4][16][FA_RSTRIDE]
    float *Bs = Rs + 4 * 16 * FA_RSTRIDE;   // [128]

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int Tp = (a.T + 15) & ~15, Kp = (a.K + 15) & ~15, Pp = (a.d_pos + 15) & ~15;

    stage_rows<DK>(Qs, Tp, a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
    if (a.w_r)
        stage_rows<DK>(Ws, Pp, a.d_pos, [&](int r) { return a.w_r + ((int64_t)h * a.d_pos + r) * DK; });
    auto kvrow = [&](int r) {
        return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r) : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) +
               (int64_t)h * DK;
    };
    stage_rows<DK>(Ks, Kp, a.K, kvrow);
    stage_rows<DK>(Vs, Kp, a.K, [&](int r) { return kvrow(r) + (int64_t)a.H * DK; });
    for (int idx = t; idx < FA_KMAX; idx += 256)
        Bs[idx] = (a.b_r && idx < a.K) ? a.b_r[(int64_t)h * a.K + idx] : 0.0f;
    __syncthreads();

    const int il = lane & 15, g = lane >> 4, i0 = 16 * w;
    if (i0 >= Tp) return; // no barrier below: wavefronts are independent from here on
    const int i = i0 + il;

    // query fragments: B operand (k-slot g, column il) for every 4-wide k-step
    float qf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) qf[s] = Qs[i * RS + 4 * s + g];

    float *Rw = Rs + (w * 16 + il) * FA_RSTRIDE; // this lane's column of rel
    if (a.w_r) {
        for (int pt = 0; pt < Pp / 16; pt++) {
            floatx4_t acc = { 0, 0, 0, 0 };
            const float *wrow = Ws + (pt * 16 + il) * RS + g;
#pragma unroll
            for (int s = 0; s < NS; s++) acc = mfma16(wrow[4 * s], qf[s], acc);
#pragma unroll
            for (int r = 0; r < 4; r++) Rw[pt * 16 + 4 * g + r] = acc[r];
        }
        wave_lds_sync();
    }

    // last key tile any column of this wavefront may see (causal frontier)
    int jt_end = (i0 + 15 + a.M) / 16 + 1;
    if (jt_end > Kp / 16) jt_end = Kp / 16;
    float sc[NT][4];
    float mx = -INFINITY;
#pragma unroll
    for (int jt = 0; jt < NT; jt++) {
        floatx4_t acc = { 0, 0, 0, 0 };
        if (jt < jt_end) {
            const float *krow = Ks + (jt * 16 + il) * RS + g;
#pragma unroll
            for (int s = 0; s < NS; s++) acc = mfma16(krow[4 * s], qf[s], acc);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            int j = jt * 16 + 4 * g + r;
            int delta = i + a.M - j;
            float v = -INFINITY;
            if (jt < jt_end && i < a.T && j < a.K && delta >= 0 && delta < a.attn_len) {
                v = acc[r];
                if (a.w_r) { int pi = a.d_pos - 1 - delta; v += Rw[pi > 0 ? pi : 0]; }
                v += a.b_r_scale * Bs[a.K - 1 - delta];
                v *= a.scale;
            }
            sc[jt][r] = v;
            mx = fmaxf(mx, v);
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    if (mx == -INFINITY) mx = 0.0f; // padding column
    float sum = 0.0f;
#pragma unroll
    for (int jt = 0; jt < NT; jt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float e = sc[jt][r] == -INFINITY ? 0.0f : expf(sc[jt][r] - mx);
            sc[jt][r] = e;
            sum += e;
        }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
#pragma unroll
    for (int jt = 0; jt < NT; jt++)
#pragma unroll
        for (int r = 0; r < 4; r++) sc[jt][r] *= inv;

    if (a.probs && i < a.T) {
        float *pc = a.probs + (((int64_t)b * a.H + h) * a.T + i) * a.K;
        const bool vec = (a.K & 3) == 0;
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            int j0 = jt * 16 + 4 * g;
            if (vec && j0 < a.K) {
                floatx4_t v = { sc[jt][0], sc[jt][1], sc[jt][2], sc[jt][3] };
                *reinterpret_cast<floatx4_t *>(pc + j0) = v;
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (j0 + r < a.K) pc[j0 + r] = sc[jt][r];
            }
        }
    }

    // O = V P
#pragma unroll
    for (int dt = 0; dt < DK / 16; dt++) {
        floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            if (jt < jt_end) {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    acc = mfma16(Vs[(jt * 16 + 4 * g + r) * RS + dt * 16 + il], sc[jt][r], acc);
            }
        }
        if (i < a.T) {
            float *o = a.out + (int64_t)h * DK + dt * 16 + 4 * g + a.ldo * (b + (int64_t)a.B * i);
            *reinterpret_cast<floatx4_t *>(o) = acc;
        }
    }
}

// Backward in the same shape.  Per wavefront (16 query columns):
//   dA = V^T dO in registers, dS = P (dA - colsum(P dA)) scale,
//   dq = K dS + w_r dRel  (dRel = rel-shift adjoint of dS, scattered into the
//   LDS strip that replaces V once every wavefront is done with it).
// Then P and dS are parked transposed in LDS (over K / w_r) and the wavefronts
// switch to owning key tiles:  dK = Q dS^T, dV = dO P^T,  and position tiles:
// dw_r[b,h] = Q dRel^T.  The per-(stream, head) dw_r / db_r partials go to
// scratch and a second kernel sums them over streams in a fixed order.
struct FusedBwdArgs {
    const float *q, *kv, *kvm, *w_r, *probs, *dout;
    float *dq, *dkv, *dkvm, *dwp, *dbp;
    int64_t ldq, ldkv, ldo;
    int H, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
};

template <int DK>
constexpr size_t fused_bwd_kw_floats()
{
    size_t a = 2 * (size_t)FA_KMAX * (DK + 4), b = 2 * (size_t)FA_KMAX * FA_PSTRIDE;
    return a > b ? a : b;
}
template <int DK>
constexpr size_t fused_bwd_v_floats()
{
    size_t a = (size_t)FA_KMAX * (DK + 4), b = (size_t)FA_TMAX * FA_RSTRIDE;
    return a > b ? a : b;
}
template <int DK>
constexpr size_t fused_bwd_lds_floats()
{
    return 2 * (size_t)FA_TMAX * (DK + 4) + fused_bwd_kw_floats<DK>() + fused_bwd_v_floats<DK>();
}

template <int DK>
__global__ __launch_bounds__(256) void relpos_attn_bwd_fused(FusedBwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int RS = DK + 4, NS = DK / 4, NT = FA_KMAX / 16, PS = FA_PSTRIDE;
    float *Qs = lds;                               // [64][RS]
    float *Os = Qs + FA_TMAX * RS;                 // [64][RS]  dO
    float *Ks = Os + FA_TMAX * RS;                 // [128][RS]
    float *Ws = Ks + FA_KMAX * RS;                 // [128][RS]
    float *Vs = Ks + fused_bwd_kw_floats<DK>();    // [128][RS]
    float *Rs = Vs;                                // [64][FA_RSTRIDE] dRel, once V is dead
    float *Pt = Ks;                                // [128][PS] P^T, once K and w_r are dead
    float *St = Ks + FA_KMAX * PS;                 // [128][PS] dS^T

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int Tp = (a.T + 15) & ~15, Kp = (a.K + 15) & ~15, Pp = (a.d_pos + 15) & ~15;
    const bool has_w = a.w_r != nullptr;

    stage_rows<DK>(Qs, Tp, a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
    stage_rows<DK>(Os, Tp, a.T, [&](int r) { return a.dout + (int64_t)h * DK + a.ldo * (b + (int64_t)a.B * r); });
    if (has_w)
        stage_rows<DK>(Ws, Pp, a.d_pos, [&](int r) { return a.w_r + ((int64_t)h * a.d_pos + r) * DK; });
    auto kvrow = [&](int r) {
        return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r) : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) +
               (int64_t)h * DK;
    };
    stage_rows<DK>(Ks, Kp, a.K, kvrow);
    stage_rows<DK>(Vs, Kp, a.K, [&](int r) { return kvrow(r) + (int64_t)a.H * DK; });
    __syncthreads();

    const int il = lane & 15, g = lane >> 4, i0 = 16 * w;
    const bool active = i0 < Tp; // uniform per wavefront
    const int i = i0 + il;
    int jt_end = (i0 + 15 + a.M) / 16 + 1;
    if (jt_end > Kp / 16) jt_end = Kp / 16;
    if (!active) jt_end = 0;

    float p[NT][4], ds[NT][4];
    floatx4_t dqa[DK / 16];
#pragma unroll
    for (int dt = 0; dt < DK / 16; dt++) dqa[dt] = floatx4_t{ 0, 0, 0, 0 };
    {
        float dof[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) dof[s] = active ? Os[i * RS + 4 * s + g] : 0.0f;
        const float *pc = a.probs + (((int64_t)b * a.H + h) * a.T + (i < a.T ? i : 0)) * a.K;
        const bool vec = (a.K & 3) == 0;
        float dot = 0.0f;
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            floatx4_t acc = { 0, 0, 0, 0 }, pv = { 0, 0, 0, 0 };
            if (jt < jt_end) {
                int j0 = jt * 16 + 4 * g;
                if (i < a.T) {
                    if (vec && j0 < a.K) pv = *reinterpret_cast<const floatx4_t *>(pc + j0);
                    else {
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (j0 + r < a.K) pv[r] = pc[j0 + r];
                    }
                }
                const float *vrow = Vs + (jt * 16 + il) * RS + g;
#pragma unroll
                for (int s = 0; s < NS; s++) acc = mfma16(vrow[4 * s], dof[s], acc);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                p[jt][r] = pv[r];
                ds[jt][r] = acc[r];
                dot += pv[r] * acc[r];
            }
        }
        dot += __shfl_xor(dot, 16, 64);
        dot += __shfl_xor(dot, 32, 64);
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
#pragma unroll
            for (int r = 0; r < 4; r++) ds[jt][r] = p[jt][r] * (ds[jt][r] - dot) * a.scale; // masked: p = 0
    }
    // dq, first part: K dS
#pragma unroll
    for (int dt = 0; dt < DK / 16; dt++)
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
            if (jt < jt_end) {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    dqa[dt] = mfma16(Ks[(jt * 16 + 4 * g + r) * RS + dt * 16 + il], ds[jt][r], dqa[dt]);
            }
    __syncthreads(); // every wavefront is done with V: its space becomes the dRel strip

    float *Rw = Rs + i * FA_RSTRIDE; // i < 64 always
    if (has_w && active) {
        // dRel[pi(delta), i] = sum of dS over the keys that read that row
        for (int pp = g; pp < Pp; pp += 4) Rw[pp] = 0.0f;
        wave_lds_sync();
        float acc0 = 0.0f;
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
            if (jt < jt_end) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    int j = jt * 16 + 4 * g + r;
                    int delta = i + a.M - j;
                    if (i < a.T && j < a.K && delta >= 0 && delta < a.attn_len) {
                        int pi = a.d_pos - 1 - delta;
                        if (pi >= 1) Rw[pi] = ds[jt][r]; // one key per row
                        else acc0 += ds[jt][r];          // row 0 collects the far keys
                    }
                }
            }
        acc0 += __shfl_xor(acc0, 16, 64);
        acc0 += __shfl_xor(acc0, 32, 64);
        if (g == 0) Rw[0] = acc0;
        wave_lds_sync();
        // dq, second part: w_r dRel
#pragma unroll
        for (int dt = 0; dt < DK / 16; dt++)
            for (int pt = 0; pt < Pp / 16; pt++) {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    dqa[dt] = mfma16(Ws[(pt * 16 + 4 * g + r) * RS + dt * 16 + il], Rw[pt * 16 + 4 * g + r], dqa[dt]);
            }
    }
    if (active && i < a.T) {
#pragma unroll
        for (int dt = 0; dt < DK / 16; dt++) {
            float *o = a.dq + (int64_t)h * DK + dt * 16 + 4 * g + a.ldq * (b + (int64_t)a.B * i);
            *reinterpret_cast<floatx4_t *>(o) = dqa[dt];
        }
    }
    __syncthreads(); // K and w_r are dead: park P^T and dS^T over them
    if (active) {
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
            if (jt * 16 < Kp) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    int j = jt * 16 + 4 * g + r;
                    Pt[j * PS + i] = p[jt][r];
                    St[j * PS + i] = ds[jt][r];
                }
            }
    }
    __syncthreads();

    // the contraction now runs over the query index; k-slot g of step s is
    // query 16*(s/4) + 4g + s%4, which keeps the Q / dO reads conflict-free
    const int nsq = Tp / 4;
    // dK = Q dS^T, dV = dO P^T: wavefront w owns key tiles w, w+4
    for (int jt = w; jt < Kp / 16; jt += 4) {
        // queries below jt*16 - M never see this key tile
        int s_lo = jt * 16 - a.M;
        s_lo = s_lo > 0 ? (s_lo / 16) * 4 : 0;
        float sb[FA_TMAX / 4], pb[FA_TMAX / 4];
#pragma unroll
        for (int s = 0; s < FA_TMAX / 4; s++) {
            int iq = 16 * (s >> 2) + 4 * g + (s & 3);
            bool on = s >= s_lo && s < nsq;
            sb[s] = on ? St[(jt * 16 + il) * PS + iq] : 0.0f;
            pb[s] = on ? Pt[(jt * 16 + il) * PS + iq] : 0.0f;
        }
        const int j = jt * 16 + il;
        float *dst = nullptr;
        if (j < a.K)
            dst = (j < a.M ? a.dkvm + a.ldkv * (b + (int64_t)a.B * j) : a.dkv + a.ldkv * (b + (int64_t)a.B * (j - a.M))) +
                  (int64_t)h * DK;
#pragma unroll
        for (int dt = 0; dt < DK / 16; dt++) {
            floatx4_t ak = { 0, 0, 0, 0 }, av = { 0, 0, 0, 0 };
#pragma unroll
            for (int s = 0; s < FA_TMAX / 4; s++)
                if (s >= s_lo && s < nsq) {
                    int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                    ak = mfma16(Qs[iq * RS + dt * 16 + il], sb[s], ak);
                    av = mfma16(Os[iq * RS + dt * 16 + il], pb[s], av);
                }
            if (dst) {
                *reinterpret_cast<floatx4_t *>(dst + dt * 16 + 4 * g) = ak;
                *reinterpret_cast<floatx4_t *>(dst + (int64_t)a.H * DK + dt * 16 + 4 * g) = av;
            }
        }
    }
    // dw_r partial of this (stream, head): Q dRel^T, wavefront w owns position tiles w, w+4
    if (has_w) {
        float *dwz = a.dwp + ((int64_t)b * a.H + h) * a.d_pos * DK;
        for (int pt = w; pt < Pp / 16; pt += 4) {
            float rb[FA_TMAX / 4];
#pragma unroll
            for (int s = 0; s < FA_TMAX / 4; s++) {
                int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                rb[s] = s < nsq ? Rs[iq * FA_RSTRIDE + pt * 16 + il] : 0.0f;
            }
            const int pp = pt * 16 + il;
#pragma unroll
            for (int dt = 0; dt < DK / 16; dt++) {
                floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
                for (int s = 0; s < FA_TMAX / 4; s++)
                    if (s < nsq) {
                        int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                        acc = mfma16(Qs[iq * RS + dt * 16 + il], rb[s], acc);
                    }
                if (pp < a.d_pos)
                    *reinterpret_cast<floatx4_t *>(dwz + (int64_t)pp * DK + dt * 16 + 4 * g) = acc;
            }
        }
    }
    // db_r partial: row K-1-delta collects the diagonal delta of dS
    if (a.dbp) {
        float *dbz = a.dbp + ((int64_t)b * a.H + h) * a.K;
        for (int delta = t; delta < a.K; delta += 256) {
            float acc = 0.0f;
            for (int iq = 0; iq < a.T; iq++) {
                int j = iq + a.M - delta;
                if (j >= 0 && j < a.K) acc += St[j * PS + iq];
            }
            dbz[a.K - 1 - delta] = a.b_r_scale * acc;
        }
    }
}

// dw_r (n_w) and db_r (n_b) = sums over the B per-stream partials, in stream order
__global__ __launch_bounds__(TPB) void attn_param_grad_reduce(const float *dwp, float *dw, int64_t n_w,
                                                              const float *dbp, float *db, int64_t n_b, int B)
{
    int64_t e = (int64_t)blockIdx.x * TPB + threadIdx.x;
    const float *src;
    float *dst;
    int64_t n;
    if (e < n_w) { src = dwp + e; dst = dw + e; n = n_w; }
    else if (e < n_w + n_b) { src = dbp + (e - n_w); dst = db + (e - n_w); n = n_b; }
    else return;
    float acc = 0.0f;
    for (int b = 0; b < B; b++) acc += src[(int64_t)b * n];
    *dst = acc;
}

template <typename KernelT>
bool allow_lds(KernelT kern, size_t bytes)
{
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)bytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return true;
}

template <int DK>
int launch_fused_fwd(hipStream_t st, const FusedFwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * fused_fwd_lds_floats<DK>();
    static const bool ok = allow_lds(relpos_attn_fwd_fused<DK>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL(relpos_attn_fwd_fused<DK>, dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int DK>
int launch_fused_bwd(hipStream_t st, const FusedBwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * fused_bwd_lds_floats<DK>();
    static const bool ok = allow_lds(relpos_attn_bwd_fused<DK>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL(relpos_attn_bwd_fused<DK>, dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

bool al16(const void *p) { return ((uintptr_t)p & 15) == 0; }

bool gen1_forced()
{
    static const char *e = getenv("NCHIP_ATTN_GEN1");
    return e && e[0] == '1';
}

// shapes the single-kernel path takes (one head of Q, K, V, w_r resident in LDS)
bool fused_shape_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr, int precision)
{
    return !gen1_forced() && precision == 0 && dk == dv && (dk == 64 || dk == 32) && T <= FA_TMAX &&
           K <= FA_KMAX && (!has_wr || d_pos <= FA_KMAX);
}

thread_local int g_last_launches = 0;

int bad(const char *msg)
{
    fprintf(stderr, "nchip_relpos_attn: %s\n", msg);
    return -1;
}

int check_shapes(int H, int dk, int dv, int B, int T, int M, int d_pos, int attn_len, bool has_wr)
{
    if (H < 1 || dk < 1 || dv < 1 || B < 1 || T < 1 || M < 0) return bad("non-positive dimension");
    if (M + T > 64 * MAXR) return bad("K = M + T exceeds 512");
    if (has_wr && (d_pos < 1 || d_pos > M + T)) return bad("d_pos must be in [1, K]");
    if (attn_len < 1) return bad("attn_len must be >= 1");
    if ((int64_t)B * H > 65535) return bad("B*H exceeds the grid limit");
    return 0;
}

} // namespace

extern "C" int nchip_relpos_attn_fwd(void *stream, const float *q, int64_t ldq,
                                     const float *kv, const float *kvm, int64_t ldkv,
                                     const float *w_r, const float *b_r,
                                     float *out, int64_t ldo, float *probs, float *rel,
                                     int H, int dk, int dv, int B, int T, int M, int d_pos,
                                     int attn_len, float b_r_scale, int precision)
{
    if (check_shapes(H, dk, dv, B, T, M, d_pos, attn_len, w_r != nullptr)) return -1;
    if (!q || !kv || !out || !probs || (M > 0 && !kvm) || (w_r && !rel)) return bad("null pointer");
    const int K = M + T, BH = B * H;
    const int64_t sK = (int64_t)K * T, sR = (int64_t)d_pos * T;
    int rc = 0;
    // single-kernel path when the head fits in LDS
    if (fused_shape_ok(dk, dv, T, K, d_pos, w_r != nullptr, precision) && ldq % 4 == 0 && ldkv % 4 == 0 &&
        ldo % 4 == 0 && al16(q) && al16(kv) && (!kvm || al16(kvm)) && (!w_r || al16(w_r)) && al16(out) &&
        al16(probs)) {
        FusedFwdArgs a;
        a.q = q; a.kv = kv; a.kvm = kvm; a.w_r = w_r; a.b_r = b_r; a.out = out; a.probs = probs;
        a.ldq = ldq; a.ldkv = ldkv; a.ldo = ldo;
        a.H = H; a.B = B; a.T = T; a.M = M; a.K = K; a.d_pos = w_r ? d_pos : 1; a.attn_len = attn_len;
        a.b_r_scale = b_r_scale; a.scale = 1.0f / sqrtf((float)dk);
        int frc = dk == 64 ? launch_fused_fwd<64>((hipStream_t)stream, a) : launch_fused_fwd<32>((hipStream_t)stream, a);
        if (frc == 0) { g_last_launches = 1; return 0; }
    }
    if (w_r) // rel = w_r[h]^T q
        rc |= nchip_gemm2(stream, 1, 0, d_pos, T, dk, 1.0f, w_r, dk, 0, (int64_t)dk * d_pos,
                          q, ldq * B, ldq, dk, 0.0f, rel, d_pos, sR * H, sR, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
    if (M > 0) // scores of the memory keys
        rc |= nchip_gemm2(stream, 1, 0, M, T, dk, 1.0f, kvm, ldkv * B, ldkv, dk,
                          q, ldq * B, ldq, dk, 0.0f, probs, K, sK * H, sK, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
    rc |= nchip_gemm2(stream, 1, 0, T, T, dk, 1.0f, kv, ldkv * B, ldkv, dk,
                      q, ldq * B, ldq, dk, 0.0f, probs + M, K, sK * H, sK, BH, H,
                      nullptr, 0, nullptr, precision, 1, nullptr);
    ScoreArgs a;
    a.probs = probs; a.rel = w_r ? rel : nullptr; a.b_r = b_r;
    a.H = H; a.B = B; a.T = T; a.M = M; a.K = K; a.d_pos = d_pos; a.attn_len = attn_len;
    a.b_r_scale = b_r_scale; a.scale = 1.0f / sqrtf((float)dk);
    int64_t ncol = (int64_t)T * BH;
    hipLaunchKernelGGL(score_softmax_fwd, dim3((unsigned)((ncol + WPB - 1) / WPB)), dim3(TPB), 0,
                       (hipStream_t)stream, a);
    // out = V_mem A[0:M] + V_cur A[M:K]
    if (M > 0)
        rc |= nchip_gemm2(stream, 0, 0, dv, T, M, 1.0f, kvm + (int64_t)H * dk, ldkv * B, ldkv, dv,
                          probs, K, sK * H, sK, 0.0f, out, ldo * B, ldo, dv, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
    rc |= nchip_gemm2(stream, 0, 0, dv, T, T, 1.0f, kv + (int64_t)H * dk, ldkv * B, ldkv, dv,
                      probs + M, K, sK * H, sK, M > 0 ? 1.0f : 0.0f, out, ldo * B, ldo, dv, BH, H,
                      nullptr, 0, nullptr, precision, 1, nullptr);
    if (hipGetLastError() != hipSuccess) return bad("kernel launch failed");
    g_last_launches = (w_r ? 1 : 0) + (M > 0 ? 2 : 0) + 3;
    return rc;
}

extern "C" int nchip_relpos_attn_last_launches(void) { return g_last_launches; }

extern "C" size_t nchip_relpos_attn_bwd_scratch(int H, int dk, int B, int T, int M, int d_pos)
{
    size_t K = (size_t)M + T, BH = (size_t)B * H;
    size_t inner = (size_t)dk * d_pos * H;
    // dS + drel + per-stream dw_r + reduction temporaries
    return K * T * BH + (size_t)d_pos * T * BH + inner * B + inner * (B / 8 + 2) + 64;
}

extern "C" int nchip_relpos_attn_bwd(void *stream, const float *q, int64_t ldq,
                                     const float *kv, const float *kvm, int64_t ldkv,
                                     const float *w_r, const float *probs,
                                     const float *dout, int64_t ldo,
                                     float *dq, float *dkv, float *dkvm, float *dw_r, float *db_r,
                                     int H, int dk, int dv, int B, int T, int M, int d_pos,
                                     int attn_len, float b_r_scale, int precision, float *scratch)
{
    if (check_shapes(H, dk, dv, B, T, M, d_pos, attn_len, w_r != nullptr)) return -1;
    if (!q || !kv || !probs || !dout || !dq || !dkv || !scratch || (M > 0 && (!kvm || !dkvm)) ||
        (w_r && !dw_r))
        return bad("null pointer");
    const int K = M + T, BH = B * H;
    const int64_t sK = (int64_t)K * T, sR = (int64_t)d_pos * T;
    float *ds = scratch;
    float *drel = ds + sK * BH;
    float *dwp = drel + (w_r ? sR * BH : 0);
    float *rtmp = dwp + (w_r ? (int64_t)dk * d_pos * BH : 0);
    hipStream_t st = (hipStream_t)stream;
    int rc = 0;
    if (fused_shape_ok(dk, dv, T, K, d_pos, w_r != nullptr, precision) && ldq % 4 == 0 && ldkv % 4 == 0 &&
        ldo % 4 == 0 && al16(q) && al16(kv) && (!kvm || al16(kvm)) && (!w_r || al16(w_r)) && al16(probs) &&
        al16(dout) && al16(dq) && al16(dkv) && (!dkvm || al16(dkvm)) && al16(scratch)) {
        FusedBwdArgs a;
        const int64_t n_w = w_r ? (int64_t)dk * d_pos * H : 0, n_b = db_r ? (int64_t)K * H : 0;
        a.q = q; a.kv = kv; a.kvm = kvm; a.w_r = w_r; a.probs = probs; a.dout = dout;
        a.dq = dq; a.dkv = dkv; a.dkvm = dkvm;
        a.dwp = scratch; a.dbp = db_r ? scratch + n_w * B : nullptr;
        a.ldq = ldq; a.ldkv = ldkv; a.ldo = ldo;
        a.H = H; a.B = B; a.T = T; a.M = M; a.K = K; a.d_pos = w_r ? d_pos : 1; a.attn_len = attn_len;
        a.b_r_scale = b_r_scale; a.scale = 1.0f / sqrtf((float)dk);
        int frc = dk == 64 ? launch_fused_bwd<64>(st, a) : launch_fused_bwd<32>(st, a);
        if (frc == 0) {
            g_last_launches = 1;
            if (n_w + n_b > 0) {
                hipLaunchKernelGGL(attn_param_grad_reduce, dim3((unsigned)((n_w + n_b + TPB - 1) / TPB)), dim3(TPB),
                                   0, st, (const float *)a.dwp, dw_r, n_w, (const float *)a.dbp, db_r, n_b, B);
                g_last_launches = 2;
            }
            if (hipGetLastError() != hipSuccess) return bad("kernel launch failed");
            return 0;
        }
    }
    const float *vm = kvm ? kvm + (int64_t)H * dk : nullptr, *vc = kv + (int64_t)H * dk;
    // dA = V^T dO
    if (M > 0)
        rc |= nchip_gemm2(stream, 1, 0, M, T, dv, 1.0f, vm, ldkv * B, ldkv, dv,
                          dout, ldo * B, ldo, dv, 0.0f, ds, K, sK * H, sK, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
    rc |= nchip_gemm2(stream, 1, 0, T, T, dv, 1.0f, vc, ldkv * B, ldkv, dv,
                      dout, ldo * B, ldo, dv, 0.0f, ds + M, K, sK * H, sK, BH, H,
                      nullptr, 0, nullptr, precision, 1, nullptr);
    ScoreBwdArgs a;
    a.probs = probs; a.ds = ds; a.drel = w_r ? drel : nullptr;
    a.H = H; a.B = B; a.T = T; a.M = M; a.K = K; a.d_pos = d_pos; a.attn_len = attn_len;
    a.scale = 1.0f / sqrtf((float)dk);
    int64_t ncol = (int64_t)T * BH;
    hipLaunchKernelGGL(score_softmax_bwd, dim3((unsigned)((ncol + WPB - 1) / WPB)), dim3(TPB), 0, st, a);
    // dq = K_mem dS[0:M] + K_cur dS[M:K] + w_r drel
    if (M > 0)
        rc |= nchip_gemm2(stream, 0, 0, dk, T, M, 1.0f, kvm, ldkv * B, ldkv, dk,
                          ds, K, sK * H, sK, 0.0f, dq, ldq * B, ldq, dk, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
    rc |= nchip_gemm2(stream, 0, 0, dk, T, T, 1.0f, kv, ldkv * B, ldkv, dk,
                      ds + M, K, sK * H, sK, M > 0 ? 1.0f : 0.0f, dq, ldq * B, ldq, dk, BH, H,
                      nullptr, 0, nullptr, precision, 1, nullptr);
    if (w_r) {
        rc |= nchip_gemm2(stream, 0, 0, dk, T, d_pos, 1.0f, w_r, dk, 0, (int64_t)dk * d_pos,
                          drel, d_pos, sR * H, sR, 1.0f, dq, ldq * B, ldq, dk, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
        // per-stream dw_r[b][h] = q dRel^T, then a fixed-order sum over streams
        rc |= nchip_gemm2(stream, 0, 1, dk, d_pos, T, 1.0f, q, ldq * B, ldq, dk,
                          drel, d_pos, sR * H, sR, 0.0f, dwp, dk, (int64_t)dk * d_pos * H,
                          (int64_t)dk * d_pos, BH, H, nullptr, 0, nullptr, precision, 1, nullptr);
        k_reduce_trailing(st, dwp, nullptr, dw_r, rtmp, (int64_t)dk * d_pos * H, B);
    }
    // dK = q dS^T, dV = dO A^T (memory part, then current part)
    if (M > 0) {
        rc |= nchip_gemm2(stream, 0, 1, dk, M, T, 1.0f, q, ldq * B, ldq, dk,
                          ds, K, sK * H, sK, 0.0f, dkvm, ldkv * B, ldkv, dk, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
        rc |= nchip_gemm2(stream, 0, 1, dv, M, T, 1.0f, dout, ldo * B, ldo, dv,
                          probs, K, sK * H, sK, 0.0f, dkvm + (int64_t)H * dk, ldkv * B, ldkv, dv, BH, H,
                          nullptr, 0, nullptr, precision, 1, nullptr);
    }
    rc |= nchip_gemm2(stream, 0, 1, dk, T, T, 1.0f, q, ldq * B, ldq, dk,
                      ds + M, K, sK * H, sK, 0.0f, dkv, ldkv * B, ldkv, dk, BH, H,
                      nullptr, 0, nullptr, precision, 1, nullptr);
    rc |= nchip_gemm2(stream, 0, 1, dv, T, T, 1.0f, dout, ldo * B, ldo, dv,
                      probs + M, K, sK * H, sK, 0.0f, dkv + (int64_t)H * dk, ldkv * B, ldkv, dv, BH, H,
                      nullptr, 0, nullptr, precision, 1, nullptr);
    if (db_r)
        hipLaunchKernelGGL(bias_grad_kernel, dim3(K, H), dim3(TPB), 0, st, (const float *)ds, db_r,
                           H, B, T, K, b_r_scale);
    if (hipGetLastError() != hipSuccess) return bad("kernel launch failed");
    g_last_launches = 5 + (M > 0 ? 4 : 0) + (w_r ? 4 : 0) + (db_r ? 1 : 0);
    return rc;
}
