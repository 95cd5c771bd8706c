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

// db_r[p, h] = b_r_scale * sum_{b,i} dS[j = p-(T-1-i), i, h, b], in two steps:
// workgroup (h, c) sums chunk c of the streams with one thread per p (for a
// fixed query i consecutive p read consecutive keys j, so the reads of a
// wavefront are contiguous), then the chunk sums are added in chunk order.
__global__ __launch_bounds__(TPB) void bias_grad_partial(const float *ds, float *part, int H, int B,
                                                         int T, int K, int nchunk)
{
    const int h = blockIdx.x, c = blockIdx.y;
    const int b0 = (int)((int64_t)B * c / nchunk), b1 = (int)((int64_t)B * (c + 1) / nchunk);
    for (int p = threadIdx.x; p < K; p += TPB) {
        float acc = 0.0f;
        const int ilo = max(0, T - 1 - p); // j = p - (T-1-i) >= 0; j < K always holds for p < K
        for (int b = b0; b < b1; b++) {
            const float *row = ds + (int64_t)(b * H + h) * T * K + (p - (T - 1));
#pragma unroll 8
            for (int i = ilo; i < T; i++) acc += row[(int64_t)i * (K + 1)];
        }
        part[((int64_t)c * H + h) * K + p] = acc;
    }
}

__global__ __launch_bounds__(TPB) void bias_grad_final(const float *part, float *db, int64_t n, int nchunk,
                                                       float b_r_scale)
{
    int64_t e = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (e >= n) return;
    float acc = 0.0f;
    for (int c = 0; c < nchunk; c++) acc += part[(int64_t)c * n + e];
    db[e] = b_r_scale * acc;
}

thread_local int g_last_launches = 0;

bool al16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// single-kernel path (k_attn_fused.hip) unless NCHIP_ATTN_GEN1=1 forces the
// batched-GEMM path below, which also serves the shapes that do not fit in LDS
bool fused_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr, int precision)
{
    static const char *e = getenv("NCHIP_ATTN_GEN1");
    if (e && e[0] == '1') return false;
    return precision == 0 && k_attn_fused_shape_ok(dk, dv, T, K, d_pos, has_wr);
}

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
    if (fused_ok(dk, dv, T, K, d_pos, w_r != nullptr, precision) && ldq % 4 == 0 && ldkv % 4 == 0 &&
        ldo % 4 == 0 && al16(q) && al16(kv) && (!kvm || al16(kvm)) && (!w_r || al16(w_r)) && al16(out) &&
        al16(probs)) {
        FusedAttnFwdArgs a;
        a.q = q; a.kv = kv; a.kvm = kvm; a.w_r = w_r; a.b_r = b_r; a.out = out; a.probs = probs;
        a.ldq = ldq; a.ldkv = ldkv; a.ldo = ldo;
        a.H = H; a.B = B; a.T = T; a.M = M; a.K = K; a.d_pos = w_r ? d_pos : 1; a.attn_len = attn_len;
        a.b_r_scale = b_r_scale; a.scale = 1.0f / sqrtf((float)dk);
        a.q_only = -1;
        if (k_attn_fused_fwd((hipStream_t)stream, a, dk) == 0) { g_last_launches = 1; return 0; }
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

extern "C" int nchip_relpos_attn_fwd_step(void *stream, const float *q, int64_t ldq,
                                          const float *kv, const float *kvm, int64_t ldkv,
                                          const float *w_r, const float *b_r, float *out, int64_t ldo,
                                          int H, int dk, int dv, int B, int T, int M, int d_pos,
                                          int attn_len, float b_r_scale, int t)
{
    if (check_shapes(H, dk, dv, B, T, M, d_pos, attn_len, w_r != nullptr)) return -1;
    if (!q || !kv || !out || (M > 0 && !kvm)) return bad("null pointer");
    if (t < 0 || t >= T) return bad("query position outside the segment");
    const int K = M + T;
    if (!k_attn_fused_step_ok(dk, dv, T, K, d_pos, w_r != nullptr) || ldq % 4 || ldkv % 4 || ldo % 4 ||
        !al16(q) || !al16(kv) || (kvm && !al16(kvm)) || (w_r && !al16(w_r)) || !al16(out))
        return bad("single-query attention needs the single-kernel shapes (d_head 32/64, T <= 64, K <= 128)");
    FusedAttnFwdArgs a;
    a.q = q; a.kv = kv; a.kvm = kvm; a.w_r = w_r; a.b_r = b_r; a.out = out; a.probs = nullptr;
    a.ldq = ldq; a.ldkv = ldkv; a.ldo = ldo;
    a.H = H; a.B = B; a.T = T; a.M = M; a.K = K; a.d_pos = w_r ? d_pos : 1; a.attn_len = attn_len;
    a.b_r_scale = b_r_scale; a.scale = 1.0f / sqrtf((float)dk);
    a.q_only = t;
    if (k_attn_fused_fwd((hipStream_t)stream, a, dk)) return bad("kernel launch failed");
    g_last_launches = 1;
    return 0;
}

extern "C" size_t nchip_relpos_attn_bwd_scratch(int H, int dk, int B, int T, int M, int d_pos)
{
    size_t K = (size_t)M + T, BH = (size_t)B * H;
    size_t inner = (size_t)dk * d_pos * H;
    // dS + drel + per-stream dw_r + reduction temporaries + 16 chunk sums of db_r
    return K * T * BH + (size_t)d_pos * T * BH + inner * B + inner * (B / 8 + 2) + 64 + 16 * K * (size_t)H;
}

extern "C" int nchip_relpos_attn_bwd(void *stream, const float *q, int64_t ldq,
                                     const float *kv, const float *kvm, int64_t ldkv,
                                     const float *w_r, const float *probs,
                                     const float *dout, int64_t ldo,
                                     float *dq, float *dkv, float *dkvm, float *dw_r, float *db_r,
                                     int H, int dk, int dv, int B, int T, int M, int d_pos,
                                     int attn_len, float b_r_scale, int precision, float *scratch,
                                     int keep_partials)
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
    if (fused_ok(dk, dv, T, K, d_pos, w_r != nullptr, precision) && ldq % 4 == 0 && ldkv % 4 == 0 &&
        ldo % 4 == 0 && al16(q) && al16(kv) && (!kvm || al16(kvm)) && (!w_r || al16(w_r)) && al16(probs) &&
        al16(dout) && al16(dq) && al16(dkv) && (!dkvm || al16(dkvm)) && al16(scratch)) {
        FusedAttnBwdArgs a;
        const int64_t n_w = w_r ? (int64_t)dk * d_pos * H : 0, n_b = db_r ? (int64_t)K * H : 0;
        a.q = q; a.kv = kv; a.kvm = kvm; a.w_r = w_r; a.probs = probs; a.dout = dout;
        a.dq = dq; a.dkv = dkv; a.dkvm = dkvm;
        a.dwp = scratch; a.dbp = db_r ? scratch + n_w * B : nullptr;
        a.ldq = ldq; a.ldkv = ldkv; a.ldo = ldo;
        a.H = H; a.B = B; a.T = T; a.M = M; a.K = K; a.d_pos = w_r ? d_pos : 1; a.attn_len = attn_len;
        a.b_r_scale = b_r_scale; a.scale = 1.0f / sqrtf((float)dk);
        int nl = 0;
        int frc = k_attn_fused_bwd(st, a, dk, dw_r, db_r, n_w, n_b, &nl, keep_partials != 0);
        if (frc == -2) return bad("kernel launch failed");
        if (frc == 0) { g_last_launches = nl; return (keep_partials && n_w + n_b > 0) ? 1 : 0; }
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
    if (db_r) {
        const int nchunk = B < 16 ? B : 16;
        const int64_t inner = (int64_t)dk * d_pos * H;
        float *bpart = scratch + sK * BH + sR * BH + inner * B + inner * (B / 8 + 2) + 64; // the last region
        hipLaunchKernelGGL(bias_grad_partial, dim3(H, nchunk), dim3(TPB), 0, st, (const float *)ds, bpart,
                           H, B, T, K, nchunk);
        hipLaunchKernelGGL(bias_grad_final, dim3((unsigned)(((int64_t)H * K + TPB - 1) / TPB)), dim3(TPB), 0, st,
                           (const float *)bpart, db_r, (int64_t)H * K, nchunk, b_r_scale);
    }
    if (hipGetLastError() != hipSuccess) return bad("kernel launch failed");
    g_last_launches = 5 + (M > 0 ? 4 : 0) + (w_r ? 4 : 0) + (db_r ? 2 : 0);
    return rc;
}
