// Relative-position causal attention (nncp.c:722-800 and its gradient) on the bf16 matrix
// cores, for the bf16-operand variant: one kernel per direction, one workgroup (4 wavefronts)
// per (stream, head), d_head 64, up to 64 queries and 128 / 256 keys and relative positions.
//
// Every operand arrives as bf16 - the copies that the producing products and the optimiser
// leave next to their fp32 results (queries, keys, values, the gradient of the output, the
// position vectors) - so a workgroup fetches half the bytes of the fp32 kernels, and all
// products run on v_mfma_f32_16x16x32_bf16 with fp32 accumulation; scores, the relative
// shift, bias, mask and softmax stay fp32 in registers as in the fp32 kernels
// (k_attn_fused.hip), whose structure this follows: wavefront w owns query columns
// 16w .. 16w+15, a column lives in lanes il, il+16, il+32, il+48 (g = lane / 16), and an
// accumulator register r of lane (il, g) is row 4g + r of column il.
//
// What changes with 8 contraction values packed per lane: an operand must hold 8 consecutive
// contraction indices in 16 contiguous bytes of LDS.  Tiles contracted over the features
// (rel = w_r^T q, S = K^T q, dP = V^T dO) are staged as they lie in memory, [token][feature].
// Tiles contracted over keys or positions (O = V P, dq = K dS + w_r dRel) are staged
// transposed, [feature][slot], and in the slot order the score registers already have: the
// 8 values a lane holds for a pair of key tiles (2u, 2u+1) are keys 32u + 16t + 4g + r
// (t = 0, 1; r = 0..3), so key 32u + 16t + 4g + r sits in slot 32u + 8g + 4t + r and P (dS,
// dRel) goes from registers into the MFMA without a shuffle.  Tiles contracted over the
// queries (dK = Q dS^T, dV = dO P^T, dw_r = Q dRel^T) need Q and dO as [feature][query]
// and dS, P, dRel as [key][query], which the wavefronts park in LDS once dq is done.
//
// The probabilities are saved for the backward as the very bf16 values the forward
// multiplied with V.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include "k_internal.h"
#include "k_addrspace.h"
#include "k_bf16.h"

namespace {

typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int BT = 64; // queries per head

__device__ __forceinline__ floatx4_t mfma_bf16(u32x4 a, u32x4 b, floatx4_t c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// slot of token j in a transposed tile (see the header): j = 32u + 16t + 4g + r -> 32u + 8g + 4t + r
__device__ __forceinline__ int slot_of(int j)
{
    return (j & ~31) | ((j & 12) << 1) | ((j & 16) >> 2) | (j & 3);
}

// element offset of 16-byte chunk `chunk` in row `frow` of a transposed tile (rows TS apart):
// the chunks of feature rows 8c .. 8c+7 are stored at chunk ^ c (see park_transposed)
template <int TS>
__device__ __forceinline__ int tr_off(int frow, int chunk)
{
    return frow * TS + ((chunk ^ ((frow >> 3) & 7)) << 3);
}

// the 8 bf16 values of a lane for the pair of tiles (2u, 2u + 1): element e = 4t + r
__device__ __forceinline__ u32x4 pack8(const float (&lo)[4], const float (&hi)[4])
{
    return u32x4{ pack_bf16(lo[0], lo[1]), pack_bf16(lo[2], lo[3]), pack_bf16(hi[0], hi[1]), pack_bf16(hi[2], hi[3]) };
}

// One tile of ROWS token rows of DK bf16 features each: loads (16 bytes per thread and
// step, rows >= rows_valid read row 0 and are zeroed at the store) and the two ways of
// parking them.  Loads and stores are separate calls so that all loads of a kernel are in
// flight before the first store waits for one.
template <int DK, int ROWS>
struct RowTile {
    static constexpr int C8 = DK / 8, N = ROWS * C8 / 256;
    static_assert(ROWS * C8 % 256 == 0, "whole steps");
    u32x4 v[N];

    template <typename F>
    __device__ __forceinline__ void fetch(int rows_valid, F src)
    {
#pragma unroll
        for (int it = 0; it < N; it++) {
            const int idx = threadIdx.x + it * 256, row = idx / C8, c = idx % C8;
            v[it] = *as_global(reinterpret_cast<const u32x4 *>(src(row < rows_valid ? row : 0) + c * 8));
        }
    }

    // [token][feature], rows RB elements apart
    template <int RB>
    __device__ __forceinline__ void park_rows(uint16_t *dst, int rows_valid) const
    {
#pragma unroll
        for (int it = 0; it < N; it++) {
            const int idx = threadIdx.x + it * 256, row = idx / C8, c = idx % C8;
            *reinterpret_cast<u32x4 *>(dst + row * RB + c * 8) = row < rows_valid ? v[it] : u32x4{ 0, 0, 0, 0 };
        }
    }

    // [feature][token position], rows TS elements apart; SLOTS: tokens in slot order
    template <int TS, bool SLOTS>
    __device__ __forceinline__ void park_transposed(uint16_t *dst, int rows_valid) const
    {
#pragma unroll
        for (int it = 0; it < N; it++) {
            const int idx = threadIdx.x + it * 256, row = idx / C8, c = idx % C8;
            const int col = SLOTS ? slot_of(row) : row;
            // feature rows 8c .. 8c+7 keep their 16-byte chunks at chunk ^ c (tr_off): the 8 lanes
            // that hold one token then write 8 different banks instead of one
            const int pcol = (((col >> 3) ^ (c & 7)) << 3) | (col & 7);
            const bool on = row < rows_valid;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t w = on ? v[it][e] : 0u;
                dst[(c * 8 + 2 * e) * TS + pcol] = (uint16_t)(w & 0xffffu);
                dst[(c * 8 + 2 * e + 1) * TS + pcol] = (uint16_t)(w >> 16);
            }
        }
    }
};

template <int DK, int NT>
struct Dims {
    static constexpr int KR = NT * 16;     // key / position rows of the tiles
    static constexpr int RB = DK + 8;      // [token][feature] row, in bf16 elements (16-byte multiple)
    static constexpr int TS = KR + 8;      // [feature][slot] row
    static constexpr int QS = BT + 8;      // [feature][query] and [key][query] rows
    static constexpr int RST = KR + 3;     // strip row in floats (odd: columns fall on different banks)
    static constexpr int NB = 2 * KR;      // bias row: zero from K up to the largest index a masked key forms
    static constexpr int NKS = DK / 32;    // MFMAs per feature contraction
    static constexpr int ND = DK / 16;     // feature tiles
};

template <int DK, int NT>
struct FwdLds {
    using D = Dims<DK, NT>;
    // bytes.  w: the position vectors, then (once every wavefront has its rel strip) V^T
    static constexpr int wv_a = D::KR * D::RB * 2, wv_b = DK * D::TS * 2, wv = wv_a > wv_b ? wv_a : wv_b;
    static constexpr int q = 0, w = q + BT * D::RB * 2, k = w + wv, r = k + D::KR * D::RB * 2,
                         b = r + BT * D::RST * 4, bytes = b + D::NB * 4;
};

template <int DK, int NT>
__global__ __launch_bounds__(256) void relpos_attn_fwd_bf16(Bf16AttnFwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using D = Dims<DK, NT>;
    using L = FwdLds<DK, NT>;
    constexpr int KR = D::KR, RB = D::RB, TS = D::TS, RST = D::RST, NKS = D::NKS, ND = D::ND;
    uint8_t *base = reinterpret_cast<uint8_t *>(lds);
    uint16_t *Qs = reinterpret_cast<uint16_t *>(base + L::q), *Ws = reinterpret_cast<uint16_t *>(base + L::w);
    uint16_t *Ks = reinterpret_cast<uint16_t *>(base + L::k), *Vt = Ws;
    float *Rs = reinterpret_cast<float *>(base + L::r), *Bs = reinterpret_cast<float *>(base + L::b);

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B; // consecutive workgroups: consecutive streams
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    const bool has_w = a.w_r != nullptr;

    // all global loads up front, in the order they are waited for
    float bias_t[D::NB / 256];
#pragma unroll
    for (int u = 0; u < D::NB / 256; u++) {
        const int e = t + 256 * u;
        bias_t[u] = (a.b_r && e < a.K) ? as_global(a.b_r)[(int64_t)h * a.K + e] : 0.0f;
    }
    const uint16_t *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    RowTile<DK, BT> tq;
    RowTile<DK, KR> tw, tk, tv;
    {
        auto kvrow = [&](int r) {
            return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                            : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
        };
        tq.fetch(a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
        tw.fetch(n_w, [&](int r) { return w_base + (int64_t)r * DK; });
        tk.fetch(a.K, kvrow);
        tv.fetch(a.K, [&](int r) { return kvrow(r) + (int64_t)a.H * DK; });
    }
#pragma unroll
    for (int u = 0; u < D::NB / 256; u++) Bs[t + 256 * u] = bias_t[u] * (a.b_r_scale * a.scale);
    tq.template park_rows<RB>(Qs, a.T);
    tw.template park_rows<RB>(Ws, n_w);
    tk.template park_rows<RB>(Ks, a.K);
    __syncthreads();

    // the wavefront's 16 queries as B operand: column il, features 32s + 8g .. + 7
    u32x4 qf[NKS];
#pragma unroll
    for (int s = 0; s < NKS; s++) qf[s] = *reinterpret_cast<const u32x4 *>(Qs + i * RB + 32 * s + 8 * g);

    float *Rw = Rs + i * RST; // this lane's column of rel (scaled)
#pragma unroll
    for (int pt = 0; pt < NT; pt++) {
        floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
        for (int s = 0; s < NKS; s++)
            acc = mfma_bf16(*reinterpret_cast<const u32x4 *>(Ws + (pt * 16 + il) * RB + 32 * s + 8 * g), qf[s], acc);
#pragma unroll
        for (int r = 0; r < 4; r++) Rw[pt * 16 + 4 * g + r] = acc[r] * a.scale;
    }
    wave_lds_sync(); // the strip is the wavefront's own: its writes before the shifted reads

    float sc[NT][4];
    float mx = -INFINITY;
    {
        const int dbase = i + a.M - 4 * g;      // delta of key 4g of tile 0
        const int pbase = a.d_pos - 1 - dbase;  // its rel row before clamping
        const int pmax = a.d_pos - 1;
        const unsigned dlim = i < a.T ? (unsigned)a.attn_len : 0u;
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
            for (int s = 0; s < NKS; s++)
                acc = mfma_bf16(*reinterpret_cast<const u32x4 *>(Ks + (jt * 16 + il) * RB + 32 * s + 8 * g), qf[s], acc);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                int pi = pbase + (jt * 16 + r); // d_pos-1-delta
                pi = pi < 0 ? 0 : (pi > pmax ? pmax : pi);
                const float relv = Rw[pi];
                const float bv = Bs[(a.K - 1 - (int)delta) & (D::NB - 1)];
                // key j < K is implied: delta >= 0 > i - T for a real column
                const float v = delta < dlim ? acc[r] * a.scale + relv + bv : -INFINITY;
                sc[jt][r] = v;
                mx = fmaxf(mx, v);
            }
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
            const float e = __expf(sc[jt][r] - mx); // exp(-inf) = 0 for masked keys
            sc[jt][r] = e;
            sum += e;
        }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
#pragma unroll
    for (int jt = 0; jt < NT; jt++)
#pragma unroll
        for (int r = 0; r < 4; r++) sc[jt][r] *= inv;

    // P as bf16: what the PV product multiplies and what the backward reads
    u32x4 pb[NT / 2];
#pragma unroll
    for (int u = 0; u < NT / 2; u++) pb[u] = pack8(sc[2 * u], sc[2 * u + 1]);
    if (a.probs && i < a.T) {
        uint16_t NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + i) * a.K;
#pragma unroll
        for (int u = 0; u < NT / 2; u++) {
            const int j0 = 32 * u + 4 * g; // keys j0 .. j0+3 and j0+16 .. j0+19
            if (j0 < a.K) *reinterpret_cast<u32x2 NCHIP_GLOBAL *>(pc + j0) = u32x2{ pb[u][0], pb[u][1] };
            if (j0 + 16 < a.K) *reinterpret_cast<u32x2 NCHIP_GLOBAL *>(pc + j0 + 16) = u32x2{ pb[u][2], pb[u][3] };
        }
    }

    // O = V P: A = V^T tile (row = feature, slots 32u + 8g .. + 7), B = P from registers.
    // V^T takes the place of the position vectors once every wavefront is past its rel phase.
    __syncthreads();
    tv.template park_transposed<TS, true>(Vt, a.K);
    __syncthreads();
    floatx4_t acc[ND];
#pragma unroll
    for (int dt = 0; dt < ND; dt++) acc[dt] = floatx4_t{ 0, 0, 0, 0 };
#pragma unroll
    for (int u = 0; u < NT / 2; u++)
#pragma unroll
        for (int dt = 0; dt < ND; dt++)
            acc[dt] = mfma_bf16(*reinterpret_cast<const u32x4 *>(Vt + tr_off<TS>(dt * 16 + il, 4 * u + g)), pb[u], acc[dt]);
    if (i < a.T) {
        const int64_t o = (int64_t)h * DK + 4 * g + a.ldo * (b + (int64_t)a.B * i);
#pragma unroll
        for (int dt = 0; dt < ND; dt++) {
            *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(as_global(a.out) + o + dt * 16) = acc[dt];
            if (a.out16)
                *reinterpret_cast<u32x2 NCHIP_GLOBAL *>(as_global(a.out16) + o + dt * 16) =
                    u32x2{ pack_bf16(acc[dt][0], acc[dt][1]), pack_bf16(acc[dt][2], acc[dt][3]) };
        }
    }
}

template <int DK, int NT>
struct BwdLds {
    using D = Dims<DK, NT>;
    static constexpr int rows = D::KR * D::RB * 2, slots = DK * D::TS * 2, byq = D::KR * D::QS * 2;
    static constexpr int va = rows > byq ? rows : byq, kb = slots > byq ? slots : byq;
    // bytes.  v: V, then dS^T;  kt: K^T, then P^T;  wt: w_r^T;  rt: dRel^T (+ one dump row)
    static constexpr int v = 0, kt = v + va, wt = kt + kb, rt = wt + slots, qt = rt + byq + D::QS * 2,
                         ot = qt + DK * D::QS * 2, bytes = ot + DK * D::QS * 2;
};

template <int DK, int NT>
__global__ __launch_bounds__(256) void relpos_attn_bwd_bf16(Bf16AttnBwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using D = Dims<DK, NT>;
    using L = BwdLds<DK, NT>;
    constexpr int KR = D::KR, RB = D::RB, TS = D::TS, QS = D::QS, NKS = D::NKS, ND = D::ND;
    constexpr int NQS = BT / 32; // MFMAs per contraction over the queries
    uint8_t *base = reinterpret_cast<uint8_t *>(lds);
    uint16_t *Vs = reinterpret_cast<uint16_t *>(base + L::v), *Kt = reinterpret_cast<uint16_t *>(base + L::kt);
    uint16_t *Wt = reinterpret_cast<uint16_t *>(base + L::wt), *Qt = reinterpret_cast<uint16_t *>(base + L::qt);
    uint16_t *Ot = reinterpret_cast<uint16_t *>(base + L::ot);
    uint16_t *Rt = reinterpret_cast<uint16_t *>(base + L::rt); // [KR + 1][QS]: dRel^T, row KR a dump row
    uint16_t *St = Vs, *Pt = Kt;                                // [KR][QS] each, once V and K^T are dead

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B;
    const bool has_w = a.w_r != nullptr;
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    const int ic = i < a.T ? i : 0; // a readable column for the padding lanes

    // every global load up front, in the order the phases need them
    const uint16_t *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    RowTile<DK, KR> tv, tk, tw;
    RowTile<DK, BT> tq, to;
    u32x4 dof[NKS];
    u32x2 praw[NT];
    {
        auto kvrow = [&](int r) {
            return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                            : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
        };
        const uint16_t *orow = a.dout + (int64_t)h * DK + a.ldo * (b + (int64_t)a.B * ic);
#pragma unroll
        for (int s = 0; s < NKS; s++) dof[s] = *as_global(reinterpret_cast<const u32x4 *>(orow + 32 * s + 8 * g));
        tv.fetch(a.K, [&](int r) { return kvrow(r) + (int64_t)a.H * DK; });
        const uint16_t NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + ic) * a.K;
#pragma unroll
        for (int jt = 0; jt < NT; jt++) { // clamped addresses; masked at first use
            const int j0 = jt * 16 + 4 * g;
            praw[jt] = *reinterpret_cast<const u32x2 NCHIP_GLOBAL *>(pc + (j0 < a.K ? j0 : 0));
        }
        tk.fetch(a.K, kvrow);
        tw.fetch(n_w, [&](int r) { return w_base + (int64_t)r * DK; });
        tq.fetch(a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
        to.fetch(a.T, [&](int r) { return a.dout + (int64_t)h * DK + a.ldo * (b + (int64_t)a.B * r); });
    }
    if (i >= a.T) {
#pragma unroll
        for (int s = 0; s < NKS; s++) dof[s] = u32x4{ 0, 0, 0, 0 };
    }
    tv.template park_rows<RB>(Vs, a.K);
    // dRel^T starts at zero: a row that no key of a column reads stays zero
    for (int e = t; e < (KR + 1) * QS / 8; e += 256) reinterpret_cast<u32x4 *>(Rt)[e] = u32x4{ 0, 0, 0, 0 };
    __syncthreads();

    // dP = V^T dO, then dS = P (dP - colsum(P dP)) / sqrt(dk)
    float p[NT][4], ds[NT][4];
    {
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            const bool on = i < a.T && jt * 16 + 4 * g < a.K; // (K is a multiple of 4)
            p[jt][0] = on ? bf16_bits_to_f32(praw[jt][0] & 0xffffu) : 0.0f;
            p[jt][1] = on ? bf16_bits_to_f32(praw[jt][0] >> 16) : 0.0f;
            p[jt][2] = on ? bf16_bits_to_f32(praw[jt][1] & 0xffffu) : 0.0f;
            p[jt][3] = on ? bf16_bits_to_f32(praw[jt][1] >> 16) : 0.0f;
        }
        float dot = 0.0f;
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
            for (int s = 0; s < NKS; s++)
                acc = mfma_bf16(*reinterpret_cast<const u32x4 *>(Vs + (jt * 16 + il) * RB + 32 * s + 8 * g), dof[s], acc);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                ds[jt][r] = acc[r];
                dot += p[jt][r] * acc[r];
            }
        }
        dot += __shfl_xor(dot, 16, 64);
        dot += __shfl_xor(dot, 32, 64);
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
#pragma unroll
            for (int r = 0; r < 4; r++) ds[jt][r] = p[jt][r] * (ds[jt][r] - dot) * a.scale; // masked: p = 0
    }
    tk.template park_transposed<TS, true>(Kt, a.K);
    tw.template park_transposed<TS, true>(Wt, n_w);
    tq.template park_transposed<QS, false>(Qt, a.T);
    to.template park_transposed<QS, false>(Ot, a.T);

    // dRel[pi(delta), i] = sum of dS over the keys that read that row, written as bf16 (what the
    // products below multiply) straight into dRel^T: rows >= 1 receive exactly one key of a
    // column, row 0 collects the far keys, masked keys go to the dump row
    {
        const int dbase = i + a.M - 4 * g, pbase = a.d_pos - 1 - dbase;
        const unsigned dlim = (i < a.T && has_w) ? (unsigned)a.attn_len : 0u;
        float acc0 = 0.0f;
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                const int pi = pbase + (jt * 16 + r);
                const bool on = delta < dlim;
                Rt[((on && pi >= 1) ? pi : KR) * QS + i] = f32_to_bf16_rne(ds[jt][r]);
                acc0 += (on && pi < 1) ? ds[jt][r] : 0.0f;
            }
        acc0 += __shfl_xor(acc0, 16, 64);
        acc0 += __shfl_xor(acc0, 32, 64);
        if (g == 0) Rt[i] = f32_to_bf16_rne(acc0);
    }
    __syncthreads(); // K^T, w_r^T, Q^T, dO^T and dRel^T visible

    // dq = K dS + w_r dRel: B operands from registers / the strip, in slot order
    {
        floatx4_t dqa[ND];
#pragma unroll
        for (int dt = 0; dt < ND; dt++) dqa[dt] = floatx4_t{ 0, 0, 0, 0 };
#pragma unroll
        for (int u = 0; u < NT / 2; u++) {
            const u32x4 sb = pack8(ds[2 * u], ds[2 * u + 1]);
            uint32_t rv[8]; // dRel of positions 32u + 16t + 4g + r for this lane's column
#pragma unroll
            for (int e = 0; e < 8; e++) rv[e] = Rt[(32 * u + 16 * (e >> 2) + 4 * g + (e & 3)) * QS + i];
            const u32x4 rb = { rv[0] | (rv[1] << 16), rv[2] | (rv[3] << 16), rv[4] | (rv[5] << 16), rv[6] | (rv[7] << 16) };
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                dqa[dt] = mfma_bf16(*reinterpret_cast<const u32x4 *>(Kt + tr_off<TS>(dt * 16 + il, 4 * u + g)), sb, dqa[dt]);
                dqa[dt] = mfma_bf16(*reinterpret_cast<const u32x4 *>(Wt + tr_off<TS>(dt * 16 + il, 4 * u + g)), rb, dqa[dt]);
            }
        }
        if (i < a.T) {
            const int64_t o = (int64_t)h * DK + 4 * g + a.ldq * (b + (int64_t)a.B * i);
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(as_global(a.dq) + o + dt * 16) = dqa[dt];
                if (a.dq16)
                    *reinterpret_cast<u32x2 NCHIP_GLOBAL *>(as_global(a.dq16) + o + dt * 16) =
                        u32x2{ pack_bf16(dqa[dt][0], dqa[dt][1]), pack_bf16(dqa[dt][2], dqa[dt][3]) };
            }
        }
    }
    __syncthreads(); // V and K^T are dead: park dS^T and P^T over them
#pragma unroll
    for (int jt = 0; jt < NT; jt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int j = jt * 16 + 4 * g + r;
            St[j * QS + i] = f32_to_bf16_rne(ds[jt][r]);
            Pt[j * QS + i] = f32_to_bf16_rne(p[jt][r]);
        }
    __syncthreads();

    // The contraction now runs over the queries.  Wavefront w owns key tiles w, w+4, ...:
    // D[feature 4g + r][key il] = sum_i Q^T[feature][i] dS^T[key][i]  (dK), dO^T, P^T (dV)
#pragma unroll
    for (int u = 0; u < NT / 4; u++) {
        const int jt = w + 4 * u;
        u32x4 sb[NQS], pb[NQS];
#pragma unroll
        for (int s = 0; s < NQS; s++) {
            sb[s] = *reinterpret_cast<const u32x4 *>(St + (jt * 16 + il) * QS + 32 * s + 8 * g);
            pb[s] = *reinterpret_cast<const u32x4 *>(Pt + (jt * 16 + il) * QS + 32 * s + 8 * g);
        }
        floatx4_t ak[ND], av[ND];
#pragma unroll
        for (int dt = 0; dt < ND; dt++) {
            ak[dt] = floatx4_t{ 0, 0, 0, 0 };
            av[dt] = floatx4_t{ 0, 0, 0, 0 };
#pragma unroll
            for (int s = 0; s < NQS; s++) {
                ak[dt] = mfma_bf16(*reinterpret_cast<const u32x4 *>(Qt + tr_off<QS>(dt * 16 + il, 4 * s + g)), sb[s], ak[dt]);
                av[dt] = mfma_bf16(*reinterpret_cast<const u32x4 *>(Ot + tr_off<QS>(dt * 16 + il, 4 * s + g)), pb[s], av[dt]);
            }
        }
        const int j = jt * 16 + il;
        if (j < a.K) {
            const bool mem = j < a.M;
            const int64_t o = a.ldkv * (b + (int64_t)a.B * (mem ? j : j - a.M)) + (int64_t)h * DK + 4 * g;
            float NCHIP_GLOBAL *dst = as_global(mem ? a.dkvm : a.dkv) + o;
            uint16_t *d16 = mem ? a.dkvm16 : a.dkv16;
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(dst + dt * 16) = ak[dt];
                *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(dst + (int64_t)a.H * DK + dt * 16) = av[dt];
                if (d16) {
                    *reinterpret_cast<u32x2 NCHIP_GLOBAL *>(as_global(d16) + o + dt * 16) =
                        u32x2{ pack_bf16(ak[dt][0], ak[dt][1]), pack_bf16(ak[dt][2], ak[dt][3]) };
                    *reinterpret_cast<u32x2 NCHIP_GLOBAL *>(as_global(d16) + o + (int64_t)a.H * DK + dt * 16) =
                        u32x2{ pack_bf16(av[dt][0], av[dt][1]), pack_bf16(av[dt][2], av[dt][3]) };
                }
            }
        }
    }
    // dw_r partial of this (stream, head): D[feature 4g + r][position il] = Q^T dRel^T
    if (has_w) {
        float NCHIP_GLOBAL *dwz = as_global(a.dwp) + ((int64_t)b * a.H + h) * a.d_pos * DK;
#pragma unroll
        for (int u = 0; u < NT / 4; u++) {
            const int pt = w + 4 * u;
            u32x4 rb[NQS];
#pragma unroll
            for (int s = 0; s < NQS; s++) rb[s] = *reinterpret_cast<const u32x4 *>(Rt + (pt * 16 + il) * QS + 32 * s + 8 * g);
            const int pp = pt * 16 + il;
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
                for (int s = 0; s < NQS; s++)
                    acc = mfma_bf16(*reinterpret_cast<const u32x4 *>(Qt + tr_off<QS>(dt * 16 + il, 4 * s + g)), rb[s], acc);
                if (pp < a.d_pos) *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(dwz + (int64_t)pp * DK + dt * 16 + 4 * g) = acc;
            }
        }
    }
    // db_r partial: row K-1-delta collects the diagonal delta of dS (from dS^T: the bf16 values
    // the products above multiplied, summed in fp32 in query order)
    if (a.dbp) {
        for (int delta = t; delta < a.K; delta += 256) {
            float acc = 0.0f;
            for (int iq = 0; iq < a.T; iq++) {
                const int j = iq + a.M - delta;
                const bool on = j >= 0 && j < a.K;
                const float v = bf16_bits_to_f32(St[(on ? j : 0) * QS + iq]);
                acc += on ? v : 0.0f;
            }
            as_global(a.dbp)[((int64_t)b * a.H + h) * a.K + (a.K - 1 - delta)] = a.b_r_scale * acc;
        }
    }
}

template <int DK, int NT>
int launch_fwd(hipStream_t st, const Bf16AttnFwdArgs &a)
{
    constexpr int bytes = FwdLds<DK, NT>::bytes;
    static_assert(bytes <= 160 * 1024, "forward tiles exceed LDS");
    static const bool ok = hipFuncSetAttribute(reinterpret_cast<const void *>(relpos_attn_fwd_bf16<DK, NT>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess;
    if (!ok) return -2;
    hipLaunchKernelGGL((relpos_attn_fwd_bf16<DK, NT>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

template <int DK, int NT>
int launch_bwd(hipStream_t st, const Bf16AttnBwdArgs &a)
{
    constexpr int bytes = BwdLds<DK, NT>::bytes;
    static_assert(bytes <= 160 * 1024, "backward tiles exceed LDS");
    static const bool ok = hipFuncSetAttribute(reinterpret_cast<const void *>(relpos_attn_bwd_bf16<DK, NT>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess;
    if (!ok) return -2;
    hipLaunchKernelGGL((relpos_attn_bwd_bf16<DK, NT>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

} // namespace

// d_head 64 (keys and values), up to 64 queries, up to 256 keys / positions, K a multiple of 8
// (a lane's probabilities move as 8-byte units), every operand column 16-byte aligned
bool k_attn_bf16_shape_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr)
{
    return dk == 64 && dv == 64 && T >= 1 && T <= BT && K >= 1 && K <= 256 && K % 8 == 0 &&
           (!has_wr || (d_pos >= 1 && d_pos <= K));
}

int k_attn_bf16_fwd(hipStream_t st, const Bf16AttnFwdArgs &a)
{
    const int kmax = a.K > a.d_pos ? a.K : a.d_pos;
    if (kmax <= 128) return launch_fwd<64, 8>(st, a);
    return launch_fwd<64, 16>(st, a);
}

int k_attn_bf16_bwd(hipStream_t st, const Bf16AttnBwdArgs &a)
{
    const int kmax = a.K > a.d_pos ? a.K : a.d_pos;
    if (kmax <= 128) return launch_bwd<64, 8>(st, a);
    return launch_bwd<64, 16>(st, a);
}

// ---- raw entry points (include/nchip_kernels.h) -------------------------------------------
extern "C" int nchip_relpos_attn_fwd_bf16(void *stream, const uint16_t *q16, int64_t ldq, const uint16_t *kv16,
                                          const uint16_t *kvm16, int64_t ldkv, const uint16_t *w_r16, const float *b_r,
                                          float *out, uint16_t *out16, int64_t ldo, uint16_t *probs16, int H, int dk,
                                          int dv, int B, int T, int M, int d_pos, int attn_len, float b_r_scale)
{
    if (!q16 || !kv16 || !out || !probs16 || H < 1 || B < 1 || (M > 0 && !kvm16)) return -1;
    if (!k_attn_bf16_shape_ok(dk, dv, T, M + T, d_pos, w_r16 != nullptr) || ldq % 8 || ldkv % 8 || ldo % 4) return 1;
    Bf16AttnFwdArgs g;
    g.q = q16; g.kv = kv16; g.kvm = kvm16; g.w_r = w_r16; g.b_r = b_r; g.out = out; g.out16 = out16; g.probs = probs16;
    g.ldq = ldq; g.ldkv = ldkv; g.ldo = ldo;
    g.H = H; g.B = B; g.T = T; g.M = M; g.K = M + T; g.d_pos = w_r16 ? d_pos : 1; g.attn_len = attn_len;
    g.b_r_scale = b_r_scale; g.scale = 1.0f / sqrtf((float)dk);
    return k_attn_bf16_fwd((hipStream_t)stream, g);
}

extern "C" int nchip_relpos_attn_bwd_bf16(void *stream, const uint16_t *q16, int64_t ldq, const uint16_t *kv16,
                                          const uint16_t *kvm16, int64_t ldkv, const uint16_t *w_r16,
                                          const uint16_t *probs16, const uint16_t *dout16, int64_t ldo,
                                          float *dq, uint16_t *dq16, float *dkv, uint16_t *dkv16, float *dkvm,
                                          uint16_t *dkvm16, float *dw_r, float *db_r, int H, int dk, int dv, int B,
                                          int T, int M, int d_pos, int attn_len, float b_r_scale, float *scratch)
{
    if (!q16 || !kv16 || !probs16 || !dout16 || !dq || !dkv || H < 1 || B < 1 || (M > 0 && (!kvm16 || !dkvm)) ||
        ((dw_r || db_r) && !scratch) || (dw_r && !w_r16))
        return -1;
    if (!k_attn_bf16_shape_ok(dk, dv, T, M + T, d_pos, w_r16 != nullptr) || ldq % 8 || ldkv % 8 || ldo % 8) return 1;
    const int K = M + T, dp = w_r16 ? d_pos : 1;
    const int64_t n_w = dw_r ? (int64_t)dk * dp * H : 0, n_b = db_r ? (int64_t)K * H : 0;
    Bf16AttnBwdArgs g;
    g.q = q16; g.kv = kv16; g.kvm = kvm16; g.w_r = w_r16; g.probs = probs16; g.dout = dout16;
    g.dq = dq; g.dkv = dkv; g.dkvm = dkvm; g.dwp = dw_r ? scratch : nullptr; g.dbp = db_r ? scratch + n_w * B : nullptr;
    g.dq16 = dq16; g.dkv16 = dkv16; g.dkvm16 = dkvm16;
    g.ldq = ldq; g.ldkv = ldkv; g.ldo = ldo;
    g.H = H; g.B = B; g.T = T; g.M = M; g.K = K; g.d_pos = dp; g.attn_len = attn_len;
    g.b_r_scale = b_r_scale; g.scale = 1.0f / sqrtf((float)dk);
    int rc = k_attn_bf16_bwd((hipStream_t)stream, g);
    if (rc == 0 && (dw_r || db_r))
        rc = k_attn_param_grad_reduce((hipStream_t)stream, scratch, dw_r, n_w, scratch + n_w * B, db_r, n_b, B);
    return rc;
}
