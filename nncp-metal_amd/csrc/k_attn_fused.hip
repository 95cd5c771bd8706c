// Relative-position causal attention (nncp.c:722-800 and its gradient) as ONE
// kernel per direction for heads that fit in LDS: d_head 32 or 64, up to 64
// queries and 128 keys / relative positions.
//
// A workgroup (4 wavefronts) owns one (stream, head).  Q, the position vectors
// w_r[:, :, h], K and V of that head are staged once in LDS as [token][feature]
// rows of DK + 4 floats: with that stride both fragment shapes of
// v_mfma_f32_16x16x4_f32 read LDS at the 2-lanes-per-bank minimum
// ("row = token, k = feature": bank 4*il + g; "row = feature, k = token
// 4g + r": bank 16g + il).  Every tile is zero-filled to its full static size,
// so the compute phases are straight-line code without bounds branches: rows
// and columns outside the problem contribute exact zeros or are masked by
// selects, and only the global stores are guarded.  (Branches around MFMA
// groups make the compiler shuttle accumulators between AGPRs and VGPRs, which
// drains the matrix pipeline; skipping the causally dead key tiles would not
// shorten the workgroup, whose last wavefront sees every key.)
//
// Forward, wavefront w = query columns 16w..16w+15:
//   rel = w_r^T q -> per-wavefront LDS strip;  S = K^T q + shifted rel + bias
//   (1/sqrt(dk) folded into q), causal/window mask, all in registers;  softmax
//   over the keys with two xor-shuffles (a column lives in lanes l, l^16, l^32,
//   l^48);  O = V P with P fed to the MFMA straight from the score registers.
// Backward: dA = V^T dO and dS in registers, dq = K dS + w_r dRel (dRel = the
// rel-shift adjoint of dS, scattered into an LDS strip that replaces V); then
// P^T and dS^T are parked in LDS over K / w_r and the wavefronts switch to
// owning key tiles (dK = Q dS^T, dV = dO P^T) and position tiles
// (dw_r[b,h] = Q dRel^T).  Per-(stream, head) dw_r / db_r partials go to scratch
// and a second kernel sums them over streams in stream order.  No atomics.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include "k_internal.h"
#include "k_addrspace.h"

namespace {

typedef float floatx4_t __attribute__((ext_vector_type(4)));

constexpr int FA_TMAX = 64;     // queries per head
constexpr int FA_RSTRIDE = 131; // rel strip row: shifted reads and tile writes both <= 4 lanes per bank
constexpr int FA_PSTRIDE = 65;  // transposed P / dS tiles of the backward
constexpr int FA_NB = 256;      // bias row: K entries, zero up to the largest index a masked key can form

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

// Staging of a [ROWS][DK + 4] LDS tile from global rows of DK floats, split in
// two so that the loads of every tile are in flight before the first LDS store
// waits on one: fetch_rows only issues the float4 loads (rows >= rows_valid read
// a clamped, valid row), put_rows zeroes those rows and stores the whole tile.
// Nothing touches a loaded register between the two - a select right after the
// load would be scheduled early and wait for everything in flight.  src(row) is
// the row address; src(0) must be readable even when rows_valid is 0.
template <int DK, int ROWS, typename F>
__device__ __forceinline__ void fetch_rows(floatx4_t (&v)[ROWS * (DK / 4) / 256], int rows_valid, F src)
{
    constexpr int C4 = DK / 4;
#pragma unroll
    for (int it = 0; it < ROWS * C4 / 256; it++) {
        int idx = threadIdx.x + it * 256;
        int row = idx / C4, c = (idx % C4) * 4;
        int rc = row < rows_valid ? row : rows_valid - 1;
        v[it] = *as_global(reinterpret_cast<const floatx4_t *>(src(rc < 0 ? 0 : rc) + c));
    }
}

template <int DK, int ROWS>
__device__ __forceinline__ void put_rows(float *dst, const floatx4_t (&v)[ROWS * (DK / 4) / 256], int rows_valid)
{
    constexpr int RS = DK + 4, C4 = DK / 4;
#pragma unroll
    for (int it = 0; it < ROWS * C4 / 256; it++) {
        int idx = threadIdx.x + it * 256;
        int row = idx / C4, c = (idx % C4) * 4;
        *reinterpret_cast<floatx4_t *>(dst + row * RS + c) = row < rows_valid ? v[it] : floatx4_t{ 0, 0, 0, 0 };
    }
}

// a slice [it0, it1) of put_rows' stores, for callers that spread a tile's stores over a loop
template <int DK, int ROWS>
__device__ __forceinline__ void put_rows_part(float *dst, const floatx4_t (&v)[ROWS * (DK / 4) / 256], int rows_valid,
                                              int it0, int it1)
{
    constexpr int RS = DK + 4, C4 = DK / 4;
#pragma unroll
    for (int it = 0; it < ROWS * C4 / 256; it++) {
        if (it < it0 || it >= it1) continue;
        int idx = threadIdx.x + it * 256;
        int row = idx / C4, c = (idx % C4) * 4;
        *reinterpret_cast<floatx4_t *>(dst + row * RS + c) = row < rows_valid ? v[it] : floatx4_t{ 0, 0, 0, 0 };
    }
}

// Optional per-phase shader-clock stamps of one workgroup (debug builds only).
#ifdef NCHIP_ATTN_PHASE_CLOCKS
__device__ long long *g_phase_clk = nullptr;
#define PHASE_MARK(k)                                                                          \
    do {                                                                                       \
        if (g_phase_clk && blockIdx.x == 0 && (threadIdx.x & 63) == 0)                         \
            g_phase_clk[(threadIdx.x >> 6) * 16 + (k)] = clock64();                            \
    } while (0)
#else
#define PHASE_MARK(k) do { } while (0)
#endif

// Keeps the LDS reads of the next tile ahead of the MFMAs of the current one:
// without the fence the scheduler sinks each read next to its use and every
// MFMA pair then waits a full LDS round trip.
#define PIPELINE_FENCE() __builtin_amdgcn_sched_barrier(0)

// A operands of one 16-row tile for a DK-deep contraction (row = il, k-slot g)
template <int NS>
__device__ __forceinline__ void load_afrag(float (&f)[NS], const float *row_g)
{
#pragma unroll
    for (int s = 0; s < NS; s++) f[s] = row_g[4 * s];
}

// A operands of 4 k-steps (tokens tile*16 + 4g + r) x ND feature tiles
template <int ND, int RS>
__device__ __forceinline__ void load_tokfrag(float (&f)[ND][4], const float *base, int tile, int g, int il)
{
#pragma unroll
    for (int dt = 0; dt < ND; dt++)
#pragma unroll
        for (int r = 0; r < 4; r++) f[dt][r] = base[(tile * 16 + 4 * g + r) * RS + dt * 16 + il];
}

// NT = key / position tiles of 16 (4: up to 64 keys, 8: up to 128)
template <int DK, int NT>
struct FwdLayout {
    static constexpr int RS = DK + 4, KR = NT * 16;
    static constexpr int q = 0, w = q + FA_TMAX * RS, k = w + KR * RS, v = k + KR * RS,
                         r = v + KR * RS, b = r + 4 * 16 * FA_RSTRIDE, floats = b + FA_NB;
};

// VEC: K is a multiple of 4, so a lane's four probabilities of a key tile move as one 16-byte
// access; otherwise four clamped 4-byte accesses.  A compile-time choice keeps the loads and
// stores straight-line: with both forms behind a run-time branch the compiler waits for
// everything in flight (s_waitcnt vmcnt(0)) after each one.
template <int DK, int NT, bool VEC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void relpos_attn_fwd_fused(FusedAttnFwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using L = FwdLayout<DK, NT>;
    constexpr int RS = DK + 4, NS = DK / 4, ND = DK / 16, KR = NT * 16;
    float *Qs = lds + L::q, *Ws = lds + L::w, *Ks = lds + L::k, *Vs = lds + L::v;
    float *Rs = lds + L::r; // [4][16][FA_RSTRIDE]
    float *Bs = lds + L::b; // bias * b_r_scale / sqrt(dk), zero past K

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    // consecutive workgroups (one per XCD in turn) take consecutive streams, so
    // an XCD fetches whole token columns (every head of its streams)
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B;
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    const bool has_w = a.w_r != nullptr;
    PHASE_MARK(0);

    // All global loads are issued up front, in the order they are waited for (a wait for one
    // load is a wait for every older one): the bias row, Q and the position vectors for the
    // rel phase, then K and V, which arrive under that phase.
    const float bias_t = (a.b_r && t < a.K) ? as_global(a.b_r)[(int64_t)h * a.K + t] : 0.0f;
    // position vectors of this head (without them: no valid row, the clamped reads hit q)
    const float *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    floatx4_t vq[FA_TMAX * (DK / 4) / 256], vw[KR * (DK / 4) / 256], vk[KR * (DK / 4) / 256],
        vv[KR * (DK / 4) / 256];
    {
        auto kvrow = [&](int r) {
            return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                            : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
        };
        // single-query mode: every row of the Q tile is the one query; its column
        // q_only goes through exactly the arithmetic of a whole-segment call
        fetch_rows<DK, FA_TMAX>(vq, a.T, [&](int r) {
            return a.q + (int64_t)h * DK + a.ldq * (b + (a.q_only >= 0 ? 0 : (int64_t)a.B * r));
        });
        fetch_rows<DK, KR>(vw, n_w, [&](int r) { return w_base + (int64_t)r * DK; });
        fetch_rows<DK, KR>(vk, a.K, kvrow);
        fetch_rows<DK, KR>(vv, a.K, [&](int r) { return kvrow(r) + (int64_t)a.H * DK; });
    }
    if (t < FA_NB) Bs[t] = bias_t * (a.b_r_scale * a.scale);
    put_rows<DK, FA_TMAX>(Qs, vq, a.T);
    put_rows<DK, KR>(Ws, vw, n_w);
    __syncthreads();
    PHASE_MARK(1);

    // query fragments: B operand (k-slot g, column il) of every 4-wide k-step
    float qf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) qf[s] = Qs[i * RS + 4 * s + g] * a.scale; // 1/sqrt(dk) folded in

    float *Rw = Rs + (w * 16 + il) * FA_RSTRIDE; // this lane's column of rel
    {
        // two position tiles at a time: their accumulation chains alternate in the MFMA
        // pipe (a dependent MFMA waits about twice its own issue time for its predecessor)
        static_assert(NT % 2 == 0, "tiles are taken in pairs");
        float af[2][2][NS];
        load_afrag<NS>(af[0][0], Ws + il * RS + g);
        load_afrag<NS>(af[0][1], Ws + (16 + il) * RS + g);
#pragma unroll
        for (int pp = 0; pp < NT / 2; pp++) {
            if (pp + 1 < NT / 2) {
                load_afrag<NS>(af[(pp + 1) & 1][0], Ws + ((2 * pp + 2) * 16 + il) * RS + g);
                load_afrag<NS>(af[(pp + 1) & 1][1], Ws + ((2 * pp + 3) * 16 + il) * RS + g);
            }
            PIPELINE_FENCE();
            floatx4_t acc0 = { 0, 0, 0, 0 }, acc1 = { 0, 0, 0, 0 };
#pragma unroll
            for (int s = 0; s < NS; s++) {
                acc0 = mfma16(af[pp & 1][0][s], qf[s], acc0);
                acc1 = mfma16(af[pp & 1][1][s], qf[s], acc1);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                Rw[(2 * pp) * 16 + 4 * g + r] = acc0[r];
                Rw[(2 * pp + 1) * 16 + 4 * g + r] = acc1[r];
            }
            // K and V are parked in their own regions a slice per tile pair, under the MFMAs of
            // the next pair (they arrive during this phase; the key slices come first, in load order)
            constexpr int NV = KR * (DK / 4) / 256, PER = (2 * NV + NT / 2 - 1) / (NT / 2);
#pragma unroll
            for (int e = 0; e < PER; e++) {
                const int u = pp * PER + e; // 0 .. 2 NV - 1: first the key stores, then the value stores
                if (u < NV) put_rows_part<DK, KR>(Ks, vk, a.K, u, u + 1);
                else if (u < 2 * NV) put_rows_part<DK, KR>(Vs, vv, a.K, u - NV, u - NV + 1);
            }
        }
        wave_lds_sync();
    }
    __syncthreads();
    PHASE_MARK(2);

    float sc[NT][4];
    float mx = -INFINITY;
    {
        const int dbase = i + a.M - 4 * g;      // delta of key 4g of tile 0
        const int pbase = a.d_pos - 1 - dbase;  // its rel row before clamping
        const int pmax = a.d_pos - 1;
        const unsigned dlim = i < a.T ? (unsigned)a.attn_len : 0u;
        float af[2][2][NS]; // key tiles in pairs, as the position tiles above
        load_afrag<NS>(af[0][0], Ks + il * RS + g);
        load_afrag<NS>(af[0][1], Ks + (16 + il) * RS + g);
#pragma unroll
        for (int jp = 0; jp < NT / 2; jp++) {
            if (jp + 1 < NT / 2) {
                load_afrag<NS>(af[(jp + 1) & 1][0], Ks + ((2 * jp + 2) * 16 + il) * RS + g);
                load_afrag<NS>(af[(jp + 1) & 1][1], Ks + ((2 * jp + 3) * 16 + il) * RS + g);
            }
            PIPELINE_FENCE();
            // shifted rel and bias of the 4 keys of this lane: loaded unconditionally
            // (clamped / padded, always inside the arrays) and selected afterwards
            float relv[2][4], bv[2][4];
#pragma unroll
            for (int e = 0; e < 2; e++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int jt = 2 * jp + e;
                    int delta = dbase - (jt * 16 + r);
                    int pi = pbase + (jt * 16 + r); // d_pos-1-delta
                    pi = pi < 0 ? 0 : (pi > pmax ? pmax : pi);
                    relv[e][r] = Rw[pi];
                    bv[e][r] = Bs[(a.K - 1 - delta) & (FA_NB - 1)];
                }
            floatx4_t acc[2] = { { 0, 0, 0, 0 }, { 0, 0, 0, 0 } };
#pragma unroll
            for (int s = 0; s < NS; s++) {
                acc[0] = mfma16(af[jp & 1][0][s], qf[s], acc[0]);
                acc[1] = mfma16(af[jp & 1][1][s], qf[s], acc[1]);
            }
#pragma unroll
            for (int e = 0; e < 2; e++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    // key j < K is implied: delta >= 0 > i - T for a real column
                    const int jt = 2 * jp + e;
                    unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                    float v = delta < dlim ? acc[e][r] + relv[e][r] + bv[e][r] : -INFINITY;
                    sc[jt][r] = v;
                    mx = fmaxf(mx, v);
                }
        }
    }
    PHASE_MARK(3);
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    if (mx == -INFINITY) mx = 0.0f; // padding column
    float sum = 0.0f;
#pragma unroll
    for (int jt = 0; jt < NT; jt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float e = __expf(sc[jt][r] - mx); // exp(-inf) = 0 for masked keys
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
        float NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + i) * a.K;
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            int j0 = jt * 16 + 4 * g;
            if (VEC) {
                if (j0 < a.K) {
                    floatx4_t v = { sc[jt][0], sc[jt][1], sc[jt][2], sc[jt][3] };
                    *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(pc + j0) = v;
                }
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (j0 + r < a.K) pc[j0 + r] = sc[jt][r];
            }
        }
    }
    PHASE_MARK(4);

    // O = V P: the ND feature tiles are independent accumulation chains
    {
        floatx4_t acc[ND];
#pragma unroll
        for (int dt = 0; dt < ND; dt++) acc[dt] = floatx4_t{ 0, 0, 0, 0 };
        float vf[2][ND][4];
        load_tokfrag<ND, RS>(vf[0], Vs, 0, g, il);
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            if (jt + 1 < NT) load_tokfrag<ND, RS>(vf[(jt + 1) & 1], Vs, jt + 1, g, il);
            PIPELINE_FENCE();
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int dt = 0; dt < ND; dt++) acc[dt] = mfma16(vf[jt & 1][dt][r], sc[jt][r], acc[dt]);
        }
        if (a.q_only >= 0 ? i == a.q_only : i < a.T) {
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                float NCHIP_GLOBAL *o = as_global(a.out) + (int64_t)h * DK + dt * 16 + 4 * g +
                                        a.ldo * (b + (a.q_only >= 0 ? 0 : (int64_t)a.B * i));
                *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(o) = acc[dt];
            }
        }
    }
    PHASE_MARK(5);
}

template <int DK, int NT>
struct BwdLayout {
    static constexpr int RS = DK + 4, KR = NT * 16;
    static constexpr int kw_a = 2 * KR * RS, kw_b = 2 * KR * FA_PSTRIDE, kw = kw_a > kw_b ? kw_a : kw_b;
    static constexpr int v_a = KR * RS, v_b = FA_TMAX * FA_RSTRIDE, vsz = v_a > v_b ? v_a : v_b;
    static constexpr int q = 0, o = q + FA_TMAX * RS, k = o + FA_TMAX * RS, w = k + KR * RS,
                         v = k + kw, floats = v + vsz;
    static constexpr int pt = k, st = k + KR * FA_PSTRIDE; // over K / w_r once they are dead
    static constexpr int red = o;                          // db_r halves, over dO once it is dead
};

template <int DK, int NT, bool VEC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void relpos_attn_bwd_fused(FusedAttnBwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using L = BwdLayout<DK, NT>;
    constexpr int RS = DK + 4, NS = DK / 4, ND = DK / 16, KR = NT * 16, PS = FA_PSTRIDE;
    constexpr int NSQ = FA_TMAX / 4;
    float *Qs = lds + L::q, *Os = lds + L::o, *Ks = lds + L::k, *Ws = lds + L::w, *Vs = lds + L::v;
    float *Rs = Vs;           // [64][FA_RSTRIDE] dRel, once V is dead
    float *Pt = lds + L::pt;  // [KR][PS] P^T
    float *St = lds + L::st;  // [KR][PS] dS^T

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B; // as in the forward
    const bool has_w = a.w_r != nullptr;
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    PHASE_MARK(0);

    // every global load is issued up front, in the order the phases need the
    // tiles; each tile is parked in LDS just before its first use
    const float *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    floatx4_t vq[FA_TMAX * (DK / 4) / 256], vo[FA_TMAX * (DK / 4) / 256], vw[KR * (DK / 4) / 256],
        vk[KR * (DK / 4) / 256], vv[KR * (DK / 4) / 256];
    float p[NT][4], ds[NT][4];
    floatx4_t praw[NT];
    {
        auto kvrow = [&](int r) {
            return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                            : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
        };
        fetch_rows<DK, FA_TMAX>(vo, a.T, [&](int r) { return a.dout + (int64_t)h * DK + a.ldo * (b + (int64_t)a.B * r); });
        fetch_rows<DK, KR>(vv, a.K, [&](int r) { return kvrow(r) + (int64_t)a.H * DK; });
        const float NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + (i < a.T ? i : 0)) * a.K;
#pragma unroll
        for (int jt = 0; jt < NT; jt++) { // unconditional loads from clamped addresses; masked at first use
            int j0 = jt * 16 + 4 * g;
            if (VEC) {
                praw[jt] = *reinterpret_cast<const floatx4_t NCHIP_GLOBAL *>(pc + (j0 < a.K ? j0 : 0));
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) praw[jt][r] = pc[j0 + r < a.K ? j0 + r : 0];
            }
        }
        fetch_rows<DK, KR>(vk, a.K, kvrow);
        fetch_rows<DK, KR>(vw, n_w, [&](int r) { return w_base + (int64_t)r * DK; });
        fetch_rows<DK, FA_TMAX>(vq, a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
    }
    put_rows<DK, FA_TMAX>(Os, vo, a.T);
    put_rows<DK, KR>(Vs, vv, a.K);
    __syncthreads();
    PHASE_MARK(1);

    // dA = V^T dO, then dS = P (dA - colsum(P dA)) / sqrt(dk)
    {
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                p[jt][r] = (i < a.T && jt * 16 + 4 * g + r < a.K) ? praw[jt][r] : 0.0f;
        float dof[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) dof[s] = Os[i * RS + 4 * s + g];
        float af[2][2][NS]; // key tiles in pairs: two accumulation chains alternate in the MFMA pipe
        load_afrag<NS>(af[0][0], Vs + il * RS + g);
        load_afrag<NS>(af[0][1], Vs + (16 + il) * RS + g);
        float dot = 0.0f;
#pragma unroll
        for (int jp = 0; jp < NT / 2; jp++) {
            if (jp + 1 < NT / 2) {
                load_afrag<NS>(af[(jp + 1) & 1][0], Vs + ((2 * jp + 2) * 16 + il) * RS + g);
                load_afrag<NS>(af[(jp + 1) & 1][1], Vs + ((2 * jp + 3) * 16 + il) * RS + g);
            }
            PIPELINE_FENCE();
            floatx4_t acc[2] = { { 0, 0, 0, 0 }, { 0, 0, 0, 0 } };
#pragma unroll
            for (int s = 0; s < NS; s++) {
                acc[0] = mfma16(af[jp & 1][0][s], dof[s], acc[0]);
                acc[1] = mfma16(af[jp & 1][1][s], dof[s], acc[1]);
            }
#pragma unroll
            for (int e = 0; e < 2; e++)
#pragma unroll
                for (int r = 0; r < 4; r++) { // (the sum keeps its key order)
                    ds[2 * jp + e][r] = acc[e][r];
                    dot += p[2 * jp + e][r] * acc[e][r];
                }
        }
        dot += __shfl_xor(dot, 16, 64);
        dot += __shfl_xor(dot, 32, 64);
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
#pragma unroll
            for (int r = 0; r < 4; r++) ds[jt][r] = p[jt][r] * (ds[jt][r] - dot) * a.scale; // masked: p = 0
    }
    PHASE_MARK(2);
    put_rows<DK, KR>(Ks, vk, a.K);
    put_rows<DK, KR>(Ws, vw, n_w);
    put_rows<DK, FA_TMAX>(Qs, vq, a.T);
    __syncthreads(); // K, w_r, Q visible; every wavefront is done with V: its space becomes the dRel strip
    PHASE_MARK(3);

    float *Rw = Rs + i * FA_RSTRIDE;
    {
        // dRel[pi(delta), i] = sum of dS over the keys that read that row
        for (int pp = g; pp < KR; pp += 4) Rw[pp] = 0.0f;
        wave_lds_sync();
        const int dbase = i + a.M - 4 * g, pbase = a.d_pos - 1 - dbase;
        const unsigned dlim = (i < a.T && has_w) ? (unsigned)a.attn_len : 0u;
        float acc0 = 0.0f;
#pragma unroll
        for (int jt = 0; jt < NT; jt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                int pi = pbase + (jt * 16 + r);
                // rows >= 1 receive exactly one key; row 0 collects the far keys;
                // masked keys go to a dump slot past the strip (never read)
                const bool on = delta < dlim;
                Rw[(on && pi >= 1) ? pi : FA_RSTRIDE - 1] = ds[jt][r];
                acc0 += (on && pi < 1) ? ds[jt][r] : 0.0f;
            }
        acc0 += __shfl_xor(acc0, 16, 64);
        acc0 += __shfl_xor(acc0, 32, 64);
        if (g == 0) Rw[0] = acc0;
        wave_lds_sync();
    }
    // dq = K dS + w_r dRel: ND independent accumulation chains
    {
        floatx4_t dqa[ND];
#pragma unroll
        for (int dt = 0; dt < ND; dt++) dqa[dt] = floatx4_t{ 0, 0, 0, 0 };
        float kf[2][ND][4], rf[2][4];
        load_tokfrag<ND, RS>(kf[0], Ks, 0, g, il);
#pragma unroll
        for (int jt = 0; jt < NT; jt++) {
            if (jt + 1 < NT) load_tokfrag<ND, RS>(kf[(jt + 1) & 1], Ks, jt + 1, g, il);
            else {
                load_tokfrag<ND, RS>(kf[(jt + 1) & 1], Ws, 0, g, il);
#pragma unroll
                for (int r = 0; r < 4; r++) rf[(jt + 1) & 1][r] = Rw[4 * g + r];
            }
            PIPELINE_FENCE();
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int dt = 0; dt < ND; dt++) dqa[dt] = mfma16(kf[jt & 1][dt][r], ds[jt][r], dqa[dt]);
        }
#pragma unroll
        for (int pt = 0; pt < NT; pt++) {
            constexpr int o = NT & 1; // buffer parity continues from the key loop
            if (pt + 1 < NT) {
                load_tokfrag<ND, RS>(kf[(pt + 1 + o) & 1], Ws, pt + 1, g, il);
#pragma unroll
                for (int r = 0; r < 4; r++) rf[(pt + 1 + o) & 1][r] = Rw[(pt + 1) * 16 + 4 * g + r];
            }
            PIPELINE_FENCE();
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int dt = 0; dt < ND; dt++)
                    dqa[dt] = mfma16(kf[(pt + o) & 1][dt][r], rf[(pt + o) & 1][r], dqa[dt]);
        }
        if (i < a.T) {
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                float *o = a.dq + (int64_t)h * DK + dt * 16 + 4 * g + a.ldq * (b + (int64_t)a.B * i);
                *reinterpret_cast<floatx4_t *>(o) = dqa[dt];
            }
        }
    }
    PHASE_MARK(4);
    __syncthreads(); // K and w_r are dead: park P^T and dS^T over them
#pragma unroll
    for (int jt = 0; jt < NT; jt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            int j = jt * 16 + 4 * g + r;
            Pt[j * PS + i] = p[jt][r];
            St[j * PS + i] = ds[jt][r];
        }
    __syncthreads();
    PHASE_MARK(5);

    // the contraction now runs over the query index; k-slot g of step s is
    // query 16*(s/4) + 4g + s%4, which keeps the Q / dO reads conflict-free
    auto load_qd = [&](float (&f)[ND], const float *base, int s) {
        int iq = 16 * (s >> 2) + 4 * g + (s & 3);
#pragma unroll
        for (int dt = 0; dt < ND; dt++) f[dt] = base[iq * RS + dt * 16 + il];
    };
    // dK = Q dS^T, dV = dO P^T: wavefront w owns key tiles w, w+4, ...
#pragma unroll
    for (int u = 0; u < NT / 4; u++) {
        const int jt = w + 4 * u;
        float sb[NSQ], pb[NSQ];
#pragma unroll
        for (int s = 0; s < NSQ; s++) {
            int iq = 16 * (s >> 2) + 4 * g + (s & 3);
            sb[s] = St[(jt * 16 + il) * PS + iq];
            pb[s] = Pt[(jt * 16 + il) * PS + iq];
        }
        floatx4_t ak[ND], av[ND];
#pragma unroll
        for (int dt = 0; dt < ND; dt++) { ak[dt] = floatx4_t{ 0, 0, 0, 0 }; av[dt] = floatx4_t{ 0, 0, 0, 0 }; }
        float qa[2][ND], oa[2][ND];
        load_qd(qa[0], Qs, 0);
        load_qd(oa[0], Os, 0);
#pragma unroll
        for (int s = 0; s < NSQ; s++) {
            if (s + 1 < NSQ) { load_qd(qa[(s + 1) & 1], Qs, s + 1); load_qd(oa[(s + 1) & 1], Os, s + 1); }
            PIPELINE_FENCE();
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                ak[dt] = mfma16(qa[s & 1][dt], sb[s], ak[dt]);
                av[dt] = mfma16(oa[s & 1][dt], pb[s], av[dt]);
            }
        }
        const int j = jt * 16 + il;
        if (j < a.K) {
            float *dst = (j < a.M ? a.dkvm + a.ldkv * (b + (int64_t)a.B * j)
                                  : a.dkv + a.ldkv * (b + (int64_t)a.B * (j - a.M))) + (int64_t)h * DK;
#pragma unroll
            for (int dt = 0; dt < ND; dt++) {
                *reinterpret_cast<floatx4_t *>(dst + dt * 16 + 4 * g) = ak[dt];
                *reinterpret_cast<floatx4_t *>(dst + (int64_t)a.H * DK + dt * 16 + 4 * g) = av[dt];
            }
        }
    }
    PHASE_MARK(6);
    // dw_r partial of this (stream, head): Q dRel^T, wavefront w owns position tiles w, w+4, ...
    if (has_w) {
        float *dwz = a.dwp + ((int64_t)b * a.H + h) * a.d_pos * DK;
#pragma unroll
        for (int u = 0; u < NT / 4; u++) {
            const int pt = w + 4 * u;
            float rb[NSQ];
#pragma unroll
            for (int s = 0; s < NSQ; s++) {
                int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                rb[s] = Rs[iq * FA_RSTRIDE + pt * 16 + il];
            }
            floatx4_t acc[ND];
#pragma unroll
            for (int dt = 0; dt < ND; dt++) acc[dt] = floatx4_t{ 0, 0, 0, 0 };
            float qa[2][ND];
            load_qd(qa[0], Qs, 0);
#pragma unroll
            for (int s = 0; s < NSQ; s++) {
                if (s + 1 < NSQ) load_qd(qa[(s + 1) & 1], Qs, s + 1);
                PIPELINE_FENCE();
#pragma unroll
                for (int dt = 0; dt < ND; dt++) acc[dt] = mfma16(qa[s & 1][dt], rb[s], acc[dt]);
            }
            const int pp = pt * 16 + il;
            if (pp < a.d_pos) {
#pragma unroll
                for (int dt = 0; dt < ND; dt++)
                    *reinterpret_cast<floatx4_t *>(dwz + (int64_t)pp * DK + dt * 16 + 4 * g) = acc[dt];
            }
        }
    }
    PHASE_MARK(7);
    // db_r partial: row K-1-delta collects the diagonal delta of dS.  Threads
    // t and t+128 sum the two halves of the query range; the halves meet in LDS
    // (over dO, dead once every wavefront has left the dK/dV phase).
    if (a.dbp) {
        __syncthreads();
        float *red = lds + L::red;
        const int delta = t & 127, half = t >> 7;
        float acc = 0.0f;
        if (delta < a.K) {
#pragma unroll 8
            for (int q8 = 0; q8 < FA_TMAX / 2; q8++) {
                int iq = half * (FA_TMAX / 2) + q8;
                int j = iq + a.M - delta;
                bool on = iq < a.T && j >= 0 && j < a.K;
                float v = St[(on ? j : 0) * PS + iq];
                acc += on ? v : 0.0f;
            }
        }
        if (half) red[delta] = acc;
        __syncthreads();
        if (!half && delta < a.K)
            a.dbp[((int64_t)b * a.H + h) * a.K + (a.K - 1 - delta)] = a.b_r_scale * (acc + red[delta]);
    }
    PHASE_MARK(8);
}

// dw_r (n_w) and db_r (n_b) = sums over the B per-stream partials, in stream order
__global__ __launch_bounds__(256) void attn_param_grad_reduce(const float *dwp, float *dw, int64_t n_w,
                                                              const float *dbp, float *db, int64_t n_b, int B)
{
    int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const float *src;
    float *dst;
    int64_t n;
    if (e < n_w) { src = dwp + e; dst = dw + e; n = n_w; }
    else if (e < n_w + n_b) { src = dbp + (e - n_w); dst = db + (e - n_w); n = n_b; }
    else return;
    // the partials are added in stream order; eight loads at a time are in flight (added one
    // after the other as they are: a loop of dependent load-and-add pays a memory round trip per stream)
    float acc = 0.0f;
    int b = 0;
    for (; b + 8 <= B; b += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = src[(int64_t)(b + u) * n];
#pragma unroll
        for (int u = 0; u < 8; u++) acc += v[u];
    }
    for (; b < B; b++) acc += src[(int64_t)b * n];
    *dst = acc;
}

} // namespace

int k_attn_param_grad_reduce(hipStream_t st, const float *dwp, float *dw, int64_t n_w,
                             const float *dbp, float *db, int64_t n_b, int B)
{
    if (n_w + n_b <= 0) return 0;
    hipLaunchKernelGGL(attn_param_grad_reduce, dim3((unsigned)((n_w + n_b + 255) / 256)), dim3(256), 0, st,
                       dwp, dw, n_w, dbp, db, n_b, B);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

namespace {

// ---- more than 128 keys: the same arithmetic with the key / position axis in chunks ------
// Up to 320 keys and relative positions (NTT 16-key tiles, a multiple of 4).  Q, the rel
// strips and the bias row stay in LDS for the whole kernel; w_r, K and V pass through ONE
// staging tile of 128 rows, chunk after chunk (global -> registers two chunks ahead ->
// LDS), two barriers per chunk.  A column's scores for all keys live in registers
// (NTT x 4 per lane), so the softmax is the one-pass softmax of the kernels above: maximum
// and sum over all keys, no running rescale.
template <int NTT>
struct TiledDims {
    static_assert(NTT % 4 == 0 && NTT > 8 && NTT <= 20, "12, 16 or 20 key tiles");
    static constexpr int NCH = (NTT + 7) / 8;       // chunks of up to 8 tiles
    static constexpr int KP = NTT * 16;             // padded key / position count
    static constexpr int RST = KP + 3;              // rel strip row
    static constexpr int NB = 1024;                 // bias row incl. every index a masked key can form
    static constexpr int tiles_of(int c) { return NTT - 8 * c < 8 ? NTT - 8 * c : 8; }
};

template <int DK, int NTT>
struct FwdTiledLayout {
    using D = TiledDims<NTT>;
    static constexpr int RS = DK + 4;
    static constexpr int q = 0, st = q + FA_TMAX * RS, r = st + 128 * RS, b = r + 4 * 16 * D::RST,
                         floats = b + D::NB;
};

template <int DK, int NTT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void relpos_attn_fwd_tiled(FusedAttnFwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using L = FwdTiledLayout<DK, NTT>;
    using D = TiledDims<NTT>;
    constexpr int RS = DK + 4, NS = DK / 4, ND = DK / 16, NCH = D::NCH, RST = D::RST, NI = 3 * NCH;
    float *Qs = lds + L::q, *Ss = lds + L::st, *Rs = lds + L::r, *Bs = lds + L::b;

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B;
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    const bool has_w = a.w_r != nullptr;
    const float *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    auto kvrow = [&](int r) {
        return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                        : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
    };
    // staging items in the order they are used: position chunks, key chunks, value chunks
    floatx4_t vq[FA_TMAX * (DK / 4) / 256], vs[2][128 * (DK / 4) / 256];
    auto rows_of = [&](int item) { // valid rows of the item's chunk
        const int c = item % NCH, total = item < NCH ? n_w : a.K;
        const int left = total - 128 * c;
        return left < 0 ? 0 : (left > 128 ? 128 : left);
    };
    auto fetch = [&](int item, floatx4_t (&v)[128 * (DK / 4) / 256]) {
        const int c = item % NCH, kind = item / NCH, nv = rows_of(item);
        if (kind == 0) fetch_rows<DK, 128>(v, nv, [&](int r) { return w_base + (int64_t)(nv ? r + 128 * c : 0) * DK; });
        else if (kind == 1) fetch_rows<DK, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0); });
        else fetch_rows<DK, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0) + (int64_t)a.H * DK; });
    };
    for (int e = t; e < D::NB; e += 256)
        Bs[e] = (a.b_r && e < a.K) ? as_global(a.b_r)[(int64_t)h * a.K + e] * (a.b_r_scale * a.scale) : 0.0f;
    fetch_rows<DK, FA_TMAX>(vq, a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
    fetch(0, vs[0]);
    fetch(1, vs[1]);
    put_rows<DK, FA_TMAX>(Qs, vq, a.T);

    float qf[NS];
    float *Rw = Rs + (w * 16 + il) * RST; // this lane's column of rel
    float sc[NTT][4];
    float mx = -INFINITY;
    floatx4_t oacc[ND];
#pragma unroll
    for (int dt = 0; dt < ND; dt++) oacc[dt] = floatx4_t{ 0, 0, 0, 0 };
    const int dbase = i + a.M - 4 * g;      // delta of key 4g of tile 0
    const int pbase = a.d_pos - 1 - dbase;  // its rel row before clamping
    const int pmax = a.d_pos - 1;
    const unsigned dlim = i < a.T ? (unsigned)a.attn_len : 0u;

#pragma unroll
    for (int item = 0; item < NI; item++) {
        const int c = item % NCH, kind = item / NCH;
        constexpr int dummy = 0; (void)dummy;
        if (item > 0) __syncthreads(); // every wavefront has left the staging tile
        put_rows<DK, 128>(Ss, vs[item & 1], rows_of(item));
        if (item + 2 < NI) fetch(item + 2, vs[item & 1]);
        __syncthreads();
        if (item == 0) {
#pragma unroll
            for (int s = 0; s < NS; s++) qf[s] = Qs[i * RS + 4 * s + g] * a.scale; // 1/sqrt(dk) folded in
        }
        const int nt = D::tiles_of(c);
        if (kind == 0) {
            // rel = w_r^T q for the positions of this chunk -> strip
            float af[2][NS];
            load_afrag<NS>(af[0], Ss + il * RS + g);
#pragma unroll
            for (int pt = 0; pt < 8; pt++) {
                if (pt >= nt) break;
                if (pt + 1 < nt) load_afrag<NS>(af[(pt + 1) & 1], Ss + ((pt + 1) * 16 + il) * RS + g);
                PIPELINE_FENCE();
                floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
                for (int s = 0; s < NS; s++) acc = mfma16(af[pt & 1][s], qf[s], acc);
#pragma unroll
                for (int r = 0; r < 4; r++) Rw[(8 * c + pt) * 16 + 4 * g + r] = acc[r];
            }
            if (c == NCH - 1) wave_lds_sync();
        } else if (kind == 1) {
            float af[2][NS];
            load_afrag<NS>(af[0], Ss + il * RS + g);
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) load_afrag<NS>(af[(jl + 1) & 1], Ss + ((jl + 1) * 16 + il) * RS + g);
                PIPELINE_FENCE();
                float relv[4], bv[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    int delta = dbase - (jt * 16 + r);
                    int pi = pbase + (jt * 16 + r); // d_pos-1-delta
                    pi = pi < 0 ? 0 : (pi > pmax ? pmax : pi);
                    relv[r] = Rw[pi];
                    bv[r] = Bs[(a.K - 1 - delta) & (D::NB - 1)];
                }
                floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
                for (int s = 0; s < NS; s++) acc = mfma16(af[jl & 1][s], qf[s], acc);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                    float v = delta < dlim ? acc[r] + relv[r] + bv[r] : -INFINITY;
                    sc[jt][r] = v;
                    mx = fmaxf(mx, v);
                }
            }
            if (c == NCH - 1) {
                // softmax over all keys of the column (lanes l, l^16, l^32, l^48 share it)
                mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                if (mx == -INFINITY) mx = 0.0f; // padding column
                float sum = 0.0f;
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        float e = __expf(sc[jt][r] - mx); // exp(-inf) = 0 for masked keys
                        sc[jt][r] = e;
                        sum += e;
                    }
                sum += __shfl_xor(sum, 16, 64);
                sum += __shfl_xor(sum, 32, 64);
                float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) sc[jt][r] *= inv;
                if (a.probs && i < a.T) {
                    float NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + i) * a.K;
#pragma unroll
                    for (int jt = 0; jt < NTT; jt++) {
                        int j0 = jt * 16 + 4 * g;
                        if (j0 < a.K) { // K is a multiple of 4: whole quads
                            floatx4_t v = { sc[jt][0], sc[jt][1], sc[jt][2], sc[jt][3] };
                            *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(pc + j0) = v;
                        }
                    }
                }
            }
        } else {
            // O += V P over the keys of this chunk
            float vf[2][ND][4];
            load_tokfrag<ND, RS>(vf[0], Ss, 0, g, il);
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) load_tokfrag<ND, RS>(vf[(jl + 1) & 1], Ss, jl + 1, g, il);
                PIPELINE_FENCE();
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int dt = 0; dt < ND; dt++) oacc[dt] = mfma16(vf[jl & 1][dt][r], sc[jt][r], oacc[dt]);
            }
        }
    }
    if (i < a.T) {
#pragma unroll
        for (int dt = 0; dt < ND; dt++) {
            float NCHIP_GLOBAL *o = as_global(a.out) + (int64_t)h * DK + dt * 16 + 4 * g + a.ldo * (b + (int64_t)a.B * i);
            *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(o) = oacc[dt];
        }
    }
}

template <int DK, int NTT>
struct BwdTiledLayout {
    using D = TiledDims<NTT>;
    static constexpr int RS = DK + 4;
    static_assert(2 * 64 * FA_PSTRIDE <= 128 * RS, "the transposed P / dS tiles of 64 keys fit in the staging tile");
    static constexpr int q = 0, o = q + FA_TMAX * RS, st = o + FA_TMAX * RS, r = st + 128 * RS,
                         floats = r + FA_TMAX * D::RST;
};

// Backward for more than 128 keys.  dO, Q and the dRel strip stay in LDS; V, K and w_r pass
// through the staging tile in chunks of 128 rows (dA, then dq), and P^T / dS^T are parked
// in the same tile 64 keys at a time for dK, dV and the db_r diagonals.  The probabilities
// and dS of a column for all keys live in registers.
template <int DK, int NTT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void relpos_attn_bwd_tiled(FusedAttnBwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using L = BwdTiledLayout<DK, NTT>;
    using D = TiledDims<NTT>;
    constexpr int RS = DK + 4, NS = DK / 4, ND = DK / 16, NCH = D::NCH, RST = D::RST, NI = 3 * NCH, PS = FA_PSTRIDE;
    constexpr int NSQ = FA_TMAX / 4, KP = D::KP;
    float *Qs = lds + L::q, *Os = lds + L::o, *Ss = lds + L::st, *Rs = lds + L::r;
    float *Pt = Ss, *St = Ss + 64 * PS; // [64 keys][PS] each

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B;
    const bool has_w = a.w_r != nullptr;
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    const float *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    auto kvrow = [&](int r) {
        return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                        : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
    };
    // staging items: value chunks (dA), key chunks (dq), position chunks (dq)
    floatx4_t vq[FA_TMAX * (DK / 4) / 256], vo[FA_TMAX * (DK / 4) / 256], vs[2][128 * (DK / 4) / 256];
    auto rows_of = [&](int item) {
        const int c = item % NCH, total = item < 2 * NCH ? a.K : n_w;
        const int left = total - 128 * c;
        return left < 0 ? 0 : (left > 128 ? 128 : left);
    };
    auto fetch = [&](int item, floatx4_t (&v)[128 * (DK / 4) / 256]) {
        const int c = item % NCH, kind = item / NCH, nv = rows_of(item);
        if (kind == 0) fetch_rows<DK, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0) + (int64_t)a.H * DK; });
        else if (kind == 1) fetch_rows<DK, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0); });
        else fetch_rows<DK, 128>(v, nv, [&](int r) { return w_base + (int64_t)(nv ? r + 128 * c : 0) * DK; });
    };
    float p[NTT][4], ds[NTT][4];
    fetch_rows<DK, FA_TMAX>(vo, a.T, [&](int r) { return a.dout + (int64_t)h * DK + a.ldo * (b + (int64_t)a.B * r); });
    fetch(0, vs[0]);
    {
        const float NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + (i < a.T ? i : 0)) * a.K;
#pragma unroll
        for (int jt = 0; jt < NTT; jt++) { // unconditional loads from clamped addresses; masked at first use
            int j0 = jt * 16 + 4 * g;
            floatx4_t v = *reinterpret_cast<const floatx4_t NCHIP_GLOBAL *>(pc + (j0 < a.K ? j0 : 0));
#pragma unroll
            for (int r = 0; r < 4; r++) p[jt][r] = v[r];
        }
    }
    fetch(1, vs[1]);
    fetch_rows<DK, FA_TMAX>(vq, a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
    put_rows<DK, FA_TMAX>(Os, vo, a.T);
    put_rows<DK, FA_TMAX>(Qs, vq, a.T);

    float dof[NS];
    float dot = 0.0f;
    float *Rw = Rs + i * RST;
    floatx4_t dqa[ND];
#pragma unroll
    for (int dt = 0; dt < ND; dt++) dqa[dt] = floatx4_t{ 0, 0, 0, 0 };

#pragma unroll
    for (int item = 0; item < NI; item++) {
        const int c = item % NCH, kind = item / NCH;
        if (item > 0) __syncthreads(); // every wavefront has left the staging tile
        put_rows<DK, 128>(Ss, vs[item & 1], rows_of(item));
        if (item + 2 < NI) fetch(item + 2, vs[item & 1]);
        __syncthreads();
        const int nt = D::tiles_of(c);
        if (kind == 0) {
            if (item == 0) {
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        p[jt][r] = (i < a.T && jt * 16 + 4 * g + r < a.K) ? p[jt][r] : 0.0f;
#pragma unroll
                for (int s = 0; s < NS; s++) dof[s] = Os[i * RS + 4 * s + g];
            }
            // dA = V^T dO for the keys of this chunk
            float af[2][NS];
            load_afrag<NS>(af[0], Ss + il * RS + g);
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) load_afrag<NS>(af[(jl + 1) & 1], Ss + ((jl + 1) * 16 + il) * RS + g);
                PIPELINE_FENCE();
                floatx4_t acc = { 0, 0, 0, 0 };
#pragma unroll
                for (int s = 0; s < NS; s++) acc = mfma16(af[jl & 1][s], dof[s], acc);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    ds[jt][r] = acc[r];
                    dot += p[jt][r] * acc[r];
                }
            }
            if (c == NCH - 1) {
                // dS = P (dA - colsum(P dA)) / sqrt(dk), then its rel-shift adjoint into the strip
                dot += __shfl_xor(dot, 16, 64);
                dot += __shfl_xor(dot, 32, 64);
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) ds[jt][r] = p[jt][r] * (ds[jt][r] - dot) * a.scale; // masked: p = 0
                for (int pp = g; pp < KP; pp += 4) Rw[pp] = 0.0f;
                wave_lds_sync();
                const int dbase = i + a.M - 4 * g, pbase = a.d_pos - 1 - dbase;
                const unsigned dlim = (i < a.T && has_w) ? (unsigned)a.attn_len : 0u;
                float acc0 = 0.0f;
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                        int pi = pbase + (jt * 16 + r);
                        // rows >= 1 receive exactly one key; row 0 collects the far keys;
                        // masked keys go to a dump slot past the strip (never read)
                        const bool on = delta < dlim;
                        Rw[(on && pi >= 1) ? pi : RST - 1] = ds[jt][r];
                        acc0 += (on && pi < 1) ? ds[jt][r] : 0.0f;
                    }
                acc0 += __shfl_xor(acc0, 16, 64);
                acc0 += __shfl_xor(acc0, 32, 64);
                if (g == 0) Rw[0] = acc0;
                wave_lds_sync();
            }
        } else {
            // dq += K dS (kind 1) or w_r dRel (kind 2) over the rows of this chunk
            float kf[2][ND][4], rf[2][4];
            load_tokfrag<ND, RS>(kf[0], Ss, 0, g, il);
            if (kind == 2) {
#pragma unroll
                for (int r = 0; r < 4; r++) rf[0][r] = Rw[(8 * c) * 16 + 4 * g + r];
            }
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) {
                    load_tokfrag<ND, RS>(kf[(jl + 1) & 1], Ss, jl + 1, g, il);
                    if (kind == 2) {
#pragma unroll
                        for (int r = 0; r < 4; r++) rf[(jl + 1) & 1][r] = Rw[(jt + 1) * 16 + 4 * g + r];
                    }
                }
                PIPELINE_FENCE();
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int dt = 0; dt < ND; dt++)
                        dqa[dt] = mfma16(kf[jl & 1][dt][r], kind == 1 ? ds[jt][r] : rf[jl & 1][r], dqa[dt]);
            }
        }
    }
    if (i < a.T) {
#pragma unroll
        for (int dt = 0; dt < ND; dt++) {
            float *o = a.dq + (int64_t)h * DK + dt * 16 + 4 * g + a.ldq * (b + (int64_t)a.B * i);
            *reinterpret_cast<floatx4_t *>(o) = dqa[dt];
        }
    }

    // the contraction now runs over the query index; k-slot g of step s is
    // query 16*(s/4) + 4g + s%4, which keeps the Q / dO reads conflict-free
    auto load_qd = [&](float (&f)[ND], const float *base, int s) {
        int iq = 16 * (s >> 2) + 4 * g + (s & 3);
#pragma unroll
        for (int dt = 0; dt < ND; dt++) f[dt] = base[iq * RS + dt * 16 + il];
    };
    // dK = Q dS^T, dV = dO P^T, 64 keys at a time: wavefront w owns key tile 4*hc + w;
    // db_r: thread t sums the diagonals delta = t and t + 256 over the parked keys
    float dbacc[2] = { 0.0f, 0.0f };
#pragma unroll
    for (int hc = 0; hc < NTT / 4; hc++) {
        __syncthreads(); // the staging tile (or the previous 64 keys) is dead
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int jl = e * 16 + 4 * g + r;
                Pt[jl * PS + i] = p[4 * hc + e][r];
                St[jl * PS + i] = ds[4 * hc + e][r];
            }
        __syncthreads();
        {
            float sb[NSQ], pb[NSQ];
#pragma unroll
            for (int s = 0; s < NSQ; s++) {
                int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                sb[s] = St[(w * 16 + il) * PS + iq];
                pb[s] = Pt[(w * 16 + il) * PS + iq];
            }
            floatx4_t ak[ND], av[ND];
#pragma unroll
            for (int dt = 0; dt < ND; dt++) { ak[dt] = floatx4_t{ 0, 0, 0, 0 }; av[dt] = floatx4_t{ 0, 0, 0, 0 }; }
            float qa[2][ND], oa[2][ND];
            load_qd(qa[0], Qs, 0);
            load_qd(oa[0], Os, 0);
#pragma unroll
            for (int s = 0; s < NSQ; s++) {
                if (s + 1 < NSQ) { load_qd(qa[(s + 1) & 1], Qs, s + 1); load_qd(oa[(s + 1) & 1], Os, s + 1); }
                PIPELINE_FENCE();
#pragma unroll
                for (int dt = 0; dt < ND; dt++) {
                    ak[dt] = mfma16(qa[s & 1][dt], sb[s], ak[dt]);
                    av[dt] = mfma16(oa[s & 1][dt], pb[s], av[dt]);
                }
            }
            const int j = (4 * hc + w) * 16 + il;
            if (j < a.K) {
                float *dst = (j < a.M ? a.dkvm + a.ldkv * (b + (int64_t)a.B * j)
                                      : a.dkv + a.ldkv * (b + (int64_t)a.B * (j - a.M))) + (int64_t)h * DK;
#pragma unroll
                for (int dt = 0; dt < ND; dt++) {
                    *reinterpret_cast<floatx4_t *>(dst + dt * 16 + 4 * g) = ak[dt];
                    *reinterpret_cast<floatx4_t *>(dst + (int64_t)a.H * DK + dt * 16 + 4 * g) = av[dt];
                }
            }
        }
        if (a.dbp) {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int delta = t + 256 * u;
                // keys 64*hc .. 64*hc+63 of diagonal delta belong to queries lo .. lo+63
                const int lo = delta - a.M + 64 * hc;
                float acc = 0.0f;
#pragma unroll 8
                for (int q8 = 0; q8 < 64; q8++) {
                    const int iq = lo + q8;
                    const bool on = delta < a.K && iq >= 0 && iq < a.T && 64 * hc + q8 < a.K;
                    float v = St[(on ? q8 : 0) * PS + (on ? iq : 0)];
                    acc += on ? v : 0.0f;
                }
                dbacc[u] += acc;
            }
        }
    }
    // dw_r partial of this (stream, head): Q dRel^T, wavefront w owns position tiles w, w+4, ...
    if (has_w) {
        float *dwz = a.dwp + ((int64_t)b * a.H + h) * a.d_pos * DK;
#pragma unroll
        for (int u = 0; u < NTT / 4; u++) {
            const int pt = w + 4 * u;
            float rb[NSQ];
#pragma unroll
            for (int s = 0; s < NSQ; s++) {
                int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                rb[s] = Rs[iq * RST + pt * 16 + il];
            }
            floatx4_t acc[ND];
#pragma unroll
            for (int dt = 0; dt < ND; dt++) acc[dt] = floatx4_t{ 0, 0, 0, 0 };
            float qa[2][ND];
            load_qd(qa[0], Qs, 0);
#pragma unroll
            for (int s = 0; s < NSQ; s++) {
                if (s + 1 < NSQ) load_qd(qa[(s + 1) & 1], Qs, s + 1);
                PIPELINE_FENCE();
#pragma unroll
                for (int dt = 0; dt < ND; dt++) acc[dt] = mfma16(qa[s & 1][dt], rb[s], acc[dt]);
            }
            const int pp = pt * 16 + il;
            if (pp < a.d_pos) {
#pragma unroll
                for (int dt = 0; dt < ND; dt++)
                    *reinterpret_cast<floatx4_t *>(dwz + (int64_t)pp * DK + dt * 16 + 4 * g) = acc[dt];
            }
        }
    }
    if (a.dbp) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int delta = t + 256 * u;
            if (delta < a.K)
                a.dbp[((int64_t)b * a.H + h) * a.K + (a.K - 1 - delta)] = a.b_r_scale * dbacc[u];
        }
    }
}

// ---- heads of 128 features --------------------------------------------------------------
// The chunked kernels again with the feature axis in halves of 64 (DK = 64 NH): a staging
// tile holds 128 rows x 64 features, every chunk of w_r, K and V passes through it once per
// half, and only Q (forward) or dO (backward, until its fragments are in registers) is held
// at full width.  Contractions over the features (rel, scores, dA) chain through the halves:
// the accumulator of half 1 starts from the result of half 0, so a 128-deep sum is formed in
// the same order as one uninterrupted MFMA chain.  Products whose OUTPUT runs over the
// features (O, dq, dK, dV, dw_r) simply own one set of accumulators per half.  The backward
// fetches Q and dO again, one half at a time, for the key- and position-owned phase.
template <int NTT>
struct WideDims {
    static_assert(NTT % 4 == 0 && NTT >= 8 && NTT <= 20, "8, 12, 16 or 20 key tiles");
    static constexpr int NCH = (NTT + 7) / 8;       // chunks of up to 8 tiles
    static constexpr int KP = NTT * 16;             // padded key / position count
    static constexpr int RST = KP + 3;              // rel strip row
    static constexpr int NB = 1024;                 // bias row incl. every index a masked key can form
    static constexpr int tiles_of(int c) { return NTT - 8 * c < 8 ? NTT - 8 * c : 8; }
};

template <int NH, int NTT>
struct FwdWideLayout {
    using D = WideDims<NTT>;
    static constexpr int RSQ = 64 * NH + 4, RS = 68;
    static constexpr int q = 0, st = q + FA_TMAX * RSQ, r = st + 128 * RS, b = r + 4 * 16 * D::RST,
                         floats = b + D::NB;
};

template <int NH, int NTT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void relpos_attn_fwd_wide(FusedAttnFwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using L = FwdWideLayout<NH, NTT>;
    using D = WideDims<NTT>;
    constexpr int DK = 64 * NH, RSQ = L::RSQ, RS = L::RS, NS = 16, ND = 4, NCH = D::NCH, RST = D::RST,
                  NI = 3 * NCH * NH;
    float *Qs = lds + L::q, *Ss = lds + L::st, *Rs = lds + L::r, *Bs = lds + L::b;

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B;
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    const bool has_w = a.w_r != nullptr;
    const float *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    auto kvrow = [&](int r) {
        return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                        : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
    };
    // staging items in the order they are used: position chunks, key chunks, value chunks,
    // each chunk once per feature half
    floatx4_t vq[FA_TMAX * (DK / 4) / 256], vs[2][128 * 16 / 256];
    auto rows_of = [&](int item) { // valid rows of the item's chunk
        const int kind = item / (NCH * NH), c = (item / NH) % NCH, total = kind == 0 ? n_w : a.K;
        const int left = total - 128 * c;
        return left < 0 ? 0 : (left > 128 ? 128 : left);
    };
    auto fetch = [&](int item, floatx4_t (&v)[128 * 16 / 256]) {
        const int kind = item / (NCH * NH), c = (item / NH) % NCH, hf = item % NH, nv = rows_of(item);
        if (kind == 0) fetch_rows<64, 128>(v, nv, [&](int r) { return w_base + (int64_t)(nv ? r + 128 * c : 0) * DK + 64 * hf; });
        else if (kind == 1) fetch_rows<64, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0) + 64 * hf; });
        else fetch_rows<64, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0) + (int64_t)a.H * DK + 64 * hf; });
    };
    for (int e = t; e < D::NB; e += 256)
        Bs[e] = (a.b_r && e < a.K) ? as_global(a.b_r)[(int64_t)h * a.K + e] * (a.b_r_scale * a.scale) : 0.0f;
    fetch_rows<DK, FA_TMAX>(vq, a.T, [&](int r) { return a.q + (int64_t)h * DK + a.ldq * (b + (int64_t)a.B * r); });
    fetch(0, vs[0]);
    fetch(1, vs[1]);
    put_rows<DK, FA_TMAX>(Qs, vq, a.T);

    float qf[NH][NS];
    float *Rw = Rs + (w * 16 + il) * RST; // this lane's column of rel
    float sc[NTT][4];
    float mx = -INFINITY;
    floatx4_t oacc[NH * ND];
#pragma unroll
    for (int dt = 0; dt < NH * ND; dt++) oacc[dt] = floatx4_t{ 0, 0, 0, 0 };
    const int dbase = i + a.M - 4 * g;      // delta of key 4g of tile 0
    const int pbase = a.d_pos - 1 - dbase;  // its rel row before clamping
    const int pmax = a.d_pos - 1;
    const unsigned dlim = i < a.T ? (unsigned)a.attn_len : 0u;

#pragma unroll
    for (int item = 0; item < NI; item++) {
        const int kind = item / (NCH * NH), c = (item / NH) % NCH, hf = item % NH;
        if (item > 0) __syncthreads(); // every wavefront has left the staging tile
        put_rows<64, 128>(Ss, vs[item & 1], rows_of(item));
        if (item + 2 < NI) fetch(item + 2, vs[item & 1]);
        __syncthreads();
        if (item == 0) {
#pragma unroll
            for (int hh = 0; hh < NH; hh++)
#pragma unroll
                for (int s = 0; s < NS; s++) qf[hh][s] = Qs[i * RSQ + 64 * hh + 4 * s + g] * a.scale; // 1/sqrt(dk) folded in
        }
        const int nt = D::tiles_of(c);
        if (kind == 0) {
            // rel = w_r^T q for the positions of this chunk -> strip (half 1 continues half 0's sums)
            float af[2][NS];
            load_afrag<NS>(af[0], Ss + il * RS + g);
#pragma unroll
            for (int pt = 0; pt < 8; pt++) {
                if (pt >= nt) break;
                if (pt + 1 < nt) load_afrag<NS>(af[(pt + 1) & 1], Ss + ((pt + 1) * 16 + il) * RS + g);
                float *rw = Rw + (8 * c + pt) * 16 + 4 * g;
                floatx4_t acc = { 0, 0, 0, 0 };
                if (hf > 0) {
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[r] = rw[r]; // written by this lane in the half before
                }
                PIPELINE_FENCE();
#pragma unroll
                for (int s = 0; s < NS; s++) acc = mfma16(af[pt & 1][s], qf[hf][s], acc);
#pragma unroll
                for (int r = 0; r < 4; r++) rw[r] = acc[r];
            }
            if (c == NCH - 1 && hf == NH - 1) wave_lds_sync();
        } else if (kind == 1) {
            float af[2][NS];
            load_afrag<NS>(af[0], Ss + il * RS + g);
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) load_afrag<NS>(af[(jl + 1) & 1], Ss + ((jl + 1) * 16 + il) * RS + g);
                PIPELINE_FENCE();
                floatx4_t acc = { 0, 0, 0, 0 };
                if (hf > 0) {
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[r] = sc[jt][r];
                }
#pragma unroll
                for (int s = 0; s < NS; s++) acc = mfma16(af[jl & 1][s], qf[hf][s], acc);
                if (hf < NH - 1) {
#pragma unroll
                    for (int r = 0; r < 4; r++) sc[jt][r] = acc[r];
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                        int pi = pbase + (jt * 16 + r); // d_pos-1-delta
                        pi = pi < 0 ? 0 : (pi > pmax ? pmax : pi);
                        const float relv = Rw[pi];
                        const float bv = Bs[(a.K - 1 - (int)delta) & (D::NB - 1)];
                        float v = delta < dlim ? acc[r] + relv + bv : -INFINITY;
                        sc[jt][r] = v;
                        mx = fmaxf(mx, v);
                    }
                }
            }
            if (c == NCH - 1 && hf == NH - 1) {
                // softmax over all keys of the column (lanes l, l^16, l^32, l^48 share it)
                mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                if (mx == -INFINITY) mx = 0.0f; // padding column
                float sum = 0.0f;
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        float e = __expf(sc[jt][r] - mx); // exp(-inf) = 0 for masked keys
                        sc[jt][r] = e;
                        sum += e;
                    }
                sum += __shfl_xor(sum, 16, 64);
                sum += __shfl_xor(sum, 32, 64);
                float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) sc[jt][r] *= inv;
                if (a.probs && i < a.T) {
                    float NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + i) * a.K;
#pragma unroll
                    for (int jt = 0; jt < NTT; jt++) {
                        int j0 = jt * 16 + 4 * g;
                        if (j0 < a.K) { // K is a multiple of 4: whole quads
                            floatx4_t v = { sc[jt][0], sc[jt][1], sc[jt][2], sc[jt][3] };
                            *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(pc + j0) = v;
                        }
                    }
                }
            }
        } else {
            // O[:, half] += V[:, half] P over the keys of this chunk
            float vf[2][ND][4];
            load_tokfrag<ND, RS>(vf[0], Ss, 0, g, il);
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) load_tokfrag<ND, RS>(vf[(jl + 1) & 1], Ss, jl + 1, g, il);
                PIPELINE_FENCE();
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int dt = 0; dt < ND; dt++)
                        oacc[hf * ND + dt] = mfma16(vf[jl & 1][dt][r], sc[jt][r], oacc[hf * ND + dt]);
            }
        }
    }
    if (i < a.T) {
#pragma unroll
        for (int dt = 0; dt < NH * ND; dt++) {
            float NCHIP_GLOBAL *o = as_global(a.out) + (int64_t)h * DK + dt * 16 + 4 * g + a.ldo * (b + (int64_t)a.B * i);
            *reinterpret_cast<floatx4_t NCHIP_GLOBAL *>(o) = oacc[dt];
        }
    }
}

template <int NH, int NTT>
struct BwdWideLayout {
    using D = WideDims<NTT>;
    static constexpr int RSQ = 64 * NH + 4, RS = 68;
    // x: dO at full width until its fragments are in registers, then one half of Q and of dO
    static constexpr int xsz = FA_TMAX * RSQ > 2 * FA_TMAX * RS ? FA_TMAX * RSQ : 2 * FA_TMAX * RS;
    static_assert(2 * 64 * FA_PSTRIDE <= 128 * RS, "the transposed P / dS tiles of 64 keys fit in the staging tile");
    static constexpr int x = 0, st = x + xsz, r = st + 128 * RS, floats = r + FA_TMAX * D::RST;
};

template <int NH, int NTT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void relpos_attn_bwd_wide(FusedAttnBwdArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    using L = BwdWideLayout<NH, NTT>;
    using D = WideDims<NTT>;
    constexpr int DK = 64 * NH, RSQ = L::RSQ, RS = L::RS, NS = 16, ND = 4, NCH = D::NCH, RST = D::RST,
                  NI = 3 * NCH * NH, PS = FA_PSTRIDE;
    constexpr int NSQ = FA_TMAX / 4, KP = D::KP;
    float *Xs = lds + L::x, *Ss = lds + L::st, *Rs = lds + L::r;
    float *Qh = Xs, *Oh = Xs + FA_TMAX * RS; // [64 queries][RS] each, one feature half
    float *Pt = Ss, *St = Ss + 64 * PS;      // [64 keys][PS] each

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B;
    const bool has_w = a.w_r != nullptr;
    const int il = lane & 15, g = lane >> 4;
    const int i = 16 * w + il;
    const float *w_base = has_w ? a.w_r + (int64_t)h * a.d_pos * DK : a.q;
    const int n_w = has_w ? a.d_pos : 0;
    auto kvrow = [&](int r) {
        return (r < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * r)
                        : a.kv + a.ldkv * (b + (int64_t)a.B * (r - a.M))) + (int64_t)h * DK;
    };
    // staging items: value chunks (dA), key chunks (dq), position chunks (dq), once per half
    floatx4_t vo[FA_TMAX * (DK / 4) / 256], vs[2][128 * 16 / 256];
    auto rows_of = [&](int item) {
        const int kind = item / (NCH * NH), c = (item / NH) % NCH, total = kind < 2 ? a.K : n_w;
        const int left = total - 128 * c;
        return left < 0 ? 0 : (left > 128 ? 128 : left);
    };
    auto fetch = [&](int item, floatx4_t (&v)[128 * 16 / 256]) {
        const int kind = item / (NCH * NH), c = (item / NH) % NCH, hf = item % NH, nv = rows_of(item);
        if (kind == 0) fetch_rows<64, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0) + (int64_t)a.H * DK + 64 * hf; });
        else if (kind == 1) fetch_rows<64, 128>(v, nv, [&](int r) { return kvrow(nv ? r + 128 * c : 0) + 64 * hf; });
        else fetch_rows<64, 128>(v, nv, [&](int r) { return w_base + (int64_t)(nv ? r + 128 * c : 0) * DK + 64 * hf; });
    };
    float p[NTT][4], ds[NTT][4];
    fetch_rows<DK, FA_TMAX>(vo, a.T, [&](int r) { return a.dout + (int64_t)h * DK + a.ldo * (b + (int64_t)a.B * r); });
    fetch(0, vs[0]);
    {
        const float NCHIP_GLOBAL *pc = as_global(a.probs) + (((int64_t)b * a.H + h) * a.T + (i < a.T ? i : 0)) * a.K;
#pragma unroll
        for (int jt = 0; jt < NTT; jt++) { // unconditional loads from clamped addresses; masked at first use
            int j0 = jt * 16 + 4 * g;
            floatx4_t v = *reinterpret_cast<const floatx4_t NCHIP_GLOBAL *>(pc + (j0 < a.K ? j0 : 0));
#pragma unroll
            for (int r = 0; r < 4; r++) p[jt][r] = v[r];
        }
    }
    fetch(1, vs[1]);
    put_rows<DK, FA_TMAX>(Xs, vo, a.T);

    float dof[NH][NS];
    float dot = 0.0f;
    float *Rw = Rs + i * RST;
    floatx4_t dqa[NH * ND];
#pragma unroll
    for (int dt = 0; dt < NH * ND; dt++) dqa[dt] = floatx4_t{ 0, 0, 0, 0 };

#pragma unroll
    for (int item = 0; item < NI; item++) {
        const int kind = item / (NCH * NH), c = (item / NH) % NCH, hf = item % NH;
        if (item > 0) __syncthreads(); // every wavefront has left the staging tile
        put_rows<64, 128>(Ss, vs[item & 1], rows_of(item));
        if (item + 2 < NI) fetch(item + 2, vs[item & 1]);
        __syncthreads();
        const int nt = D::tiles_of(c);
        if (kind == 0) {
            if (item == 0) {
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        p[jt][r] = (i < a.T && jt * 16 + 4 * g + r < a.K) ? p[jt][r] : 0.0f;
#pragma unroll
                for (int hh = 0; hh < NH; hh++)
#pragma unroll
                    for (int s = 0; s < NS; s++) dof[hh][s] = Xs[i * RSQ + 64 * hh + 4 * s + g];
            }
            // dA = V^T dO for the keys of this chunk (half 1 continues half 0's sums)
            float af[2][NS];
            load_afrag<NS>(af[0], Ss + il * RS + g);
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) load_afrag<NS>(af[(jl + 1) & 1], Ss + ((jl + 1) * 16 + il) * RS + g);
                PIPELINE_FENCE();
                floatx4_t acc = { 0, 0, 0, 0 };
                if (hf > 0) {
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[r] = ds[jt][r];
                }
#pragma unroll
                for (int s = 0; s < NS; s++) acc = mfma16(af[jl & 1][s], dof[hf][s], acc);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    ds[jt][r] = acc[r];
                    if (hf == NH - 1) dot += p[jt][r] * acc[r];
                }
            }
            if (c == NCH - 1 && hf == NH - 1) {
                // dS = P (dA - colsum(P dA)) / sqrt(dk), then its rel-shift adjoint into the strip
                dot += __shfl_xor(dot, 16, 64);
                dot += __shfl_xor(dot, 32, 64);
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) ds[jt][r] = p[jt][r] * (ds[jt][r] - dot) * a.scale; // masked: p = 0
                for (int pp = g; pp < KP; pp += 4) Rw[pp] = 0.0f;
                wave_lds_sync();
                const int dbase = i + a.M - 4 * g, pbase = a.d_pos - 1 - dbase;
                const unsigned dlim = (i < a.T && has_w) ? (unsigned)a.attn_len : 0u;
                float acc0 = 0.0f;
#pragma unroll
                for (int jt = 0; jt < NTT; jt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        unsigned delta = (unsigned)(dbase - (jt * 16 + r));
                        int pi = pbase + (jt * 16 + r);
                        // rows >= 1 receive exactly one key; row 0 collects the far keys;
                        // masked keys go to a dump slot past the strip (never read)
                        const bool on = delta < dlim;
                        Rw[(on && pi >= 1) ? pi : RST - 1] = ds[jt][r];
                        acc0 += (on && pi < 1) ? ds[jt][r] : 0.0f;
                    }
                acc0 += __shfl_xor(acc0, 16, 64);
                acc0 += __shfl_xor(acc0, 32, 64);
                if (g == 0) Rw[0] = acc0;
                wave_lds_sync();
            }
        } else {
            // dq[:, half] += K[:, half] dS (kind 1) or w_r[:, half] dRel (kind 2) over the rows of this chunk
            float kf[2][ND][4], rf[2][4];
            load_tokfrag<ND, RS>(kf[0], Ss, 0, g, il);
            if (kind == 2) {
#pragma unroll
                for (int r = 0; r < 4; r++) rf[0][r] = Rw[(8 * c) * 16 + 4 * g + r];
            }
#pragma unroll
            for (int jl = 0; jl < 8; jl++) {
                if (jl >= nt) break;
                const int jt = 8 * c + jl;
                if (jl + 1 < nt) {
                    load_tokfrag<ND, RS>(kf[(jl + 1) & 1], Ss, jl + 1, g, il);
                    if (kind == 2) {
#pragma unroll
                        for (int r = 0; r < 4; r++) rf[(jl + 1) & 1][r] = Rw[(jt + 1) * 16 + 4 * g + r];
                    }
                }
                PIPELINE_FENCE();
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int dt = 0; dt < ND; dt++)
                        dqa[hf * ND + dt] = mfma16(kf[jl & 1][dt][r], kind == 1 ? ds[jt][r] : rf[jl & 1][r], dqa[hf * ND + dt]);
            }
        }
    }
    if (i < a.T) {
#pragma unroll
        for (int dt = 0; dt < NH * ND; dt++) {
            float *o = a.dq + (int64_t)h * DK + dt * 16 + 4 * g + a.ldq * (b + (int64_t)a.B * i);
            *reinterpret_cast<floatx4_t *>(o) = dqa[dt];
        }
    }

    // the contraction now runs over the query index; k-slot g of step s is
    // query 16*(s/4) + 4g + s%4, which keeps the Q / dO reads conflict-free
    auto load_qd = [&](float (&f)[ND], const float *base, int s) {
        int iq = 16 * (s >> 2) + 4 * g + (s & 3);
#pragma unroll
        for (int dt = 0; dt < ND; dt++) f[dt] = base[iq * RS + dt * 16 + il];
    };
    float dbacc[2] = { 0.0f, 0.0f };
#pragma unroll
    for (int hf = 0; hf < NH; hf++) {
        // this half of Q and dO into x (dO's full-width copy went into registers long ago; with
        // hf > 0 every wavefront must have left the half before)
        floatx4_t vqh[FA_TMAX * 16 / 256], voh[FA_TMAX * 16 / 256];
        fetch_rows<64, FA_TMAX>(vqh, a.T, [&](int r) { return a.q + (int64_t)h * DK + 64 * hf + a.ldq * (b + (int64_t)a.B * r); });
        fetch_rows<64, FA_TMAX>(voh, a.T, [&](int r) { return a.dout + (int64_t)h * DK + 64 * hf + a.ldo * (b + (int64_t)a.B * r); });
        __syncthreads();
        put_rows<64, FA_TMAX>(Qh, vqh, a.T);
        put_rows<64, FA_TMAX>(Oh, voh, a.T);
        // dK = Q dS^T, dV = dO P^T, 64 keys at a time: wavefront w owns key tile 4*hc + w;
        // db_r (first half only): thread t sums the diagonals delta = t and t + 256 over the parked keys
#pragma unroll
        for (int hc = 0; hc < NTT / 4; hc++) {
            __syncthreads(); // the staging tile (or the previous 64 keys) is dead
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int jl = e * 16 + 4 * g + r;
                    Pt[jl * PS + i] = p[4 * hc + e][r];
                    St[jl * PS + i] = ds[4 * hc + e][r];
                }
            __syncthreads();
            {
                float sb[NSQ], pb[NSQ];
#pragma unroll
                for (int s = 0; s < NSQ; s++) {
                    int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                    sb[s] = St[(w * 16 + il) * PS + iq];
                    pb[s] = Pt[(w * 16 + il) * PS + iq];
                }
                floatx4_t ak[ND], av[ND];
#pragma unroll
                for (int dt = 0; dt < ND; dt++) { ak[dt] = floatx4_t{ 0, 0, 0, 0 }; av[dt] = floatx4_t{ 0, 0, 0, 0 }; }
                float qa[2][ND], oa[2][ND];
                load_qd(qa[0], Qh, 0);
                load_qd(oa[0], Oh, 0);
#pragma unroll
                for (int s = 0; s < NSQ; s++) {
                    if (s + 1 < NSQ) { load_qd(qa[(s + 1) & 1], Qh, s + 1); load_qd(oa[(s + 1) & 1], Oh, s + 1); }
                    PIPELINE_FENCE();
#pragma unroll
                    for (int dt = 0; dt < ND; dt++) {
                        ak[dt] = mfma16(qa[s & 1][dt], sb[s], ak[dt]);
                        av[dt] = mfma16(oa[s & 1][dt], pb[s], av[dt]);
                    }
                }
                const int j = (4 * hc + w) * 16 + il;
                if (j < a.K) {
                    float *dst = (j < a.M ? a.dkvm + a.ldkv * (b + (int64_t)a.B * j)
                                          : a.dkv + a.ldkv * (b + (int64_t)a.B * (j - a.M))) + (int64_t)h * DK + 64 * hf;
#pragma unroll
                    for (int dt = 0; dt < ND; dt++) {
                        *reinterpret_cast<floatx4_t *>(dst + dt * 16 + 4 * g) = ak[dt];
                        *reinterpret_cast<floatx4_t *>(dst + (int64_t)a.H * DK + dt * 16 + 4 * g) = av[dt];
                    }
                }
            }
            if (hf == 0 && a.dbp) {
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int delta = t + 256 * u;
                    // keys 64*hc .. 64*hc+63 of diagonal delta belong to queries lo .. lo+63
                    const int lo = delta - a.M + 64 * hc;
                    float acc = 0.0f;
#pragma unroll 8
                    for (int q8 = 0; q8 < 64; q8++) {
                        const int iq = lo + q8;
                        const bool on = delta < a.K && iq >= 0 && iq < a.T && 64 * hc + q8 < a.K;
                        float v = St[(on ? q8 : 0) * PS + (on ? iq : 0)];
                        acc += on ? v : 0.0f;
                    }
                    dbacc[u] += acc;
                }
            }
        }
        // dw_r partial of this (stream, head), this half: Q dRel^T, wavefront w owns position tiles w, w+4, ...
        if (has_w) {
            float *dwz = a.dwp + ((int64_t)b * a.H + h) * a.d_pos * DK + 64 * hf;
#pragma unroll
            for (int u = 0; u < NTT / 4; u++) {
                const int pt = w + 4 * u;
                float rb[NSQ];
#pragma unroll
                for (int s = 0; s < NSQ; s++) {
                    int iq = 16 * (s >> 2) + 4 * g + (s & 3);
                    rb[s] = Rs[iq * RST + pt * 16 + il];
                }
                floatx4_t acc[ND];
#pragma unroll
                for (int dt = 0; dt < ND; dt++) acc[dt] = floatx4_t{ 0, 0, 0, 0 };
                float qa[2][ND];
                load_qd(qa[0], Qh, 0);
#pragma unroll
                for (int s = 0; s < NSQ; s++) {
                    if (s + 1 < NSQ) load_qd(qa[(s + 1) & 1], Qh, s + 1);
                    PIPELINE_FENCE();
#pragma unroll
                    for (int dt = 0; dt < ND; dt++) acc[dt] = mfma16(qa[s & 1][dt], rb[s], acc[dt]);
                }
                const int pp = pt * 16 + il;
                if (pp < a.d_pos) {
#pragma unroll
                    for (int dt = 0; dt < ND; dt++)
                        *reinterpret_cast<floatx4_t *>(dwz + (int64_t)pp * DK + dt * 16 + 4 * g) = acc[dt];
                }
            }
        }
    }
    if (a.dbp) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int delta = t + 256 * u;
            if (delta < a.K)
                a.dbp[((int64_t)b * a.H + h) * a.K + (a.K - 1 - delta)] = a.b_r_scale * dbacc[u];
        }
    }
}

// ---- one query per (stream, head): the decoder's timestep ---------------------------------
// The single query of a timestep through the arithmetic of relpos_attn_fwd_fused, on the
// vector ALUs.  An fp32 MFMA accumulates its k values one after the other with fused
// multiply-adds in increasing k, so every number of that kernel's column q_only can be
// formed by plain code in the same order: the score of key j is a chain of DK fmas over the
// features plus the position term (its own chain over w_r row d_pos-1-delta, clamped) plus the
// scaled bias; the sum of the exponentials is taken the way the four lanes of a column hold
// it (lane g: keys 16 jt + 4g + r in increasing order, then (s0 + s1) + (s2 + s3)); output
// feature d is one chain over the keys in the order the PV MFMAs meet them (tile jt, step r,
// k slot g: key 16 jt + 4g + r).  Masked keys contribute exact zeros there and are skipped.
// A workgroup is one (stream, head): four neighbouring lanes own a key (only keys inside the
// attention window are fetched), then thread d owns output feature d.
// a product that is rounded on its own (the whole-segment kernel keeps the scaled bias in
// LDS, so no multiply-add can swallow it)
__device__ __forceinline__ float rounded_product(float x, float y)
{
#pragma clang fp contract(off)
    return x * y;
}

template <int DK>
__global__ __launch_bounds__(512) void relpos_attn_step_scalar(FusedAttnFwdArgs a)
{
    constexpr int RS = DK + 4, NS = DK / 4, QP = NS / 4; // QP: 16-byte pieces of a row per lane
    __shared__ __attribute__((aligned(16))) float Vs[128 * RS];
    __shared__ __attribute__((aligned(16))) float qs[DK];
    __shared__ __attribute__((aligned(16))) float es[128];
    __shared__ float red[4];
    // four neighbouring lanes share a key: each fetches a quarter of its rows (a wavefront's
    // load then touches 16 rows instead of 64) and the chain over the features passes from
    // quarter to quarter
    const int t = threadIdx.x, j = t >> 2, sq = t & 3;
    const int b = blockIdx.x % a.B, h = blockIdx.x / a.B;
    const int i = a.q_only;
    const int delta = i + a.M - j;
    const bool valid = j < a.K && (unsigned)delta < (unsigned)a.attn_len;
    const bool has_w = a.w_r != nullptr;
    floatx4_t kr[QP], vr[QP], wr[QP];
    float bias_t = 0.0f;
    if (valid) {
        const float *row = (j < a.M ? a.kvm + a.ldkv * (b + (int64_t)a.B * j)
                                    : a.kv + a.ldkv * (b + (int64_t)a.B * (j - a.M))) + (int64_t)h * DK + 4 * QP * sq;
        const floatx4_t NCHIP_GLOBAL *kp = reinterpret_cast<const floatx4_t NCHIP_GLOBAL *>(as_global(row));
        const floatx4_t NCHIP_GLOBAL *vp = reinterpret_cast<const floatx4_t NCHIP_GLOBAL *>(as_global(row + (int64_t)a.H * DK));
#pragma unroll
        for (int p = 0; p < QP; p++) kr[p] = kp[p];
        if (has_w) {
            int pi = a.d_pos - 1 - delta;
            pi = pi < 0 ? 0 : pi; // (delta >= 0: never above d_pos - 1)
            const floatx4_t NCHIP_GLOBAL *wp = reinterpret_cast<const floatx4_t NCHIP_GLOBAL *>(
                as_global(a.w_r + ((int64_t)h * a.d_pos + pi) * DK + 4 * QP * sq));
#pragma unroll
            for (int p = 0; p < QP; p++) wr[p] = wp[p];
        }
#pragma unroll
        for (int p = 0; p < QP; p++) vr[p] = vp[p];
        if (a.b_r && sq == 3) bias_t = as_global(a.b_r)[(int64_t)h * a.K + (a.K - 1 - delta)];
    }
    if (t < NS) {
        floatx4_t q4 = *reinterpret_cast<const floatx4_t NCHIP_GLOBAL *>(as_global(a.q + (int64_t)h * DK + a.ldq * b) + 4 * t);
#pragma unroll
        for (int r = 0; r < 4; r++) qs[4 * t + r] = q4[r] * a.scale; // 1/sqrt(dk) folded in
    }
    __syncthreads();
    float sc = 0.0f, rl = 0.0f;
#pragma unroll
    for (int r = 0; r < 4; r++) { // quarter r of the features, by the lane that holds it
        if (sq == r && valid) {
#pragma unroll
            for (int p = 0; p < QP; p++) {
                const floatx4_t q4 = *reinterpret_cast<const floatx4_t *>(qs + 4 * (r * QP + p));
#pragma unroll
                for (int e = 0; e < 4; e++) sc = __builtin_fmaf(kr[p][e], q4[e], sc);
                if (has_w) {
#pragma unroll
                    for (int e = 0; e < 4; e++) rl = __builtin_fmaf(wr[p][e], q4[e], rl);
                }
            }
        }
        if (r < 3) { // the chains so far go to the lane of the next quarter
            const float sc_up = __shfl_up(sc, 1, 64), rl_up = __shfl_up(rl, 1, 64);
            if (sq == r + 1) { sc = sc_up; rl = rl_up; }
        }
    }
    if (valid) {
#pragma unroll
        for (int p = 0; p < QP; p++) *reinterpret_cast<floatx4_t *>(Vs + j * RS + 4 * (QP * sq + p)) = vr[p];
        if (sq == 3) es[j] = sc + rl + rounded_product(bias_t, a.b_r_scale * a.scale);
    } else { // a masked key's probability is an exact zero: its value row must only be finite
#pragma unroll
        for (int p = 0; p < QP; p++) *reinterpret_cast<floatx4_t *>(Vs + j * RS + 4 * (QP * sq + p)) = floatx4_t{ 0, 0, 0, 0 };
        if (sq == 3) es[j] = -INFINITY;
    }
    __syncthreads();
    // from here on thread k < 128 is key k (then output feature k)
    const float v = t < 128 ? es[t] : -INFINITY;
    // maximum over the keys (exact in any order)
    float mx = v;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if ((t & 63) == 0 && t < 128) red[t >> 6] = mx;
    __syncthreads();
    mx = fmaxf(red[0], red[1]);
    if (mx == -INFINITY) mx = 0.0f;
    const float e = __expf(v - mx); // exp(-inf) = 0 for masked keys
    if (t < 128) es[t] = e;
    __syncthreads();
    if (t < 4) { // the partial sum lane group g of the column holds in the whole-segment kernel
        floatx4_t e4[8];
#pragma unroll
        for (int jt = 0; jt < 8; jt++) e4[jt] = *reinterpret_cast<const floatx4_t *>(es + jt * 16 + 4 * t);
        float sum = 0.0f;
#pragma unroll
        for (int jt = 0; jt < 8; jt++)
#pragma unroll
            for (int r = 0; r < 4; r++) sum += e4[jt][r];
        red[t] = sum;
    }
    __syncthreads();
    const float sum = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (t < 128) es[t] = e * inv; // (every thread read its own e above; the sums are done)
    __syncthreads();
    if (t < DK) {
        const int j_hi = i + a.M, j_lo = j_hi - a.attn_len + 1; // keys inside the window (uniform)
        float acc = 0.0f;
        for (int jt = 0; jt < 8; jt++) {
            if (jt * 16 > j_hi || jt * 16 + 15 < j_lo) continue; // a tile of masked keys: sixteen exact no-ops
            floatx4_t p4[4];
            float vv[16];
#pragma unroll
            for (int g = 0; g < 4; g++) p4[g] = *reinterpret_cast<const floatx4_t *>(es + jt * 16 + 4 * g);
#pragma unroll
            for (int u = 0; u < 16; u++) vv[u] = Vs[(jt * 16 + u) * RS + t];
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int g = 0; g < 4; g++) acc = __builtin_fmaf(vv[4 * g + r], p4[g][r], acc);
        }
        as_global(a.out)[(int64_t)h * DK + t + a.ldo * b] = acc;
    }
}

int g_attn_step_scalar = 1; // 0: single-query calls go through the whole-segment kernel (testing aid)
int g_attn_wide_bwd = 0;    // 1: heads of 128 take the single-kernel backward at every key count

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

template <int DK, int NT, bool VEC>
int launch_fwd_v(hipStream_t st, const FusedAttnFwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * FwdLayout<DK, NT>::floats;
    static_assert(bytes <= 160 * 1024, "forward tiles exceed LDS");
    static const bool ok = allow_lds(relpos_attn_fwd_fused<DK, NT, VEC>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL((relpos_attn_fwd_fused<DK, NT, VEC>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// 16-byte accesses to a column of probabilities need K % 4 == 0 and an aligned base
template <typename Args>
bool probs_vec(const Args &a) { return (a.K & 3) == 0 && (((uintptr_t)a.probs) & 15) == 0; }

template <int DK, int NT>
int launch_fwd(hipStream_t st, const FusedAttnFwdArgs &a)
{
    return probs_vec(a) ? launch_fwd_v<DK, NT, true>(st, a) : launch_fwd_v<DK, NT, false>(st, a);
}

template <int DK, int NT, bool VEC>
int launch_bwd_v(hipStream_t st, const FusedAttnBwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * BwdLayout<DK, NT>::floats;
    static_assert(bytes <= 160 * 1024, "backward tiles exceed LDS");
    static const bool ok = allow_lds(relpos_attn_bwd_fused<DK, NT, VEC>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL((relpos_attn_bwd_fused<DK, NT, VEC>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int DK, int NT>
int launch_bwd(hipStream_t st, const FusedAttnBwdArgs &a)
{
    return probs_vec(a) ? launch_bwd_v<DK, NT, true>(st, a) : launch_bwd_v<DK, NT, false>(st, a);
}

template <int DK, int NTT>
int launch_fwd_tiled(hipStream_t st, const FusedAttnFwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * FwdTiledLayout<DK, NTT>::floats;
    static_assert(bytes <= 160 * 1024, "forward tiles exceed LDS");
    static const bool ok = allow_lds(relpos_attn_fwd_tiled<DK, NTT>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL((relpos_attn_fwd_tiled<DK, NTT>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int DK, int NTT>
int launch_bwd_tiled(hipStream_t st, const FusedAttnBwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * BwdTiledLayout<DK, NTT>::floats;
    static_assert(bytes <= 160 * 1024, "backward tiles exceed LDS");
    static const bool ok = allow_lds(relpos_attn_bwd_tiled<DK, NTT>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL((relpos_attn_bwd_tiled<DK, NTT>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int NH, int NTT>
int launch_fwd_wide(hipStream_t st, const FusedAttnFwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * FwdWideLayout<NH, NTT>::floats;
    static_assert(bytes <= 160 * 1024, "forward tiles exceed LDS");
    static const bool ok = allow_lds(relpos_attn_fwd_wide<NH, NTT>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL((relpos_attn_fwd_wide<NH, NTT>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int NH, int NTT>
int launch_bwd_wide(hipStream_t st, const FusedAttnBwdArgs &a)
{
    constexpr size_t bytes = sizeof(float) * BwdWideLayout<NH, NTT>::floats;
    static_assert(bytes <= 160 * 1024, "backward tiles exceed LDS");
    static const bool ok = allow_lds(relpos_attn_bwd_wide<NH, NTT>, bytes);
    if (!ok) return -1;
    hipLaunchKernelGGL((relpos_attn_bwd_wide<NH, NTT>), dim3(a.B * a.H), dim3(256), bytes, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// 16-key tiles the kernels for heads of 128 need for K keys and d_pos positions (0: not their shape)
int wide_ntt(int K, int d_pos)
{
    const int need = K > d_pos ? K : d_pos;
    int ntt = ((need + 15) / 16 + 3) / 4 * 4;
    if (ntt < 8) ntt = 8;
    return (ntt <= 20 && (K & 3) == 0) ? ntt : 0;
}

// 16-key tiles the chunked kernels need for K keys and d_pos positions (0: not their shape)
int tiled_ntt(int K, int d_pos)
{
    const int need = K > d_pos ? K : d_pos;
    const int ntt = ((need + 15) / 16 + 3) / 4 * 4;
    return (need > 128 && ntt <= 20 && (K & 3) == 0) ? ntt : 0;
}

} // namespace

bool k_attn_fused_step_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr)
{
    return dk == dv && (dk == 64 || dk == 32) && T <= FA_TMAX && K <= 128 && (!has_wr || d_pos <= 128);
}

bool k_attn_fused_shape_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr)
{
    if (k_attn_fused_step_ok(dk, dv, T, K, d_pos, has_wr)) return true;
    if (dk == 128 && dv == 128) return T <= FA_TMAX && wide_ntt(K, has_wr ? d_pos : 1) != 0;
    return dk == 64 && dv == 64 && T <= FA_TMAX && tiled_ntt(K, has_wr ? d_pos : 1) != 0;
}

// testing aid: 0 sends single-query calls through the whole-segment kernel again (every row
// of its query tile the one query), 1 (default) through the vector-ALU kernel: same bits
extern "C" void nchip_relpos_attn_step_kernel(int scalar)
{
    g_attn_step_scalar = scalar;
}

// 1: the backward of heads of 128 features runs as one kernel for every key count it holds
// (up to 320); 0 (default): only up to 128 keys, beyond that the batched products, which
// are faster there.  Same results to rounding either way.
extern "C" void nchip_relpos_attn_wide_backward(int always)
{
    g_attn_wide_bwd = always;
}

int k_attn_fused_fwd(hipStream_t st, const FusedAttnFwdArgs &a, int dk)
{
    if (a.q_only >= 0 && g_attn_step_scalar && a.K <= 128 && a.d_pos <= 128 && !a.probs) {
        if (dk == 64) hipLaunchKernelGGL(relpos_attn_step_scalar<64>, dim3(a.B * a.H), dim3(512), 0, st, a);
        else hipLaunchKernelGGL(relpos_attn_step_scalar<32>, dim3(a.B * a.H), dim3(512), 0, st, a);
        return hipGetLastError() == hipSuccess ? 0 : -1;
    }
    if (dk == 128) {
        const int ntt = wide_ntt(a.K, a.d_pos);
        if (!ntt || a.T > FA_TMAX || a.q_only >= 0 || !a.probs || !probs_vec(a)) return -1;
        return ntt == 8 ? launch_fwd_wide<2, 8>(st, a) : ntt == 12 ? launch_fwd_wide<2, 12>(st, a)
             : ntt == 16 ? launch_fwd_wide<2, 16>(st, a) : launch_fwd_wide<2, 20>(st, a);
    }
    if (const int ntt = (a.K > 128 || a.d_pos > 128) ? tiled_ntt(a.K, a.d_pos) : 0) {
        if (dk != 64 || a.q_only >= 0 || !a.probs || !probs_vec(a)) return -1;
        return ntt == 12 ? launch_fwd_tiled<64, 12>(st, a) : ntt == 16 ? launch_fwd_tiled<64, 16>(st, a)
                                                                      : launch_fwd_tiled<64, 20>(st, a);
    }
    if (a.K > 128 || a.d_pos > 128) return -1;
    const bool small = a.K <= 64 && a.d_pos <= 64;
    if (dk == 64) return small ? launch_fwd<64, 4>(st, a) : launch_fwd<64, 8>(st, a);
    return small ? launch_fwd<32, 4>(st, a) : launch_fwd<32, 8>(st, a);
}

int k_attn_fused_bwd(hipStream_t st, const FusedAttnBwdArgs &a, int dk, float *dw_r, float *db_r,
                     int64_t n_w, int64_t n_b, int *launches, bool keep_partials)
{
    const bool small = a.K <= 64 && a.d_pos <= 64;
    int rc;
    if (dk == 128) {
        const int ntt = wide_ntt(a.K, a.d_pos);
        if (!ntt || a.T > FA_TMAX || !probs_vec(a)) return -1;
        // Measured at 8 heads x 32 streams (one workgroup per CU): up to 128 keys this kernel and
        // the batched-product backward take the same time (123 us); at 320 keys the batched
        // products are faster (228 us against 340-390 us: this kernel keeps one wavefront per
        // SIMD busy with 36 staged tiles and two passes over the key-owned phase), so they
        // take those shapes unless the caller asks for this kernel.
        if (ntt > 8 && !g_attn_wide_bwd) return -1;
        rc = ntt == 8 ? launch_bwd_wide<2, 8>(st, a) : ntt == 12 ? launch_bwd_wide<2, 12>(st, a)
           : ntt == 16 ? launch_bwd_wide<2, 16>(st, a) : launch_bwd_wide<2, 20>(st, a);
    } else if (a.K > 128 || a.d_pos > 128) {
        const int ntt = tiled_ntt(a.K, a.d_pos);
        if (!ntt || dk != 64 || !probs_vec(a)) return -1;
        rc = ntt == 12 ? launch_bwd_tiled<64, 12>(st, a) : ntt == 16 ? launch_bwd_tiled<64, 16>(st, a)
                                                                    : launch_bwd_tiled<64, 20>(st, a);
    } else
        rc = dk == 64 ? (small ? launch_bwd<64, 4>(st, a) : launch_bwd<64, 8>(st, a))
                      : (small ? launch_bwd<32, 4>(st, a) : launch_bwd<32, 8>(st, a));
    if (rc) return rc;
    *launches = 1;
    if (n_w + n_b > 0 && !keep_partials) {
        hipLaunchKernelGGL(attn_param_grad_reduce, dim3((unsigned)((n_w + n_b + 255) / 256)), dim3(256), 0, st,
                           (const float *)a.dwp, dw_r, n_w, (const float *)a.dbp, db_r, n_b, a.B);
        *launches = 2;
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
