// GEMM for gfx950 (MI355X): column-major C = act(alpha*op(A)*op(B) + beta*C + bias) [+ addend].
//
// A workgroup of WM x WN wavefronts (times KW k groups) owns a BM x BN tile of C.  A and B
// tiles of depth BK are staged through LDS (double buffered, PF register sets of tiles in
// flight from global memory, k-major rows so a wavefront reads 32 consecutive floats), and
// every wavefront accumulates its part with v_mfma_f32_32x32x2_f32.  The MFMA is issued as
// D[n][m] = sum_k B[k][n]*A[k][m] so that the 32 lanes of a half-wavefront hold 32
// consecutive m of one column: the epilogue stores are 128-byte coalesced in column-major C.
//
// Tile classes (chosen from the shape only): 128x128x32 with 8 wavefronts, 128x64x32 with 8
// wavefronts, 64x64x32 with two k groups of 4 wavefronts (KW = 2: the groups split every
// 32-deep slab, C = chain0 + chain1).  Inside a class a C element is a fixed sequence of MFMA
// accumulations that does not depend on m, n or the number of columns.  The width-invariant
// class (NCHIP_GEMM_WIDTH_INVARIANT: 64x64x32, KW = 2, two accumulator sets per group = four
// chains per element, no split-K) is used by encoder and decoder alike when a column computed
// alone must equal the same column computed inside a larger matrix (bit-exact decode);
// gemm_skinny_nn issues the same sequence for products of a few columns.
//
// precision 1 rounds both operands to bf16 (nearest-even) while they are written to LDS and
// feeds v_mfma_f32_32x32x16_bf16 (fp32 accumulate); large products go through bf16 copies of
// the operands instead (cast_bf16_kernel + the BF16 = 2 tile kernels).
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include <vector>
#include "../../include/nchip_kernels.h"
#include "k_addrspace.h"
#include "k_bf16.h"
#include "k_act.h"
#include "k_norm_inline.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4))); // a first-class value, unlike the uint4 struct

// (operand loads and result stores go through global-address-space pointers: k_addrspace.h)
namespace {

constexpr int KALIGN = 16; // split-K chunk granularity
constexpr int PAD = 4;   // keeps 16-byte alignment of LDS rows, staggers banks
constexpr int NXCD = 8;

#ifdef NCHIP_GEMM_CLOCKS
// debug builds: shader-clock and wall-clock span of the k loop of workgroup 0
__device__ long long *g_gemm_clk = nullptr;
#endif

struct GemmArgs {
    const float *A, *B;
    float *C;
    const float *bias;
    const float *add; // same layout as C, added after the activation (may be NULL)
    const float *dpre; // same layout as C: the result is multiplied by act'(dpre) (may be NULL)
    int dact;
    float *pre;
    float *ws;
    uint16_t *c16; // the result once more, rounded to bf16, laid out like C (may be NULL)
    int64_t lda, ldb, ldc, sa, sb, sc;   // outer batch strides
    int64_t sa_in, sb_in, sc_in;         // inner batch strides
    int batch_in;                        // batch index z -> (z / batch_in, z % batch_in)
    int M, N, K, batch, ksplit, kchunk;
    float alpha, beta;
    int act;
    int tiles_m, tiles_n;
    int gm; // tile rows per band of the tile order (see the kernel)
    int dbg;
    const NchipGemmProblem *grp; // grouped launch: one problem per table row
    int n_grp;
    int grp_chunk; // grouped launch: consecutive tiles of the list handed to one XCD at a time
    float *rowsum; // activation-gradient epilogue only: partial row sums of the result, one row per (tile column, wavefront column, lane half)
    // second product of a few-column pair launch (gemm_skinny_nn, blockIdx.z = 1): same B, N, K
    const float *A_1, *bias_1;
    float *C_1;
    int64_t lda_1, ldc_1;
    int M_1;
    // few-column kernel that normalises B on the way in (gemm_fewcol_mfma with NV > 0): gain and
    // bias (both or neither), the normalised columns written to ln_out (leading dimension
    // ld_ln) by the first row tile when it is not NULL
    const float *ln_w, *ln_b;
    float *ln_out;
    int64_t ld_ln;
    float ln_eps;
    int ln_avg;
};

__device__ __forceinline__ float gelu_tanh(float x) { return nchip_gelu(x); } // k_act.h

// GELU of the products that round their operands to bf16: the launchers turn NCHIP_ACT_GELU
// into this code when the precision argument is not fp32 (k_act.h says why there are two)
constexpr int ACT_GELU_FAST = 3;
static_assert(ACT_GELU_FAST != NCHIP_ACT_NONE && ACT_GELU_FAST != NCHIP_ACT_GELU && ACT_GELU_FAST != NCHIP_ACT_RELU, "");
inline int act_for_precision(int act, int precision) { return (act == NCHIP_ACT_GELU && precision != 0) ? ACT_GELU_FAST : act; }

__device__ __forceinline__ float act_grad(float x, int act)
{
    if (act == NCHIP_ACT_GELU) return nchip_gelu_grad(x);
    if (act == ACT_GELU_FAST) return nchip_gelu_grad_fast(x);
    if (act == NCHIP_ACT_RELU) return x > 0.0f ? 1.0f : 0.0f;
    return 1.0f;
}

__device__ __forceinline__ float apply_act(float v, int act)
{
    if (act == NCHIP_ACT_GELU) return gelu_tanh(v);
    if (act == ACT_GELU_FAST) return nchip_gelu_fast(v);
    if (act == NCHIP_ACT_RELU) return v > 0.0f ? v : 0.0f;
    return v;
}

__device__ __forceinline__ unsigned short f32_to_bf16(float f)
{
    unsigned int u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}

// Loads a BT x BK tile (BT = BM or BN) of an operand into registers.
// MAJOR = 1: the tile's long axis (m or n) is contiguous in memory
//            (A with ta = 0, B with tb = 1);  element (i, k) at p[i + k*ld].
// MAJOR = 0: k is contiguous (A with ta = 1, B with tb = 0); (i, k) at p[k + i*ld].
//
// A k-contiguous tile is fetched row by row: BK / 4 consecutive lanes take one
// row's BK floats (whole 128-byte lines when BK = 32), so a wavefront touches
// 64 * 4 / BK rows instead of 64 - one cache line per lane was what bound these
// tiles.  Its LDS rows are BT + 1 floats apart (FPAD_K): the four transposing
// writes of a lane then fall on banks 4*(k/4) + e + i, distinct over the 32
// lanes served together.
constexpr int FPAD_K = 1;
template <int BT, int BK, int MAJOR, int NT>
struct TileLoader {
    static constexpr int NV = BT * BK / 4 / NT; // float4 per thread
    static constexpr int RS = BT + (MAJOR ? PAD : FPAD_K); // LDS row stride
    static_assert(NV >= 1 && NV * NT * 4 == BT * BK, "tile must divide evenly over the threads");
    floatx4 r[NV];

    __device__ __forceinline__ static void coords(int idx, int &i, int &k)
    {
        if (MAJOR) { i = (idx % (BT / 4)) * 4; k = idx / (BT / 4); }
        else       { i = idx / (BK / 4);       k = (idx % (BK / 4)) * 4; }
    }

    __device__ __forceinline__ void load(const float *p, int64_t ld, int i0, int k0,
                                         int imax, int kmax, bool fast, int t)
    {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            int idx = t + v * NT;
            int i, k;
            coords(idx, i, k);
            if (fast) {
                const float *src = MAJOR ? p + (int64_t)(k0 + k) * ld + (i0 + i)
                                         : p + (int64_t)(i0 + i) * ld + (k0 + k);
                r[v] = *as_global(reinterpret_cast<const floatx4 *>(src));
            } else {
                floatx4 tmp;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int ii = MAJOR ? i + e : i, kk = MAJOR ? k : k + e;
                    float val = 0.0f;
                    if (i0 + ii < imax && k0 + kk < kmax)
                        val = MAJOR ? as_global(p)[(int64_t)(k0 + kk) * ld + (i0 + ii)]
                                    : as_global(p)[(int64_t)(i0 + ii) * ld + (k0 + kk)];
                    tmp[e] = val;
                }
                r[v] = tmp;
            }
        }
    }

    // fp32 LDS tile: rows are k, RS floats each
    __device__ __forceinline__ void store_f32(float *lds, int t) const
    {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            int i, k;
            coords(t + v * NT, i, k);
            if (MAJOR) {
                *reinterpret_cast<floatx4 *>(lds + k * RS + i) = r[v];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    lds[(k + e) * RS + i] = r[v][e];
            }
        }
    }
};

// bf16 variant of the loader.  LDS holds 32-bit words of two bf16 values that
// are consecutive in k: word (kp, i) = (x[i][2kp], x[i][2kp+1]), rows kp of
// BT + PAD words.  A lane of v_mfma_f32_32x32x16_bf16 (row i, k group kg) reads
// the 4 words kp = kb*8 + kg*4 .. +3 of column i: 8 consecutive k, lanes on
// consecutive banks.  Operands whose long axis is contiguous in memory are
// fetched as 2 columns x 2 rows (k, k+1) and stored as one 8-byte LDS write;
// k-contiguous operands give two words per float4.  Rounding is to nearest
// even (v_cvt_pk_bf16_f32).
// (pack_bf16: k_bf16.h)

template <int BT, int BK, int MAJOR, int NT>
struct TileLoaderBf16 {
    static constexpr int NV = BT * BK / 4 / NT; // 4-float units per thread
    static_assert(NV >= 1 && NV * NT * 4 == BT * BK, "tile must divide evenly over the threads");
    floatx4 r[NV];

    // MAJOR = 1: a unit is 2 columns x 2 consecutive k rows, r = (x[i][k], x[i+1][k], x[i][k+1], x[i+1][k+1]);
    // MAJOR = 0: a unit is 4 consecutive k of one column
    __device__ __forceinline__ static void coords(int v, int t, int &i, int &k)
    {
        int idx = t + v * NT;
        if (MAJOR) { i = (idx % (BT / 2)) * 2; k = (idx / (BT / 2)) * 2; }
        else       { i = idx % BT;             k = (idx / BT) * 4; }
    }

    __device__ __forceinline__ void load(const float *p, int64_t ld, int i0, int k0,
                                         int imax, int kmax, bool fast, int t)
    {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            int i, k;
            coords(v, t, i, k);
            if (fast) {
                if (MAJOR) {
                    const float *src = p + (int64_t)(k0 + k) * ld + (i0 + i);
                    floatx2_t a = *as_global(reinterpret_cast<const floatx2_t *>(src));
                    floatx2_t b = *as_global(reinterpret_cast<const floatx2_t *>(src + ld));
                    r[v] = floatx4{ a[0], a[1], b[0], b[1] };
                } else {
                    r[v] = *as_global(reinterpret_cast<const floatx4 *>(p + (int64_t)(i0 + i) * ld + (k0 + k)));
                }
            } else {
                floatx4 tmp;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int ii = MAJOR ? i + (e & 1) : i, kk = MAJOR ? k + (e >> 1) : k + e;
                    float val = 0.0f;
                    if (i0 + ii < imax && k0 + kk < kmax)
                        val = MAJOR ? as_global(p)[(int64_t)(k0 + kk) * ld + (i0 + ii)]
                                    : as_global(p)[(int64_t)(i0 + ii) * ld + (k0 + kk)];
                    tmp[e] = val;
                }
                r[v] = tmp;
            }
        }
    }

    __device__ __forceinline__ void store(uint32_t *lds, int t) const
    {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            int i, k;
            coords(v, t, i, k);
            if (MAJOR) {
                uint2 w = make_uint2(pack_bf16(r[v][0], r[v][2]), pack_bf16(r[v][1], r[v][3]));
                *reinterpret_cast<uint2 *>(lds + (k >> 1) * (BT + PAD) + i) = w;
            } else {
                lds[(k >> 1) * (BT + PAD) + i] = pack_bf16(r[v][0], r[v][1]);
                lds[((k >> 1) + 1) * (BT + PAD) + i] = pack_bf16(r[v][2], r[v][3]);
            }
        }
    }
};

// Loader for operands that are already bf16 in memory (same column-major
// layout as the fp32 matrix they were rounded from, padded: the k extent is a
// whole number of tiles with zeros in the padding, and the allocation runs at
// least one tile past the last row so reads need no guard).  Same LDS layout
// as above.  Every load is 16 bytes (8 values):
//   MAJOR = 1: rows k and k+1 of 8 consecutive columns i -> 8 words, two
//              16-byte LDS writes;
//   MAJOR = 0: 8 consecutive k of one column i (row index clamped at the
//              edge) -> 4 words that already are k pairs, 4 LDS writes.
template <int BT, int BK, int MAJOR, int NT>
struct TileLoaderBf16Src {
    static constexpr int NU = MAJOR ? (BT / 8) * (BK / 2) : BT * (BK / 8); // 16-byte units per tile
    static constexpr int NV = (NU + NT - 1) / NT;
    static_assert(NU % 64 == 0 && (NU >= NT ? NU % NT == 0 : true), "whole wavefronts take part or sit out");
    u32x4 r[NV][MAJOR ? 2 : 1];

    __device__ __forceinline__ static void coords(int v, int t, int &i, int &k)
    {
        int idx = t + v * NT;
        if (MAJOR) { i = (idx % (BT / 8)) * 8; k = (idx / (BT / 8)) * 2; }
        else       { i = idx / (BK / 8);       k = (idx % (BK / 8)) * 8; }
    }

    __device__ __forceinline__ void load(const float *pf, int64_t ld, int i0, int k0,
                                         int imax, int kmax, bool fast, int t)
    {
        (void)kmax; (void)fast;
        const uint16_t *p = reinterpret_cast<const uint16_t *>(pf);
#pragma unroll
        for (int v = 0; v < NV; v++) {
            if (NU < NT && t >= NU) break;
            int i, k;
            coords(v, t, i, k);
            if (MAJOR) {
                const uint16_t *src = p + (int64_t)(k0 + k) * ld + (i0 + i);
                r[v][0] = *as_global(reinterpret_cast<const u32x4 *>(src));
                r[v][1] = *as_global(reinterpret_cast<const u32x4 *>(src + ld));
            } else {
                int row = i0 + i < imax ? i0 + i : imax - 1;
                r[v][0] = *as_global(reinterpret_cast<const u32x4 *>(p + (int64_t)row * ld + (k0 + k)));
            }
        }
    }

    // MAJOR = 1 writes the word-pair layout of TileLoaderBf16 (rows of k pairs,
    // BT + PAD words each); the two 16-byte halves of a unit go out in an
    // order that alternates every 4 lanes, so the 8 lanes served together
    // cover all 32 banks.  MAJOR = 0 keeps k contiguous: row i holds its
    // BK / 2 words, SQ words apart, and a unit is one 16-byte write.
    static constexpr int SQ = BK / 2 + 4;
    __device__ __forceinline__ void store(uint32_t *lds, int t) const
    {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            if (NU < NT && t >= NU) break;
            int i, k;
            coords(v, t, i, k);
            if (MAJOR) {
                const uint32_t a[4] = { r[v][0][0], r[v][0][1], r[v][0][2], r[v][0][3] };
                const uint32_t b[4] = { r[v][1][0], r[v][1][1], r[v][1][2], r[v][1][3] };
                uint32_t w[8];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    w[2 * e] = (a[e] & 0xffffu) | (b[e] << 16);
                    w[2 * e + 1] = (a[e] >> 16) | (b[e] & 0xffff0000u);
                }
                const bool hi_first = ((t >> 2) & 1) != 0;
                uint32_t *dst = lds + (k >> 1) * (BT + PAD) + i;
                uint32_t f[4], g[4]; // first and second write, chosen word by word (register selects)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    f[e] = hi_first ? w[4 + e] : w[e];
                    g[e] = hi_first ? w[e] : w[4 + e];
                }
                const int o1 = hi_first ? 4 : 0;
                *reinterpret_cast<u32x4 *>(dst + o1) = u32x4{ f[0], f[1], f[2], f[3] };
                *reinterpret_cast<u32x4 *>(dst + (4 - o1)) = u32x4{ g[0], g[1], g[2], g[3] };
            } else {
                *reinterpret_cast<u32x4 *>(lds + i * SQ + (k >> 1)) = r[v][0];
            }
        }
    }
};

// Epilogue of one 32x32 accumulator tile: acc[r] is C[m][nb + (r/4)*8 + r%4] (nb already
// holds the lane's (lane/32)*4).  The 16 values go to 16 columns of C.  Everything read here
// (addend, beta*C) is fetched for all 16 first, so the loads are in flight together, and the
// uniform option tests sit outside the element loops: a branch per element with a load
// behind it costs one memory round trip each.  Every product kernel ends in this function,
// so kernels that feed it the same accumulators write the same bits.
__device__ __forceinline__ void epilogue_tile(const GemmArgs &g, const floatx16 &acc, int m, int nb,
                                              float NCHIP_GLOBAL *C, float NCHIP_GLOBAL *P,
                                              const float NCHIP_GLOBAL *Radd, const float NCHIP_GLOBAL *Dp,
                                              bool full, bool plain, float NCHIP_GLOBAL *rowsum = nullptr,
                                              uint16_t NCHIP_GLOBAL *H = nullptr)
{
    if (!full && m >= g.M) return;
    float NCHIP_GLOBAL *Cp = C + (int64_t)nb * g.ldc + m; // element r lives at Cp + nofs(r)*ldc
    uint16_t NCHIP_GLOBAL *Hp = H ? H + (int64_t)nb * g.ldc + m : nullptr; // bf16 copy of the same elements
    auto nofs = [](int r) { return (r >> 2) * 8 + (r & 3); };
    if (plain && full) {
#pragma unroll
        for (int r = 0; r < 16; r++) Cp[(int64_t)nofs(r) * g.ldc] = g.alpha * acc[r];
        return;
    }
    bool ok[16];
#pragma unroll
    for (int r = 0; r < 16; r++) ok[r] = full || nb + nofs(r) < g.N;
    float extra[16]; // beta*C + addend
#pragma unroll
    for (int r = 0; r < 16; r++) extra[r] = 0.0f;
    if (Radd) {
        const float NCHIP_GLOBAL *Ap = Radd + (int64_t)nb * g.ldc + m;
#pragma unroll
        for (int r = 0; r < 16; r++) extra[r] = ok[r] ? Ap[(int64_t)nofs(r) * g.ldc] : 0.0f;
    }
    float prev[16];
    const bool has_beta = g.beta != 0.0f;
    if (has_beta) {
#pragma unroll
        for (int r = 0; r < 16; r++) prev[r] = ok[r] ? Cp[(int64_t)nofs(r) * g.ldc] : 0.0f;
    }
    const float bv = g.bias ? as_global(g.bias)[m] : 0.0f;
    float v[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        v[r] = g.alpha * acc[r];
        if (has_beta) v[r] += g.beta * prev[r];
        v[r] += bv;
    }
    if (P) {
        float NCHIP_GLOBAL *Pp = P + (int64_t)nb * g.ldc + m;
#pragma unroll
        for (int r = 0; r < 16; r++)
            if (ok[r]) Pp[(int64_t)nofs(r) * g.ldc] = v[r];
    }
    if (g.act == NCHIP_ACT_GELU) {
#pragma unroll
        for (int r = 0; r < 16; r++) v[r] = gelu_tanh(v[r]);
    } else if (g.act == ACT_GELU_FAST) {
#pragma unroll
        for (int r = 0; r < 16; r++) v[r] = nchip_gelu_fast(v[r]);
    } else if (g.act == NCHIP_ACT_RELU) {
#pragma unroll
        for (int r = 0; r < 16; r++) v[r] = v[r] > 0.0f ? v[r] : 0.0f;
    }
    if (Dp) { // gradient through an activation: times act'(pre-activation)
        const float NCHIP_GLOBAL *Dq = Dp + (int64_t)nb * g.ldc + m;
        float pz[16];
#pragma unroll
        for (int r = 0; r < 16; r++) pz[r] = ok[r] ? Dq[(int64_t)nofs(r) * g.ldc] : 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) v[r] = (v[r] + extra[r]) * act_grad(pz[r], g.dact);
#pragma unroll
        for (int r = 0; r < 16; r++)
            if (ok[r]) Cp[(int64_t)nofs(r) * g.ldc] = v[r];
        if (Hp) {
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (ok[r]) Hp[(int64_t)nofs(r) * g.ldc] = f32_to_bf16_rne(v[r]);
        }
        if (rowsum) { // this lane's 16 columns of row m, in column order: one entry of a partial row
            float sum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) sum += ok[r] ? v[r] : 0.0f;
            rowsum[m] = sum;
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < 16; r++) v[r] += extra[r];
#pragma unroll
    for (int r = 0; r < 16; r++)
        if (ok[r]) Cp[(int64_t)nofs(r) * g.ldc] = v[r];
    if (Hp) {
#pragma unroll
        for (int r = 0; r < 16; r++)
            if (ok[r]) Hp[(int64_t)nofs(r) * g.ldc] = f32_to_bf16_rne(v[r]);
    }
}

// Product with a few token columns for the width-invariant class: C (M x N, 32 columns per
// workgroup column) = A (M x K, m contiguous, M a multiple of 32) * B (K x N, k contiguous),
// fp32, K a multiple of 32, operand columns 16-byte aligned.  Per output element it issues
// exactly the MFMA sequence of the four-chain 64x64x32 tile kernel (gemm_kernel with
// NACC = 2: chain c takes k%32 in [8c, 8c+8), two k per v_mfma_f32_32x32x2_f32 in increasing
// order; C = (c0 + c1) + (c2 + c3); the same epilogue), so its columns are bit-identical to
// those of a wide product.  What differs is the plumbing.  A workgroup is one 32-row tile
// and its four wavefronts are the four chains, one per SIMD: the product then runs at the
// speed of one dependent MFMA chain of K/8 instructions, the least this arithmetic allows
// on one CU.  There is nothing to share between wavefronts, so the k loop has no barrier:
// a wavefront fetches its 8 k of every slab with ONE 16-byte load per lane and operand
// (8 x 32 rows of A, 32 columns x 8 k of B), PFD slabs ahead - at 2 microseconds of
// latency and 256 cycles of MFMA per slab the loads of 16 slabs must be in flight - and
// turns them into MFMA fragments through a private corner of LDS (in order within a
// wavefront, so a write followed by a read needs no barrier).  Columns past the edge read
// a clamped address and are never stored.
template <int PFD>
__global__ __launch_bounds__(256) void gemm_skinny_nn(GemmArgs g)
{
    static_assert(PFD % 2 == 0, "fragment registers alternate by slab parity");
    constexpr int AST = 36, BST = 12; // row strides of the staged slabs: A [8 k][32 m], B [32 n][8 k]
    __shared__ __attribute__((aligned(16))) float stage[4][8 * AST + 32 * BST];
    __shared__ float red[3][16 * 64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (blockIdx.z == 1) { // the pair's second product: its own A, C, bias and row count
        g.A = g.A_1; g.C = g.C_1; g.bias = g.bias_1; g.lda = g.lda_1; g.ldc = g.ldc_1; g.M = g.M_1;
    }
    const int m0 = blockIdx.x * 32, n0 = blockIdx.y * 32;
    if (m0 >= g.M) return; // (uniform: the grid covers the taller of the two products)
    const int kh = lane >> 5;
    const int ak = lane >> 3, am = (lane & 7) * 4; // this lane's k row and first of four rows m of the A slab
    const int bn = lane >> 1, bk = (lane & 1) * 4; // this lane's column and first of four k of the B slab
    const int bcol = n0 + bn < g.N ? n0 + bn : g.N - 1;
    const floatx4 NCHIP_GLOBAL *Ag = reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(
        as_global(g.A) + (int64_t)(8 * w + ak) * g.lda + m0 + am);
    const floatx4 NCHIP_GLOBAL *Bg = reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(
        as_global(g.B) + (int64_t)bcol * g.ldb + 8 * w + bk);
    const int64_t a_step = 8 * g.lda; // 32 k rows, in 16-byte units
    float *As = stage[w], *Bs = As + 8 * AST;
    floatx4 *aw = reinterpret_cast<floatx4 *>(As + ak * AST + am);
    floatx4 *bw = reinterpret_cast<floatx4 *>(Bs + bn * BST + bk);
    const float *ar = As + kh * AST + (lane & 31); // MFMA step s reads k = 2s + kh
    const float *br = Bs + (lane & 31) * BST + kh;
    const int nslab = g.K / 32;
    floatx4 ra[PFD], rb[PFD];
    // (register sets and fragment sets are passed by reference: every index below is a
    // constant once the loops are unrolled, so the arrays stay in registers)
    auto load = [&](floatx4 &a, floatx4 &b, int slab) {
        slab = slab < nslab ? slab : nslab - 1; // past the end: the last slab again, never used
        a = Ag[slab * a_step];
        b = Bg[slab * 8];
    };
    float fa[2][4], fb[2][4];
    auto stage_slab = [&](const floatx4 &a, const floatx4 &b, float (&xa)[4], float (&xb)[4]) { // registers -> LDS -> fragments
        *aw = a;
        *bw = b;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++) {
            xa[s4] = ar[2 * s4 * AST];
            xb[s4] = br[2 * s4];
        }
        __builtin_amdgcn_wave_barrier();
    };
#pragma unroll
    for (int j = 0; j < PFD; j++) {
        load(ra[j], rb[j], j);
        __builtin_amdgcn_sched_barrier(0); // oldest slab first, as on the back edge
    }
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    stage_slab(ra[0], rb[0], fa[0], fb[0]);
    load(ra[0], rb[0], PFD);
    for (int slab0 = 0; slab0 < nslab; slab0 += PFD) {
#pragma unroll
        for (int j = 0; j < PFD; j++) {
            // fragments of the next slab while the MFMAs of this one run
            stage_slab(ra[(j + 1) % PFD], rb[(j + 1) % PFD], fa[(j + 1) & 1], fb[(j + 1) & 1]);
            load(ra[(j + 1) % PFD], rb[(j + 1) % PFD], slab0 + j + 1 + PFD);
            __builtin_amdgcn_sched_barrier(0);
            if (slab0 + j < nslab) { // uniform
#pragma unroll
                for (int s4 = 0; s4 < 4; s4++)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j & 1][s4], fa[j & 1][s4], acc, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (w > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) red[w - 1][r * 64 + lane] = acc[r];
    }
    __syncthreads();
    if (w > 0) return;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = (acc[r] + red[0][r * 64 + lane]) + (red[1][r * 64 + lane] + red[2][r * 64 + lane]);
    const bool full = n0 + 32 <= g.N;
    float NCHIP_GLOBAL *P = g.pre ? as_global(g.pre) : nullptr;
    const float NCHIP_GLOBAL *Radd = g.add ? as_global(g.add) : nullptr;
    const float NCHIP_GLOBAL *Dp = g.dpre ? as_global(g.dpre) : nullptr;
    const bool plain = !g.bias && !P && !Radd && !Dp && g.beta == 0.0f && g.act == NCHIP_ACT_NONE;
    epilogue_tile(g, acc, m0 + (lane & 31), n0 + kh * 4, as_global(g.C), P, Radd, Dp, full, plain);
}

// The same few-column product on the vector ALUs.  An fp32 MFMA accumulates its k values
// one after the other with fused multiply-adds, in increasing k (checked bit for bit against
// v_mfma_f32_32x32x2_f32 chains, denormal products included), so an output element of the
// width-invariant class is four chains of K/4 dependent v_fma_f32 - chain c takes k%32 in
// [8c, 8c+8) - summed as (c0 + c1) + (c2 + c3).  A thread is one chain of one element: a
// workgroup of 256 threads owns an 8 x 8 tile of C (4 chains each), so a 512 x 32 product
// spreads over 256 workgroups instead of 16 and a chain costs K/4 FMAs (0.3 microseconds at
// K = 512) instead of K/8 MFMAs of 64 cycles.  Its 8 rows of A and 8 columns of B pass
// through LDS in chunks of 256 k ([row][k] with k contiguous, two buffers, one barrier per
// chunk); the loads of up to PF chunks are in flight from the start (K = 2048 whole), since
// one memory round trip is longer than all the arithmetic.  Bias and addend are fetched
// before the k loop.  alpha = 1, beta = 0, no activation gradient; M a multiple of 8.
// Row tile of workgroup x of a few-column kernel.  Consecutive workgroups go to the eight XCDs
// in turn, each with an L2 of its own, and a 128-byte line of A (32 rows of one k) spans R
// row tiles: the R tiles that share lines are given to workgroups of one XCD (x, x + 8, ...),
// so that a line is fetched into one L2 and not into R of them.
__device__ __forceinline__ int fewcol_row_tile(int x, int ntiles, int R)
{
    const int span = 8 * R, group = x / span;
    if ((group + 1) * span > ntiles) return x; // a last, partial group keeps its order
    const int in = x - group * span, xcd = in & 7, r = in >> 3;
    return group * span + xcd * R + r;
}

constexpr int FC_KC = 256, FC_RS = FC_KC + 4;
template <int PF>
__global__ __launch_bounds__(256) void gemm_fewcol_fma(GemmArgs g)
{
    __shared__ __attribute__((aligned(16))) float tile[2][16 * FC_RS]; // rows 0-7: A rows, 8-15: B columns
    const int t = threadIdx.x;
    if (blockIdx.z == 1) { // the pair's second product: its own A, C, bias and row count
        g.A = g.A_1; g.C = g.C_1; g.bias = g.bias_1; g.lda = g.lda_1; g.ldc = g.ldc_1; g.M = g.M_1;
    }
    const int m0 = fewcol_row_tile(blockIdx.x, gridDim.x, 4) * 8, n0 = blockIdx.y * 8;
    if (m0 >= g.M) return; // (uniform: the grid covers the taller of the two products)
    const int ch = t & 3, ei = (t >> 2) & 7, ej = t >> 5; // chain, row and column of this thread's element
    const int nslab = g.K / 32, nch = (g.K + FC_KC - 1) / FC_KC;
    // A chunk: 256 k x 8 rows = 512 16-byte pieces (k = piece / 2, four rows each);
    // B chunk: 8 columns x 256 k = 512 pieces (column = piece / 64, four k each)
    const int ak[2] = { t >> 1, (t + 256) >> 1 }, ah = (t & 1) * 4;
    const int bj[2] = { t >> 6, (t + 256) >> 6 }, bk = (t & 63) * 4;
    const float NCHIP_GLOBAL *Ab = as_global(g.A) + m0 + ah;
    const float NCHIP_GLOBAL *Bb[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int col = n0 + bj[u] < g.N ? n0 + bj[u] : g.N - 1;
        Bb[u] = as_global(g.B) + (int64_t)col * g.ldb;
    }
    floatx4 ra[PF][2], rb[PF][2];
    auto load = [&](floatx4 (&a)[2], floatx4 (&b)[2], int q) { // past the end: clamped, never used
#pragma unroll
        for (int u = 0; u < 2; u++) {
            int ka = q * FC_KC + ak[u], kb = q * FC_KC + bk;
            ka = ka < g.K ? ka : g.K - 1;
            kb = kb < g.K ? kb : g.K - 4;
            a[u] = *reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(Ab + (int64_t)ka * g.lda);
            b[u] = *reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(Bb[u] + kb);
        }
    };
#pragma unroll
    for (int j = 0; j < PF; j++) {
        load(ra[j], rb[j], j);
        __builtin_amdgcn_sched_barrier(0); // oldest chunk first
    }
    const int row = m0 + ei, col = n0 + ej;
    const bool ok = col < g.N;
    float NCHIP_GLOBAL *P = g.pre ? as_global(g.pre) : nullptr;
    const float NCHIP_GLOBAL *Radd = g.add ? as_global(g.add) : nullptr;
    const bool plain = !g.bias && !P && !Radd && g.act == NCHIP_ACT_NONE;
    const float bv = g.bias ? as_global(g.bias)[row] : 0.0f;
    const float extra = (Radd && ok) ? Radd[(int64_t)col * g.ldc + row] : 0.0f;
    auto park = [&](const floatx4 (&a)[2], const floatx4 (&b)[2], float *dst) { // registers -> [row][k]
#pragma unroll
        for (int u = 0; u < 2; u++) {
#pragma unroll
            for (int r = 0; r < 4; r++) dst[(ah + r) * FC_RS + ak[u]] = a[u][r];
            *reinterpret_cast<floatx4 *>(dst + (8 + bj[u]) * FC_RS + bk) = b[u];
        }
    };
    float acc = 0.0f;
    for (int q0 = 0; q0 < nch; q0 += PF) {
#pragma unroll
        for (int j = 0; j < PF; j++) {
            const int q = q0 + j;
            if (q < nch) { // uniform
                float *buf = tile[q & 1];
                park(ra[j], rb[j], buf);
                load(ra[j], rb[j], q + PF);
                __syncthreads();
                const float *wr = buf + ei * FC_RS + 8 * ch, *xr = buf + (8 + ej) * FC_RS + 8 * ch;
                const int ns = nslab - 8 * q < 8 ? nslab - 8 * q : 8;
                auto slab = [&](int s) {
                    const floatx4 w0 = *reinterpret_cast<const floatx4 *>(wr + 32 * s);
                    const floatx4 w1 = *reinterpret_cast<const floatx4 *>(wr + 32 * s + 4);
                    const floatx4 x0 = *reinterpret_cast<const floatx4 *>(xr + 32 * s);
                    const floatx4 x1 = *reinterpret_cast<const floatx4 *>(xr + 32 * s + 4);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc = __builtin_fmaf(x0[r], w0[r], acc);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc = __builtin_fmaf(x1[r], w1[r], acc);
                };
                if (ns == 8) { // a whole chunk, unrolled: the LDS reads run ahead of the chain
#pragma unroll
                    for (int s = 0; s < 8; s++) slab(s);
                } else {
                    for (int s = 0; s < ns; s++) slab(s);
                }
            }
        }
    }
    // (c0 + c1) + (c2 + c3): the four chains of an element sit in four neighbouring lanes
    float v = acc + __shfl_xor(acc, 1, 64);
    v = v + __shfl_xor(v, 2, 64);
    if (ch != 0 || !ok) return;
    float NCHIP_GLOBAL *Cp = as_global(g.C) + (int64_t)col * g.ldc + row;
    if (plain) {
        *Cp = g.alpha * v;
        return;
    }
    v = g.alpha * v + bv;
    if (P) P[(int64_t)col * g.ldc + row] = v;
    v = apply_act(v, g.act);
    *Cp = v + extra;
}

// The few-column product with v_mfma_f32_16x16x4_f32.  That instruction accumulates its
// four k in increasing order like the 32x32x2 one its two, at a quarter of the chain latency
// per k (a 16x16 tile: 8 passes per 4 k instead of 16 passes per 2 k), so chain c of a slab
// is two of them (k%32 = 8c..8c+3, 8c+4..8c+7) and the result is again the bits of the tile
// kernel.  A workgroup is a 16 x 16 tile of C and its four wavefronts are the four chains
// (combined as (c0 + c1) + (c2 + c3) through LDS at the end); a wavefront fetches only the
// 8 k per slab of its own chain - 16 rows of A and 16 columns of B, in chunks of 256 k, up
// to PF chunks in flight - into a private corner of LDS and reads its fragments from there,
// so the k loop has no workgroup barrier.  Against the vector-ALU kernel: a quarter of the
// workgroups, but 1 KB of LDS reads per slab and wavefront for 256 outputs instead of 4 KB
// for 16, which is what bounds that kernel on the taller products.  alpha = 1, beta = 0.
//
// NV > 0: B holds K = 64 NV raw features per column and the product is taken with their
// layer norm (or RMS norm) - the arithmetic of norm_fwd_reg, wavefront c normalising columns
// 4c..4c+3 of the tile before the k loop, the result kept whole in LDS (every workgroup
// repeats it for its 16 columns, which costs less than a launch of its own); the first row
// tile also writes the normalised columns out for the later consumers of that tensor.
//
// TR = 8: tiles of 8 x 8 outputs on the same instruction (rows and columns 8-15 of the MFMA
// tile repeat 0-7 and are not stored): four times the workgroups, for a long reduction and for
// products that would otherwise leave most CUs idle.  What bounds these kernels is not the
// chain (0.85 microseconds per 1024 k) but the 128-byte lines a workgroup must bring in, at
// about 0.4 lines per nanosecond and CU, with warm or cold weights alike: a launch costs about
// 2.6 microseconds plus 2.3 nanoseconds per line of its busiest workgroup.  With A stored
// rows-contiguous that is one line of A per k whatever the tile height up to 32 rows.
//
// AK = 1: A is stored with k contiguous (lda between rows: a k-major copy of a weight matrix).
// The lines a workgroup brings in for A are then TR x K/32 instead of K, which is what the
// kernel is bound by; the arithmetic is the same.
template <int PF, int NV = 0, int TR = 16, int AK = 0>
__global__ __launch_bounds__(256) void gemm_fewcol_mfma(GemmArgs g)
{
    static_assert(TR == 16 || (TR == 8 && NV == 0), "8 x 8 tiles: plain products only");
    constexpr int NU = TR / 4; // 16-byte pieces per lane, chunk and operand
    constexpr int BST = 68, ASZ = AK ? TR * BST : 64 * TR; // per wavefront: A [64 k][TR rows] (AK: [TR rows][64 k]), B [TR columns][64 k]
    constexpr int WSZ = ASZ + (NV ? 0 : TR * BST);
    constexpr int XS = 64 * NV + 4;
    __shared__ __attribute__((aligned(16))) float stage[4][WSZ];
    __shared__ float red[4][4 * 64];
    __shared__ float xn[NV ? 16 * XS : 1]; // normalised B: [16 columns][K]
    const int lane = threadIdx.x & 63, c = threadIdx.x >> 6; // wavefront = chain
    if (blockIdx.z == 1) { // the pair's second product: its own A, C, bias and row count
        g.A = g.A_1; g.C = g.C_1; g.bias = g.bias_1; g.lda = g.lda_1; g.ldc = g.ldc_1; g.M = g.M_1;
    }
    const int m0 = fewcol_row_tile(blockIdx.x, gridDim.x, 32 / TR) * TR, n0 = blockIdx.y * TR;
    if (m0 >= g.M) return; // (uniform: the grid covers the taller of the two products)
    const int il = lane & 15, gq = lane >> 4, it = il & (TR - 1); // (it: this lane's row / column of the tile)
    const int nslab = g.K / 32, nch = (g.K + 255) / 256;
    float *As = stage[c], *Bs = As + ASZ;
    // this lane's NU 16-byte pieces of A (k_local = piece / NU, four rows) and of B
    // (column = piece / 16, slab = (piece % 16) / 2, half a chain's 8 k)
    const float NCHIP_GLOBAL *Ab = as_global(g.A) + m0 + (lane & (NU - 1)) * 4;
    const float NCHIP_GLOBAL *Ar[NU]; // AK: the row of each piece (pieces laid out as those of B)
    const float NCHIP_GLOBAL *Bb[NU];
    int a_k[NU], b_k[NU];
#pragma unroll
    for (int u = 0; u < NU; u++) {
        const int pa = lane + 64 * u, kl = pa / NU;
        a_k[u] = 32 * (kl >> 3) + 8 * c + (kl & 7);
        const int pb = lane + 64 * u, colb = pb >> 4, kq = pb & 15;
        const int col = n0 + colb < g.N ? n0 + colb : g.N - 1;
        Bb[u] = as_global(g.B) + (int64_t)col * g.ldb;
        b_k[u] = 32 * (kq >> 1) + 8 * c + 4 * (kq & 1);
        Ar[u] = as_global(g.A) + (int64_t)(m0 + colb) * g.lda;
    }
    floatx4 ra[PF][NU], rb[NV ? 1 : PF][NU];
    auto load = [&](floatx4 (&a)[NU], floatx4 (&b)[NU], int q) { // past the end: clamped, never used
#pragma unroll
        for (int u = 0; u < NU; u++) {
            int ka = q * 256 + a_k[u], kb = q * 256 + b_k[u];
            ka = ka < g.K ? ka : g.K - 1;
            kb = kb < g.K ? kb : g.K - 4;
            if (AK) a[u] = *reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(Ar[u] + kb);
            else a[u] = *reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(Ab + (int64_t)ka * g.lda);
            if (NV == 0) b[u] = *reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(Bb[u] + kb);
        }
    };
    // the raw columns first: they are needed first
    float xv[NV ? 4 : 1][NV ? NV : 1], lw[NV ? NV : 1], lb[NV ? NV : 1];
    if (NV > 0) {
#pragma unroll
        for (int cc = 0; cc < 4; cc++) {
            const int colb = 4 * c + cc, gcol = n0 + colb < g.N ? n0 + colb : g.N - 1;
            const float NCHIP_GLOBAL *xc = as_global(g.B) + (int64_t)gcol * g.ldb + lane;
#pragma unroll
            for (int v = 0; v < NV; v++) xv[cc][v] = xc[64 * v];
        }
        if (g.ln_w) {
#pragma unroll
            for (int v = 0; v < NV; v++) { lw[v] = as_global(g.ln_w)[lane + 64 * v]; lb[v] = as_global(g.ln_b)[lane + 64 * v]; }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < PF; j++) {
        load(ra[j], rb[NV ? 0 : j], j);
        __builtin_amdgcn_sched_barrier(0); // oldest chunk first
    }
    if constexpr (NV > 0) {
        float hh[4][NV], yy[4][NV], rr[4];
        norm_columns_reg<NV, 4>(xv, lw, lb, g.ln_w != nullptr, g.ln_eps, g.ln_avg, hh, yy, rr);
#pragma unroll
        for (int cc = 0; cc < 4; cc++) {
            const int colb = 4 * c + cc;
#pragma unroll
            for (int v = 0; v < NV; v++) xn[colb * XS + lane + 64 * v] = yy[cc][v];
            if (g.ln_out && blockIdx.x == 0 && blockIdx.z == 0 && n0 + colb < g.N) {
                float NCHIP_GLOBAL *yo = as_global(g.ln_out) + (int64_t)(n0 + colb) * g.ld_ln + lane;
#pragma unroll
                for (int v = 0; v < NV; v++) yo[64 * v] = yy[cc][v];
            }
        }
        __syncthreads();
    }
    // epilogue operands, fetched before the k loop: wavefront c finishes row 4 gq + c of the
    // four rows a lane holds (the four chains of an element meet through LDS either way, and
    // bias, activation and addend then take a quarter of the time on each wavefront)
    const int col = n0 + il, row = m0 + 4 * gq + c;
    const bool ok = col < g.N && il < TR && gq < TR / 4; // (8 x 8 tiles: the repeated rows and columns are not stored)
    float NCHIP_GLOBAL *P = g.pre ? as_global(g.pre) : nullptr;
    const float NCHIP_GLOBAL *Radd = g.add ? as_global(g.add) : nullptr;
    const bool plain = !g.bias && !P && !Radd && g.act == NCHIP_ACT_NONE;
    const float bv = (g.bias && gq < TR / 4) ? as_global(g.bias)[row] : 0.0f;
    const float extra = (Radd && ok) ? Radd[(int64_t)col * g.ldc + row] : 0.0f;
    floatx4 acc = { 0, 0, 0, 0 };
    for (int q0 = 0; q0 < nch; q0 += PF) {
#pragma unroll
        for (int j = 0; j < PF; j++) {
            const int q = q0 + j;
            if (q < nch) { // uniform
#pragma unroll
                for (int u = 0; u < NU; u++) {
                    const int pa = lane + 64 * u;
                    if (AK) *reinterpret_cast<floatx4 *>(As + (pa >> 4) * BST + (pa & 15) * 4) = ra[j][u];
                    else *reinterpret_cast<floatx4 *>(As + (pa / NU) * TR + (pa & (NU - 1)) * 4) = ra[j][u];
                    if (NV == 0) *reinterpret_cast<floatx4 *>(Bs + (pa >> 4) * BST + (pa & 15) * 4) = rb[j][u];
                }
                load(ra[j], rb[NV ? 0 : j], q + PF);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                float fa[16], fb[16];
#pragma unroll
                for (int e = 0; e < 16; e++) { // MFMA e of the chunk: slab e / 2, k_local = 4 e + gq
                    fa[e] = AK ? As[it * BST + 4 * e + gq] : As[(4 * e + gq) * TR + it];
                    int kx = 256 * q + 32 * (e >> 1) + 8 * c + 4 * (e & 1) + gq;
                    kx = kx < g.K ? kx : g.K - 1; // (past a short last chunk: read, never used)
                    fb[e] = NV ? xn[il * XS + kx] : Bs[it * BST + 4 * e + gq];
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier(); // the fragments are in registers: the corner may be rewritten
                const int ne = (nslab - 8 * q < 8 ? nslab - 8 * q : 8) * 2;
                if (ne == 16) {
#pragma unroll
                    for (int e = 0; e < 16; e++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[e], fb[e], acc, 0, 0, 0);
                } else {
#pragma unroll
                    for (int e = 0; e < 16; e++)
                        if (e < ne) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[e], fb[e], acc, 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) red[c][r * 64 + lane] = acc[r];
    __syncthreads();
    if (!ok) return;
    // lane (il, gq) of wavefront c finishes row m0 + 4 gq + c of column n0 + il: (c0 + c1) + (c2 + c3)
    const float sum = (red[0][c * 64 + lane] + red[1][c * 64 + lane]) + (red[2][c * 64 + lane] + red[3][c * 64 + lane]);
    float NCHIP_GLOBAL *Cp = as_global(g.C) + (int64_t)col * g.ldc + row;
    if (plain) {
        *Cp = g.alpha * sum;
        return;
    }
    float v = g.alpha * sum + bv;
    if (P) P[(int64_t)col * g.ldc + row] = v;
    v = apply_act(v, g.act);
    *Cp = v + extra;
}

// KW = 2 doubles the wavefronts of a workgroup without shrinking its tile: the
// two groups of WM x WN wavefronts share the LDS tiles and split every 32-deep
// k slab, group 0 taking k%32 < 16 and group 1 the rest; group 1 hands its
// accumulators over through LDS at the end (C = chain0 + chain1, fixed order).
// NACC = 2 (the width-invariant class): each k group keeps two accumulator sets and gives
// the first four MFMA steps of every 32-deep slab to one, the last four to the other, so a
// product is four chains - chain c takes k%32 in [8c, 8c+8) - summed as (c0 + c1) + (c2 + c3).
// The products are the same; the order of the additions is what a kernel with four
// wavefronts per row tile can reproduce (gemm_skinny_nn).
template <int BM, int BN, int BK, int WM, int WN, int TA, int TB, int BF16, int KW = 1, int PF = 2, int SA = (BF16 == 2), int NACC = 1, int FRAG = 0>
__global__ __launch_bounds__(64 * WM * WN * KW) void gemm_kernel(GemmArgs g0)
{
    GemmArgs g = g0;
    static_assert(NACC == 1 || (NACC == 2 && BF16 == 0 && KW == 2 && BK == 32), "two accumulator sets: fp32 64-wide class only");
    static_assert(KW == 1 || (KW == 2 && BK % 32 == 0), "k groups split 32-deep slabs");
    constexpr int NT = 64 * WM * WN * KW;                 // threads: KW groups of WM x WN wavefronts
    constexpr int TM = BM / (32 * WM), TN = BN / (32 * WN); // 32x32 MFMA tiles per wavefront
    constexpr int WTM = BM / WM, WTN = BN / WN;           // wavefront tile
    // in 32-bit words; bf16 sources with k contiguous keep rows of BK/2 + 4 words
    constexpr int SQ = BK / 2 + 4;
    // fp32 row strides of the LDS tiles (see TileLoader)
    constexpr int RSA = BM + (TA ? FPAD_K : PAD), RSB = BN + (TB ? PAD : FPAD_K);
    constexpr int LDS_A = BF16 == 2 && TA ? BM * SQ : (BF16 ? (BK / 2) * (BM + PAD) : BK * RSA);
    constexpr int LDS_B = BF16 == 2 && !TB ? BN * SQ : (BF16 ? (BK / 2) * (BN + PAD) : BK * RSB);
    static_assert(KW == 1 || BM * BN <= 2 * (LDS_A + LDS_B), "accumulator hand-over must fit in the tile buffers");
    // tile buffers above the 64 KiB a static array may take come from the
    // launch's dynamic allocation instead
    constexpr bool BIG_LDS = 2 * (LDS_A + LDS_B) * 4 > 65536;
    __shared__ __attribute__((aligned(16))) float smem_static[BIG_LDS ? 4 : 2 * (LDS_A + LDS_B)];
    extern __shared__ __attribute__((aligned(16))) float smem_dynamic[];
    float *const smem = BIG_LDS ? smem_dynamic : smem_static;

    const int t = threadIdx.x, lane = t & 63;
    const int kg = (t >> 6) / (WM * WN), wave = (t >> 6) % (WM * WN);
    const int wm = wave % WM, wn = wave / WM;

    // XCD-aware tile order: the hardware deals consecutive workgroup ids round
    // robin over the 8 XCDs; give each XCD a contiguous run of tiles so tiles
    // that share an A/B panel also share an L2.
    int bid = blockIdx.x;
    // second k range of a grouped problem: k tiles from k1 on read A2 / B2
    const float *A2 = nullptr, *B2 = nullptr;
    int k1 = 0x7fffffff;
    if (g.grp) {
        // grouped launch: consecutive workgroup ids go to the XCDs in turn; hand each XCD
        // GC consecutive tiles of the list at a time (neighbours in a tile column, which share
        // a B panel in that XCD's L2) while the turn-taking keeps the XCDs' work balanced
        {
            const int GC = g.grp_chunk;
            const int total = gridDim.x, span = NXCD * GC;
            if (GC > 1 && (bid / span + 1) * span <= total) {
                const int in = bid % span, x = in % NXCD, slot = in / NXCD;
                bid = (bid / span) * span + x * GC + slot;
            }
        }
        // find the problem that owns this workgroup
        int lo = 0, hi = g.n_grp; // grp[lo].tile_start <= bid < grp[hi].tile_start
        while (hi - lo > 1) {
            int mid = (lo + hi) >> 1;
            if (g.grp[mid].tile_start <= bid) lo = mid; else hi = mid;
        }
        const NchipGemmProblem pr = g.grp[lo];
        bid -= pr.tile_start;
        g.A = pr.A; g.B = pr.B; g.C = pr.C;
        g.M = pr.m; g.N = pr.n; g.K = pr.k + pr.k2;
        if (pr.k2 > 0) { A2 = pr.A2; B2 = pr.B2; k1 = pr.k; }
        g.lda = pr.lda; g.ldb = pr.ldb; g.ldc = pr.ldc;
        g.alpha = pr.alpha;
        g.kchunk = pr.k + pr.k2;
        g.tiles_m = (pr.m + BM - 1) / BM;
        g.tiles_n = (pr.n + BN - 1) / BN;
    }
    int ntiles = g.tiles_m * g.tiles_n;
    if (!g.grp && ntiles % NXCD == 0)
        bid = (bid % NXCD) * (ntiles / NXCD) + bid / NXCD;
    // Tile order inside an XCD's run: bands of gm tile rows, column by column
    // inside a band, so the workgroups in flight on one XCD form a block about
    // as wide as it is tall and share both A and B panels in that XCD's L2.
    int tile_m, tile_n;
    if (g.gm > 1) {
        const int band = g.gm * g.tiles_n, bi = bid / band, first = bi * g.gm;
        const int rows = min(g.tiles_m - first, g.gm), r = bid - bi * band;
        tile_m = first + r % rows;
        tile_n = r / rows;
    } else {
        tile_m = bid % g.tiles_m;
        tile_n = bid / g.tiles_m;
    }
    const int bz = blockIdx.y;
    const int b = bz / g.ksplit, kz = bz % g.ksplit;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int kbeg = kz * g.kchunk;
    const int kend = min(g.K, kbeg + g.kchunk);

    const int b_out = b / g.batch_in, b_in = b % g.batch_in;
    const float *A = g.A + (int64_t)b_out * g.sa + (int64_t)b_in * g.sa_in;
    const float *B = g.B + (int64_t)b_out * g.sb + (int64_t)b_in * g.sb_in;

    // fast (vector, unguarded) loads need whole tiles and 16-byte alignment
    // (bf16 sources are padded and aligned by construction: always fast)
    const bool a_full = BF16 == 2 || ((m0 + BM <= g.M) && (g.lda % 4 == 0) && (((uintptr_t)A & 15) == 0));
    const bool b_full = BF16 == 2 || ((n0 + BN <= g.N) && (g.ldb % 4 == 0) && (((uintptr_t)B & 15) == 0));

    // PF register sets: while tile it is computed, tiles it+1 .. it+PF are landing
    // or in flight, so a load has PF compute phases to arrive.  Two sets are
    // enough for the wide classes; the 64x64 class, whose tiles are consumed in
    // half the time, keeps four.
    using LoaderA = std::conditional_t<BF16 == 2, TileLoaderBf16Src<BM, BK, TA ? 0 : 1, NT>,
                    std::conditional_t<BF16 == 1, TileLoaderBf16<BM, BK, TA ? 0 : 1, NT>, TileLoader<BM, BK, TA ? 0 : 1, NT>>>;
    using LoaderB = std::conditional_t<BF16 == 2, TileLoaderBf16Src<BN, BK, TB ? 1 : 0, NT>,
                    std::conditional_t<BF16 == 1, TileLoaderBf16<BN, BK, TB ? 1 : 0, NT>, TileLoader<BN, BK, TB ? 1 : 0, NT>>>;
    LoaderA la[PF];
    LoaderB lb[PF];

    floatx16 acc[TN][TM], acc2[TN][TM]; // acc2: second chain of a k group (NACC = 2)
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = acc2[i][j][r] = 0.0f;

    // One pipeline step: write the register set holding tile `it` to LDS buffer
    // it&1, barrier, refill that set with tile it+PF (when there is one), then
    // the MFMAs of tile `it`.  One barrier per tile is enough because a buffer
    // is rewritten only two tiles later.  FAST is a compile-time flag so the
    // steady-state loop carries no guarded-load code: the guarded path shares
    // registers with the vector loads and the compiler then serialises every
    // prefetch behind an s_waitcnt vmcnt(0).
    // the MFMAs of the tile held in LDS at sa / sb
    auto compute = [&](const float *sa, const float *sb) {
        if constexpr (BF16 != 0) {
            // one 32x32x16 MFMA per tile pair per 16 k; group kg takes every KW-th block
            const uint32_t *wa = reinterpret_cast<const uint32_t *>(sa) + (lane >> 5) * 4 * (BM + PAD) + wm * WTM + (lane & 31);
            const uint32_t *wb = reinterpret_cast<const uint32_t *>(sb) + (lane >> 5) * 4 * (BN + PAD) + wn * WTN + (lane & 31);
#pragma unroll
            for (int u = 0; u < BK / 16 / KW; u++) {
                const int row0 = (u * KW + kg) * 8; // word row of this 16-k block
                u32x4 fa[TM], fb[TN];
#pragma unroll
                for (int j = 0; j < TM; j++) {
                    if constexpr (BF16 == 2 && TA != 0) { // k-contiguous rows: one 16-byte read
                        fa[j] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const uint32_t *>(sa) +
                                (wm * WTM + j * 32 + (lane & 31)) * SQ + row0 + (lane >> 5) * 4);
                    } else {
                        const uint32_t *q = wa + row0 * (BM + PAD) + j * 32;
                        fa[j] = u32x4{ q[0], q[BM + PAD], q[2 * (BM + PAD)], q[3 * (BM + PAD)] };
                    }
                }
#pragma unroll
                for (int i = 0; i < TN; i++) {
                    if constexpr (BF16 == 2 && TB == 0) {
                        fb[i] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const uint32_t *>(sb) +
                                (wn * WTN + i * 32 + (lane & 31)) * SQ + row0 + (lane >> 5) * 4);
                    } else {
                        const uint32_t *q = wb + row0 * (BN + PAD) + i * 32;
                        fb[i] = u32x4{ q[0], q[BN + PAD], q[2 * (BN + PAD)], q[3 * (BN + PAD)] };
                    }
                }
#pragma unroll
                for (int i = 0; i < TN; i++)
#pragma unroll
                    for (int j = 0; j < TM; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(__attribute__((ext_vector_type(8))) __bf16, fb[i]),
                            __builtin_bit_cast(__attribute__((ext_vector_type(8))) __bf16, fa[j]),
                            acc[i][j], 0, 0, 0);
            }
        } else {
            // The k-steps of a tile go in chunks of CH: the fragments of chunk c+1 are read
            // from LDS (into the other half of fa / fb) before the MFMAs of chunk c are issued,
            // and a scheduling fence keeps them there - left alone, the scheduler sinks every
            // read next to its use and each MFMA pair then waits a full LDS round trip.
            // LDS row of step u: 2u (KW = 1), or the u-th pair of this group's half of each
            // 32-deep slab (KW = 2).
            constexpr int NSTEP = BK / 2 / KW;
            auto krow = [](int u) { return KW == 1 ? 2 * u : (u >> 3) * 32 + 2 * (u & 7); };
            constexpr int CH = NSTEP < 4 ? NSTEP : 4, NCH = NSTEP / CH;
            static_assert(NSTEP % CH == 0, "whole chunks");
            float fa[2][CH][TM], fb[2][CH][TN];
            const float *pa = sa + ((lane >> 5) + kg * 16) * RSA + wm * WTM + (lane & 31);
            const float *pb = sb + ((lane >> 5) + kg * 16) * RSB + wn * WTN + (lane & 31);
            // Issue order: with two accumulator sets the steps of the two chains alternate
            // (chain A's step p, chain B's step p, ...), so consecutive MFMAs never depend on
            // each other; each chain still sees its own steps in increasing k order.
            auto stepof = [](int v) { return NACC == 2 ? (v & 1) * 4 + (v >> 1) : v; };
            auto fetch_chunk = [&](int c, int buf) {
#pragma unroll
                for (int u = 0; u < CH; u++) {
#pragma unroll
                    for (int j = 0; j < TM; j++) fa[buf][u][j] = pa[krow(stepof(c * CH + u)) * RSA + j * 32];
#pragma unroll
                    for (int i = 0; i < TN; i++) fb[buf][u][i] = pb[krow(stepof(c * CH + u)) * RSB + i * 32];
                }
            };
            if constexpr (FRAG == 1) {
                // rolling window instead of chunks: the fragments of step u+3 are read while
                // the MFMAs of step u run, and the scheduler is left to place them (wavefronts
                // that own two or more accumulator tiles have enough MFMA time per step)
                static_assert(NACC == 1, "the rolling window feeds one accumulator set");
                constexpr int FD = NSTEP < 4 ? NSTEP : 4;
                float ga[FD][TM], gb[FD][TN];
#pragma unroll
                for (int u = 0; u < FD - 1; u++) {
#pragma unroll
                    for (int j = 0; j < TM; j++) ga[u][j] = pa[krow(u) * RSA + j * 32];
#pragma unroll
                    for (int i = 0; i < TN; i++) gb[u][i] = pb[krow(u) * RSB + i * 32];
                }
#pragma unroll
                for (int u = 0; u < NSTEP; u++) {
                    const int cur = u % FD, nxt = (u + FD - 1) % FD;
                    if (u + FD - 1 < NSTEP) {
#pragma unroll
                        for (int j = 0; j < TM; j++) ga[nxt][j] = pa[krow(u + FD - 1) * RSA + j * 32];
#pragma unroll
                        for (int i = 0; i < TN; i++) gb[nxt][i] = pb[krow(u + FD - 1) * RSB + i * 32];
                    }
#pragma unroll
                    for (int i = 0; i < TN; i++)
#pragma unroll
                        for (int j = 0; j < TM; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(gb[cur][i], ga[cur][j], acc[i][j], 0, 0, 0);
                }
                return;
            }
            fetch_chunk(0, 0);
#pragma unroll
            for (int c = 0; c < NCH; c++) {
                if (c + 1 < NCH) fetch_chunk(c + 1, (c + 1) & 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < CH; u++)
#pragma unroll
                    for (int i = 0; i < TN; i++)
#pragma unroll
                        for (int j = 0; j < TM; j++) {
                            if (NACC == 2 && stepof(c * CH + u) >= 4) // steps 4..7 of the slab: the group's second chain
                                acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[c & 1][u][i], fa[c & 1][u][j], acc2[i][j], 0, 0, 0);
                            else
                                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[c & 1][u][i], fa[c & 1][u][j], acc[i][j], 0, 0, 0);
                        }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    auto step = [&](int it, int nk, auto fast_tag, auto &la, auto &lb) {
        constexpr bool FAST = decltype(fast_tag)::value;
        float *sa = smem + (it & 1) * (LDS_A + LDS_B);
        float *sb = sa + LDS_A;
        if constexpr (BF16 != 0) {
            la.store(reinterpret_cast<uint32_t *>(sa), t);
            lb.store(reinterpret_cast<uint32_t *>(sb), t);
        } else {
            la.store_f32(sa, t);
            lb.store_f32(sb, t);
        }
        __syncthreads();
        if (FAST || it + PF < nk) {
            int k0 = kbeg + (it + PF) * BK;
            bool kf = FAST || (k0 + BK <= kend);
            const bool second = k0 >= k1; // uniform
            const float *Ak = second ? A2 : A, *Bk = second ? B2 : B;
            const int kr = second ? k0 - k1 : k0, ke = second ? kend - k1 : (kend < k1 ? kend : k1);
            la.load(Ak, g.lda, m0, kr, g.M, ke, FAST || (a_full && kf), t);
            lb.load(Bk, g.ldb, n0, kr, g.N, ke, FAST || (b_full && kf), t);
        }
        // keep the prefetch ahead of the MFMAs: without this fence the
        // scheduler sinks the global loads below the compute block and their
        // latency is paid in full at the next LDS write
        __builtin_amdgcn_sched_barrier(0);
        compute(sa, sb);
    };

#ifdef NCHIP_GEMM_CLOCKS
    long long dbg_c0 = clock64(), dbg_w0 = wall_clock64();
#endif
    const int nk = (kend - kbeg + BK - 1) / BK;
    const int nk_full = (kend - kbeg) / BK; // tiles with a complete k range
    if constexpr (SA != 0) {
        // Store-ahead order: the LDS writes of the next tile go out BEFORE the
        // MFMAs of the current one (into the other buffer, which every
        // wavefront left at the last barrier) and overlap with them; one
        // barrier per tile, after the MFMAs.  Register set (i % PF) holds tile
        // i from its load until that write; it is reloaded with tile i + PF
        // right after.
        auto fetch = [&](int tile, auto fast_tag, auto &la, auto &lb) {
            constexpr bool FAST = decltype(fast_tag)::value;
            const int k0 = kbeg + tile * BK;
            const bool kf = FAST || (k0 + BK <= kend);
            const bool second = k0 >= k1; // uniform
            const float *Ak = second ? A2 : A, *Bk = second ? B2 : B;
            const int kr = second ? k0 - k1 : k0, ke = second ? kend - k1 : (kend < k1 ? kend : k1);
            la.load(Ak, g.lda, m0, kr, g.M, ke, FAST || (a_full && kf), t);
            lb.load(Bk, g.ldb, n0, kr, g.N, ke, FAST || (b_full && kf), t);
        };
        auto park = [&](int tile, auto &la, auto &lb) {
            float *sa = smem + (tile & 1) * (LDS_A + LDS_B);
            if constexpr (BF16 != 0) {
                la.store(reinterpret_cast<uint32_t *>(sa), t);
                lb.store(reinterpret_cast<uint32_t *>(sa + LDS_A), t);
            } else {
                la.store_f32(sa, t);
                lb.store_f32(sa + LDS_A, t);
            }
        };
        auto body = [&](int cur, auto fast_tag, auto &na, auto &nb) {
            constexpr bool FAST = decltype(fast_tag)::value;
            if (FAST || cur + 1 < nk) {
                park(cur + 1, na, nb);
                if (FAST || cur + 1 + PF < nk) fetch(cur + 1 + PF, fast_tag, na, nb);
            }
            __builtin_amdgcn_sched_barrier(0);
            const float *sa = smem + (cur & 1) * (LDS_A + LDS_B);
            compute(sa, sa + LDS_A);
            __syncthreads();
        };
        int it = 0;
        if (a_full && b_full && 2 * PF < nk_full) {
            // Steady state: every tile fetched here is complete.  The first PF + 1 tiles are
            // fetched by the same straight-line sequence as inside the loop, with nothing
            // conditional between them and the loop: the compiler then sees one and the same
            // queue of outstanding loads on entry and on the back edge and waits for the
            // oldest register set only (s_waitcnt vmcnt(n)).  With a conditional fetch in
            // front of the loop it assumes the worst path and drains every load in flight at
            // the top of each trip - which is what the prefetch is there to avoid.
#pragma unroll
            for (int j = 0; j < PF; j++) {
                fetch(j, std::true_type(), la[j], lb[j]);
                __builtin_amdgcn_sched_barrier(0); // oldest tile first, as on the back edge
            }
            park(0, la[0], lb[0]);
            fetch(PF, std::true_type(), la[0], lb[0]);
            __syncthreads();
            for (; it + 2 * PF < nk_full; it += PF) {
#pragma unroll
                for (int j = 0; j < PF; j++) body(it + j, std::true_type(), la[(j + 1) % PF], lb[(j + 1) % PF]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < PF; j++)
                if (j < nk) fetch(j, std::false_type(), la[j], lb[j]);
            if (nk > 0) park(0, la[0], lb[0]);
            if (PF < nk) fetch(PF, std::false_type(), la[0], lb[0]);
            __syncthreads();
        }
        for (; it < nk; it += PF) {
#pragma unroll
            for (int j = 0; j < PF; j++)
                if (it + j < nk) body(it + j, std::false_type(), la[(j + 1) % PF], lb[(j + 1) % PF]);
        }
    } else {
    int it = 0;
    if (a_full && b_full && 2 * PF - 1 < nk_full) {
        // steady state: tiles it+PF .. it+2PF-1 are complete, unguarded vector loads.  The
        // first PF tiles are fetched by the same straight-line vector loads as inside the
        // loop: the compiler then sees one and the same sequence of outstanding loads on
        // entry and on the back edge and waits for the oldest register set only
        // (s_waitcnt vmcnt(n)) instead of for everything in flight.
#pragma unroll
        for (int j = 0; j < PF; j++) {
            la[j].load(A, g.lda, m0, kbeg + j * BK, g.M, kend, true, t);
            lb[j].load(B, g.ldb, n0, kbeg + j * BK, g.N, kend, true, t);
            __builtin_amdgcn_sched_barrier(0); // oldest tile first, as on the back edge
        }
        for (; it + 2 * PF - 1 < nk_full; it += PF) {
#pragma unroll
            for (int j = 0; j < PF; j++) step(it + j, nk, std::true_type(), la[j], lb[j]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < PF; j++)
            if (j < nk) {
                bool kf = nk_full > j;
                la[j].load(A, g.lda, m0, kbeg + j * BK, g.M, kend, a_full && kf, t);
                lb[j].load(B, g.ldb, n0, kbeg + j * BK, g.N, kend, b_full && kf, t);
            }
    }
    for (; it < nk; it++) { // edge tiles and the k tail (it is a multiple of PF when the loop starts)
#pragma unroll
        for (int j = 0; j < PF; j++)
            if (it % PF == j) step(it, nk, std::false_type(), la[j], lb[j]);
    }
    }

#ifdef NCHIP_GEMM_CLOCKS
    if (g_gemm_clk && blockIdx.y == 0 && t == 0) {
        if (blockIdx.x == 0) {
            g_gemm_clk[0] = clock64() - dbg_c0;       // shader cycles of the k loop
            g_gemm_clk[1] = wall_clock64() - dbg_w0;  // 100 MHz ticks of the same span
        }
        g_gemm_clk[4 + 3 * blockIdx.x] = dbg_w0;          // per workgroup: start,
        g_gemm_clk[5 + 3 * blockIdx.x] = wall_clock64();  // end of the k loop
    }
#endif
    if constexpr (NACC == 2) {
        static_assert(NACC == 1 || (BK / 2 / KW == 8), "chunks of four steps: one chunk per chain");
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] += acc2[i][j][r];
    }
    if (KW == 2) {
        // group 1 parks its accumulators in LDS (the tiles are dead), group 0 adds them
        __syncthreads();
        float *red = smem + (size_t)wave * (TN * TM * 16 * 64) + lane;
        if (kg == 1) {
#pragma unroll
            for (int i = 0; i < TN; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) red[((i * TM + j) * 16 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (kg == 1) return;
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] += red[((i * TM + j) * 16 + r) * 64];
    }

    // epilogue.  acc[i][j][r] is C[m][n] with
    //   m = m0 + wm*BM/2 + j*32 + lane%32
    //   n = n0 + wn*BN/2 + i*32 + (r/4)*8 + (lane/32)*4 + r%4
    const int mm_base = m0 + wm * WTM + (lane & 31);
    const int nn_base = n0 + wn * WTN + (lane >> 5) * 4;
    if (g.ksplit > 1) {
        float NCHIP_GLOBAL *ws = as_global(g.ws + ((int64_t)(kz * g.batch + b)) * g.M * g.N);
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++) {
                int m = mm_base + j * 32;
                if (m >= g.M) continue;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    int n = nn_base + i * 32 + (r >> 2) * 8 + (r & 3);
                    if (n < g.N)
                        ws[(int64_t)n * g.M + m] = acc[i][j][r];
                }
            }
        return;
    }
    const int64_t coff = (int64_t)b_out * g.sc + (int64_t)b_in * g.sc_in;
    float NCHIP_GLOBAL *C = as_global(g.C + coff);
    float NCHIP_GLOBAL *P = g.pre ? as_global(g.pre + coff) : nullptr;
    const float NCHIP_GLOBAL *Radd = g.add ? as_global(g.add + coff) : nullptr;
    const bool full = (m0 + BM <= g.M) && (n0 + BN <= g.N); // uniform
    const float NCHIP_GLOBAL *Dp = g.dpre ? as_global(g.dpre + coff) : nullptr;
    uint16_t NCHIP_GLOBAL *H16 = g.c16 ? as_global(g.c16 + coff) : nullptr;
    const bool plain = !g.bias && !P && !Radd && !Dp && !H16 && g.beta == 0.0f && g.act == NCHIP_ACT_NONE;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++) {
            float NCHIP_GLOBAL *rs = nullptr;
            if (g.rowsum) // partial row of this (tile column, wavefront column, accumulator column, lane half)
                rs = as_global(g.rowsum) + (int64_t)((((tile_n * WN + wn) * TN + i) * 2) + (lane >> 5)) * g.M;
            epilogue_tile(g, acc[i][j], mm_base + j * 32, nn_base + i * 32, C, P, Radd, Dp, full, plain, rs, H16);
        }
#ifdef NCHIP_GEMM_CLOCKS
    if (g_gemm_clk && blockIdx.y == 0 && t == 0) g_gemm_clk[6 + 3 * blockIdx.x] = wall_clock64(); // stores issued
#endif
}

// sums the ksplit partial tiles in increasing k order, then the same epilogue
__global__ __launch_bounds__(256) void gemm_splitk_reduce(GemmArgs g)
{
    int64_t total = (int64_t)g.M * g.N;
    int b = blockIdx.y;
    const int64_t coff = (int64_t)(b / g.batch_in) * g.sc + (int64_t)(b % g.batch_in) * g.sc_in;
    float *C = g.C + coff;
    float *P = g.pre ? g.pre + coff : nullptr;
    const float *Radd = g.add ? g.add + coff : nullptr;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        int m = (int)(e % g.M);
        int64_t n = e / g.M;
        float s = 0.0f;
        for (int kz = 0; kz < g.ksplit; kz++)
            s += g.ws[((int64_t)(kz * g.batch + b)) * total + e];
        int64_t off = n * g.ldc + m;
        float v = g.alpha * s;
        if (g.beta != 0.0f) v += g.beta * C[off];
        if (g.bias) v += g.bias[m];
        if (P) P[off] = v;
        v = apply_act(v, g.act);
        if (Radd) v += Radd[off];
        if (g.dpre) v *= act_grad(g.dpre[coff + off], g.dact);
        C[off] = v;
    }
}

// Rounds a column-major fp32 matrix (rows x cols, leading dimension ld_src) to
// bf16 (nearest even) in the same layout, padded with zeros to rows_pad x
// cols_pad (rows_pad a multiple of 8 = the leading dimension of the copy).
// One thread per 8 consecutive rows of one column.
__global__ __launch_bounds__(256) void cast_bf16_kernel(const float *src, uint16_t *dst, int rows, int cols,
                                                        int64_t ld_src, int rows_pad, int cols_pad, int vec)
{
    const int units = rows_pad / 8;
    const int64_t total = (int64_t)units * cols_pad;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        const int u = (int)(e % units), c = (int)(e / units), r0 = u * 8;
        float f[8];
        if (c < cols && vec && r0 + 8 <= rows) {
            const floatx4 *q = reinterpret_cast<const floatx4 *>(src + (int64_t)c * ld_src + r0);
            floatx4 a = q[0], b = q[1];
            f[0] = a[0]; f[1] = a[1]; f[2] = a[2]; f[3] = a[3];
            f[4] = b[0]; f[5] = b[1]; f[6] = b[2]; f[7] = b[3];
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++)
                f[j] = (c < cols && r0 + j < rows) ? src[(int64_t)c * ld_src + r0 + j] : 0.0f;
        }
        uint4 w = make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
        *reinterpret_cast<uint4 *>(dst + (int64_t)c * rows_pad + r0) = w;
    }
}

// dst[i] = bf16(src[i]) for i < n, 8 elements per thread and step (two 16-byte loads, one
// 16-byte store); both pointers 16-byte aligned
__global__ __launch_bounds__(256) void cast_bf16_flat_kernel(const float *src, uint16_t *dst, int64_t n)
{
    const int64_t units = n / 8, stride = (int64_t)gridDim.x * 256;
    const floatx4 NCHIP_GLOBAL *s4 = reinterpret_cast<const floatx4 NCHIP_GLOBAL *>(as_global(src));
    u32x4 NCHIP_GLOBAL *d4 = reinterpret_cast<u32x4 NCHIP_GLOBAL *>(as_global(dst));
    for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < units; u += stride) {
        const floatx4 a = s4[2 * u], b = s4[2 * u + 1];
        d4[u] = u32x4{ pack_bf16(a[0], a[1]), pack_bf16(a[2], a[3]), pack_bf16(b[0], b[1]), pack_bf16(b[2], b[3]) };
    }
    if (blockIdx.x == 0) // the last n % 8 elements
        for (int64_t i = units * 8 + threadIdx.x; i < n; i += 256) as_global(dst)[i] = f32_to_bf16_rne(as_global(src)[i]);
}

// dst[i] = float(bf16 src[i]) for i < n (exact): one streaming pass
__global__ __launch_bounds__(256) void widen_bf16_flat_kernel(const uint16_t *src, float *dst, int64_t n)
{
    const int64_t stride = (int64_t)gridDim.x * 256;
    const uint16_t NCHIP_GLOBAL *s = as_global(src);
    float NCHIP_GLOBAL *d = as_global(dst);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        d[i] = __builtin_bit_cast(float, (uint32_t)s[i] << 16);
}

// ---- optional per-launch timing (HIP events on the launch stream) ----------
struct ProfRec {
    hipEvent_t start, stop;
    int variant;
    double flops;
};
bool g_prof_on = false;
int g_force_cfg = getenv("NCHIP_GEMM_CFG") ? atoi(getenv("NCHIP_GEMM_CFG")) : 0;
int g_skinny = 3; // width-invariant products with <= 64 columns: 3 = the 16x16x4 MFMA kernel, 2 = the vector-ALU kernel, 1 = the 32x32x2 MFMA kernel, 0 = tiles

// chunks of 256 k in flight: as many as the product has, up to 8
static void launch_fewcol_fma(const GemmArgs &g, dim3 grid, hipStream_t st)
{
    const int nch = (g.K + FC_KC - 1) / FC_KC;
    if (nch <= 2) hipLaunchKernelGGL(gemm_fewcol_fma<2>, grid, dim3(256), 0, st, g);
    else if (nch <= 4) hipLaunchKernelGGL(gemm_fewcol_fma<4>, grid, dim3(256), 0, st, g);
    else hipLaunchKernelGGL(gemm_fewcol_fma<8>, grid, dim3(256), 0, st, g);
}

// 16 x 16 tiles; 8 x 8 tiles from K = 1280 on (up to 8 chunks in flight) and, with a k-major A,
// whenever 16 x 16 tiles would leave most CUs without a workgroup (mmax: the taller product
// of the launch, nz: 1 or 2 products, ak: A is k-major)
static void launch_fewcol_mfma(const GemmArgs &g, int mmax, int nz, hipStream_t st, bool ak = false)
{
    const int nch = (g.K + 255) / 256;
    const dim3 grid16(mmax / 16, (g.N + 15) / 16, nz), grid8(mmax / 8, (g.N + 7) / 8, nz);
    const bool small = nch > 4 || (ak && grid16.x * grid16.y * grid16.z < 192);
    if (!ak) {
        if (small) hipLaunchKernelGGL((gemm_fewcol_mfma<8, 0, 8>), grid8, dim3(256), 0, st, g);
        else if (nch <= 2) hipLaunchKernelGGL(gemm_fewcol_mfma<2>, grid16, dim3(256), 0, st, g);
        else hipLaunchKernelGGL(gemm_fewcol_mfma<4>, grid16, dim3(256), 0, st, g);
    } else if (small) {
        if (nch <= 2) hipLaunchKernelGGL((gemm_fewcol_mfma<2, 0, 8, 1>), grid8, dim3(256), 0, st, g);
        else if (nch <= 4) hipLaunchKernelGGL((gemm_fewcol_mfma<4, 0, 8, 1>), grid8, dim3(256), 0, st, g);
        else hipLaunchKernelGGL((gemm_fewcol_mfma<8, 0, 8, 1>), grid8, dim3(256), 0, st, g);
    } else {
        if (nch <= 2) hipLaunchKernelGGL((gemm_fewcol_mfma<2, 0, 16, 1>), grid16, dim3(256), 0, st, g);
        else hipLaunchKernelGGL((gemm_fewcol_mfma<4, 0, 16, 1>), grid16, dim3(256), 0, st, g);
    }
}
int g_force_gm = -1;
std::vector<ProfRec> g_prof;
int g_bf16ops_cls = getenv("NCHIP_GEMM_BF16OPS_CLASS") ? atoi(getenv("NCHIP_GEMM_BF16OPS_CLASS")) : 0;


// With `rec` the kernel's own start / stop timestamps are bound to the record's
// events (hipExtLaunchKernelGGL), so the measured time is the dispatch alone,
// as a kernel trace reports it, without the marker packets of hipEventRecord.
// bytes of the two tile buffer pairs when they exceed what a static array may hold (else 0)
template <int BM, int BN, int BK, int TA, int TB, int BF16>
constexpr size_t lds_dynamic_bytes()
{
    constexpr int SQ = BK / 2 + 4;
    constexpr size_t a = BF16 == 2 && TA ? BM * SQ : (BF16 ? (BK / 2) * (BM + PAD) : BK * (BM + (TA ? FPAD_K : PAD)));
    constexpr size_t b = BF16 == 2 && !TB ? BN * SQ : (BF16 ? (BK / 2) * (BN + PAD) : BK * (BN + (TB ? PAD : FPAD_K)));
    constexpr size_t bytes = 2 * (a + b) * sizeof(float);
    static_assert(bytes <= 160 * 1024, "tile buffers exceed LDS");
    return bytes > 65536 ? bytes : 0;
}

template <int BM, int BN, int BK, int WM, int WN, int BF16, int KW = 1, int PF = 2, int SA = (BF16 == 2), int NACC = 1, int FRAG = 0>
void launch_tile(hipStream_t st, int ta, int tb, GemmArgs &g, ProfRec *rec)
{
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    g.gm = g_force_gm >= 0 ? g_force_gm : 8;
    g.dbg = 0;
    dim3 grid(g.tiles_m * g.tiles_n, g.batch * g.ksplit), block(64 * WM * WN * KW);
#define LAUNCH(TA, TB)                                                                                     \
    do {                                                                                                   \
        constexpr size_t dyn = lds_dynamic_bytes<BM, BN, BK, TA, TB, BF16>();                              \
        if (dyn) {                                                                                         \
            static const bool ok = hipFuncSetAttribute(                                                    \
                reinterpret_cast<const void *>(gemm_kernel<BM, BN, BK, WM, WN, TA, TB, BF16, KW, PF, SA, NACC, FRAG>),     \
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) == hipSuccess;                       \
            if (!ok) { fprintf(stderr, "nchip_gemm: cannot reserve %zu bytes of LDS\n", dyn); abort(); }  \
        }                                                                                                  \
        if (rec) hipExtLaunchKernelGGL((gemm_kernel<BM, BN, BK, WM, WN, TA, TB, BF16, KW, PF, SA, NACC, FRAG>), grid, block, dyn, \
                                       st, rec->start, rec->stop, 0, g);                                   \
        else hipLaunchKernelGGL((gemm_kernel<BM, BN, BK, WM, WN, TA, TB, BF16, KW, PF, SA, NACC, FRAG>), grid, block, dyn, st, g); \
    } while (0)
    if (!ta && !tb) LAUNCH(0, 0);
    else if (ta && !tb) LAUNCH(1, 0);
    else if (!ta && tb) LAUNCH(0, 1);
    else LAUNCH(1, 1);
#undef LAUNCH
}

// Device scratch for the bf16 copies of one product's operands, one buffer per
// stream: successive products on a stream reuse it in stream order.  It grows
// on demand and lives until the process ends.
struct CastScratch { hipStream_t st; uint16_t *ptr; size_t cap; };
std::vector<CastScratch> g_cast;
int g_bf16src = getenv("NCHIP_GEMM_BF16SRC") ? atoi(getenv("NCHIP_GEMM_BF16SRC")) : 1;
double g_bf16src_min_flops = getenv("NCHIP_GEMM_BF16SRC_FLOPS") ? atof(getenv("NCHIP_GEMM_BF16SRC_FLOPS")) : 8e9;

uint16_t *cast_scratch(hipStream_t st, size_t elems)
{
    for (CastScratch &c : g_cast)
        if (c.st == st) {
            if (c.cap >= elems) return c.ptr;
            (void)hipStreamSynchronize(st);
            (void)hipFree(c.ptr);
            c.ptr = nullptr; c.cap = 0;
            size_t cap = elems + elems / 4;
            if (hipMalloc((void **)&c.ptr, cap * sizeof(uint16_t)) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
            c.cap = cap;
            return c.ptr;
        }
    CastScratch c = { st, nullptr, 0 };
    if (hipMalloc((void **)&c.ptr, elems * sizeof(uint16_t)) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    c.cap = elems;
    g_cast.push_back(c);
    return c.ptr;
}

constexpr int CAST_SLACK = 512; // elements past a copy that a partial edge tile may read

// copy of a column-major rows x cols operand; k_is_rows says which extent is k
// (padded to kpad); returns the leading dimension of the copy
int64_t cast_operand(hipStream_t st, const float *src, int rows, int cols, int64_t ld, bool k_is_rows,
                     int kpad, uint16_t *dst)
{
    const int rows_pad = k_is_rows ? kpad : (rows + 7) / 8 * 8;
    const int cols_pad = k_is_rows ? cols : kpad;
    const int vec = (ld % 4 == 0) && (((uintptr_t)src & 15) == 0);
    int64_t total = (int64_t)(rows_pad / 8) * cols_pad;
    int nb = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    hipLaunchKernelGGL(cast_bf16_kernel, dim3(nb), dim3(256), 0, st, src, dst, rows, cols, ld, rows_pad, cols_pad, vec);
    return rows_pad;
}

size_t cast_elems(int rows, int cols, bool k_is_rows, int kpad)
{
    const size_t rows_pad = k_is_rows ? kpad : (rows + 7) / 8 * 8;
    const size_t cols_pad = k_is_rows ? cols : kpad;
    return (rows_pad * cols_pad + CAST_SLACK + 127) / 128 * 128;
}

} // namespace

extern "C" int nchip_gemm_pick_ksplit(int m, int n, int k, int batch)
{
    // Aim at >= 512 workgroups (2 per CU on 256 CUs) when the output is small
    // and the reduction long (the weight-gradient GEMMs: k = tokens).
    int64_t tiles = (int64_t)((m + 63) / 64) * ((n + 63) / 64) * batch;
    if (tiles >= 256 || k < 1024)
        return 1;
    int s = (int)((512 + tiles - 1) / tiles);
    int smax = k / 256;
    if (s > smax) s = smax;
    if (s > 16) s = 16;
    return s < 1 ? 1 : s;
}

static int gemm2_impl(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                      const float *A, int64_t lda, int64_t sa_out, int64_t sa_in,
                      const float *B, int64_t ldb, int64_t sb_out, int64_t sb_in,
                      float beta, float *C, int64_t ldc, int64_t sc_out, int64_t sc_in,
                      int batch, int batch_in,
                      const float *bias, int act, float *pre, const float *addend, int precision,
                      int ksplit, float *workspace, const float *dpre = nullptr, int dact = 0,
                      float *rowsum = nullptr, int *rowsum_rows = nullptr)
{
    if (rowsum_rows) *rowsum_rows = 0;
    if (m <= 0 || n <= 0 || batch <= 0)
        return 0;
    if (k < 0 || !A || !B || !C || lda < (ta ? k : m) || ldb < (tb ? n : k) || ldc < m || batch_in < 1) {
        fprintf(stderr, "nchip_gemm: bad arguments (m=%d n=%d k=%d lda=%ld ldb=%ld ldc=%ld)\n",
                m, n, k, (long)lda, (long)ldb, (long)ldc);
        return -1;
    }
    const bool invariant = (precision & NCHIP_GEMM_WIDTH_INVARIANT) != 0;
    precision &= 0xff;
    if (ksplit < 1 || invariant) ksplit = 1;
    if (ksplit > 1 && !workspace) {
        fprintf(stderr, "nchip_gemm: ksplit=%d needs a workspace\n", ksplit);
        return -1;
    }
    if ((int64_t)batch * ksplit > 65535) {
        fprintf(stderr, "nchip_gemm: batch*ksplit=%ld exceeds the grid limit\n", (long)batch * ksplit);
        return -1;
    }
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = A; g.B = B; g.C = C; g.bias = bias; g.add = addend; g.pre = pre; g.ws = workspace;
    g.dpre = dpre; g.dact = act_for_precision(dact, precision);
    g.rowsum = nullptr;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.sa = sa_out; g.sb = sb_out; g.sc = sc_out;
    g.sa_in = sa_in; g.sb_in = sb_in; g.sc_in = sc_in; g.batch_in = batch_in;
    g.M = m; g.N = n; g.K = k; g.batch = batch; g.ksplit = ksplit;
    g.kchunk = ((k + ksplit - 1) / ksplit + KALIGN - 1) / KALIGN * KALIGN;
    if (g.kchunk < KALIGN) g.kchunk = KALIGN;
    g.alpha = alpha; g.beta = beta; g.act = act_for_precision(act, precision);
    g.grp = nullptr; g.n_grp = 0;
    hipStream_t st = (hipStream_t)stream;
    // tile choice from the shape only: large tiles when they still fill the chip
    int64_t t128 = (int64_t)((m + 127) / 128) * ((n + 127) / 128) * batch * ksplit;
    ProfRec rec;
    if (g_prof_on) {
        (void)hipEventCreate(&rec.start);
        (void)hipEventCreate(&rec.stop);
        rec.variant = -1;
        rec.flops = 2.0 * m * n * (double)k * batch;
    }
    ProfRec *pr = g_prof_on ? &rec : nullptr;
    if (invariant && g_skinny == 3 && ta && !tb && batch == 1 && precision == 0 && n <= 64 && k >= 32 && k % 32 == 0 &&
        m % 32 == 0 && lda % 4 == 0 && ldb % 4 == 0 && (((uintptr_t)A | (uintptr_t)B) & 15) == 0 && beta == 0.0f &&
        alpha == 1.0f && !dpre && !g_prof_on) {
        // a few token columns against a k-major A (a weight matrix's transposed copy): same chains
        launch_fewcol_mfma(g, m, 1, st, true);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            fprintf(stderr, "nchip_gemm: launch failed: %s\n", hipGetErrorString(e));
            return -2;
        }
        return 0;
    }
    if (invariant && g_skinny && !ta && !tb && batch == 1 && precision == 0 && n <= 64 && k >= 32 && k % 32 == 0 &&
        m % 32 == 0 && lda % 4 == 0 && ldb % 4 == 0 && (((uintptr_t)A | (uintptr_t)B) & 15) == 0 && beta == 0.0f && !g_prof_on) {
        // a few token columns: the same arithmetic without the tile pipeline
        if (g_skinny == 3 && alpha == 1.0f && !dpre)
            launch_fewcol_mfma(g, m, 1, st);
        else if (g_skinny >= 2 && alpha == 1.0f && !dpre)
            launch_fewcol_fma(g, dim3(m / 8, (n + 7) / 8), st);
        else
            hipLaunchKernelGGL(gemm_skinny_nn<16>, dim3(m / 32, (n + 31) / 32), dim3(256), 0, st, g);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            fprintf(stderr, "nchip_gemm: launch failed: %s\n", hipGetErrorString(e));
            return -2;
        }
        return 0;
    }
    // Tile configuration from the shape alone.  Measured on MI355X (fp32):
    // small outputs want the most workgroups and the most wavefronts per
    // workgroup (64x64x32, two k groups of 4 wavefronts); once
    // 128x64 tiles still give >= 256 workgroups, 8 wavefronts of 32x32 on a
    // 128x64x32 tile win; very large problems use 128x128x32 with 8 wavefronts.
    int cfg = invariant ? 30 : g_force_cfg; // tuning aid: 0 = choose from the shape
    int64_t nb = (int64_t)batch * ksplit;
    int64_t t128x64 = (int64_t)((m + 127) / 128) * ((n + 63) / 64) * nb;
    if (!cfg) {
        if (t128 >= 512 && m >= 128 && n >= 128) cfg = 7;
        else if (t128x64 >= 256 && m >= 128 && n >= 64) cfg = 4;
        else cfg = 10; // 64x64x32, two k groups, four register sets of tiles in flight
    }
    // Large bf16 products are bound by operand traffic from L2, not by the MFMA
    // rate: round both operands to bf16 in memory first (one streaming pass
    // each) and let the tiles load half the bytes.  The rounded values are
    // the ones the conversion inside the tile loader would produce, so the
    // result is the same either way.
    bool from_bf16 = false;
    if (precision == 1 && batch == 1 && ksplit == 1 && !invariant &&
        (g_bf16src == 2 || (g_bf16src == 1 && m >= 128 && n >= 128 && k >= 256 &&
                            2.0 * m * n * (double)k >= g_bf16src_min_flops))) {
        const int kpad = (k + 63) / 64 * 64;
        const size_t ea = cast_elems(ta ? k : m, ta ? m : k, ta != 0, kpad);
        const size_t eb = cast_elems(tb ? n : k, tb ? k : n, tb == 0, kpad);
        uint16_t *buf = cast_scratch(st, ea + eb);
        if (buf) {
            g.lda = cast_operand(st, A, ta ? k : m, ta ? m : k, lda, ta != 0, kpad, buf);
            g.ldb = cast_operand(st, B, tb ? n : k, tb ? k : n, ldb, tb == 0, kpad, buf + ea);
            g.A = reinterpret_cast<const float *>(buf);
            g.B = reinterpret_cast<const float *>(buf + ea);
            g.K = kpad; g.kchunk = kpad;
            from_bf16 = true;
        }
    }
    // partial row sums of the result (activation-gradient epilogue): one row per 16 columns of
    // the padded column range; only the plain tile classes write them
    if (rowsum && rowsum_rows && dpre && ksplit == 1 && batch == 1 && !from_bf16 &&
        (cfg == 7 || cfg == 4 || cfg == 10 || cfg == 30)) {
        const int bn = cfg == 7 ? 128 : 64;
        g.rowsum = rowsum;
        *rowsum_rows = (n + bn - 1) / bn * bn / 16;
    }
    if (from_bf16) {
        // 64x64 per wavefront, 64-deep tiles: with enough tiles for two workgroups
        // per CU four wavefronts each do best; below that, eight wavefronts in
        // two k groups share one tile
        const bool four = g_force_cfg == 13 || (g_force_cfg != 11 && g_force_cfg != 7 && t128 >= 512);
        if (g_force_cfg == 7) launch_tile<128, 128, 32, 4, 2, 2>(st, ta, tb, g, pr);
        else if (four) launch_tile<128, 128, 64, 2, 2, 2, 1>(st, ta, tb, g, pr);
        else launch_tile<128, 128, 64, 2, 2, 2, 2>(st, ta, tb, g, pr);
    } else if (precision == 1) {
        if (cfg == 7) launch_tile<128, 128, 32, 4, 2, 1>(st, ta, tb, g, pr);
        else if (cfg == 4) launch_tile<128, 64, 32, 4, 2, 1>(st, ta, tb, g, pr);
        else if (cfg == 9) launch_tile<64, 64, 64, 2, 2, 1, 2>(st, ta, tb, g, pr);
        else launch_tile<64, 64, 32, 2, 2, 1, 2>(st, ta, tb, g, pr);
    } else if (cfg == 1) {
        launch_tile<128, 128, 16, 2, 2, 0>(st, ta, tb, g, pr);
    } else if (cfg == 2) {
        launch_tile<128, 128, 16, 4, 2, 0>(st, ta, tb, g, pr);
    } else if (cfg == 3) {
        launch_tile<128, 64, 16, 2, 2, 0>(st, ta, tb, g, pr);
    } else if (cfg == 4) {
        launch_tile<128, 64, 32, 4, 2, 0>(st, ta, tb, g, pr);
    } else if (cfg == 6) {
        launch_tile<64, 128, 16, 2, 2, 0>(st, ta, tb, g, pr);
    } else if (cfg == 7) {
        launch_tile<128, 128, 32, 4, 2, 0, 1, 2, 0, 1, 1>(st, ta, tb, g, pr); // rolling fragment window: two accumulator tiles per wavefront
    } else if (cfg == 8) {
        launch_tile<64, 64, 32, 2, 2, 0, 2>(st, ta, tb, g, pr);
    } else if (cfg == 9) {
        launch_tile<64, 64, 64, 2, 2, 0, 2>(st, ta, tb, g, pr);
    } else if (cfg == 10) {
        launch_tile<64, 64, 32, 2, 2, 0, 2, 4>(st, ta, tb, g, pr);
    } else if (cfg == 30) { // the width-invariant class: four chains per element
        launch_tile<64, 64, 32, 2, 2, 0, 2, 4, 0, 2>(st, ta, tb, g, pr);
    } else {
        launch_tile<64, 64, 16, 2, 2, 0>(st, ta, tb, g, pr);
    }
    if (g_prof_on) {
        int tile = cfg == 7 ? 2 : (cfg == 4 ? 1 : ((cfg == 8 || cfg == 10 || cfg == 30) ? 3 : 0));
        rec.variant = tile * 8 + (ta ? 4 : 0) + (tb ? 2 : 0) + (precision == 1 ? 1 : 0);
        g_prof.push_back(rec);
    }
    if (ksplit > 1) {
        int64_t total = (int64_t)m * n;
        int nb = (int)((total + 255) / 256);
        if (nb > 2048) nb = 2048;
        hipLaunchKernelGGL(gemm_splitk_reduce, dim3(nb, batch), dim3(256), 0, st, g);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fprintf(stderr, "nchip_gemm: launch failed: %s\n", hipGetErrorString(e));
        return -2;
    }
    return 0;
}

extern "C" int nchip_gemm2(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                           const float *A, int64_t lda, int64_t sa_out, int64_t sa_in,
                           const float *B, int64_t ldb, int64_t sb_out, int64_t sb_in,
                           float beta, float *C, int64_t ldc, int64_t sc_out, int64_t sc_in,
                           int batch, int batch_in,
                           const float *bias, int act, float *pre, int precision,
                           int ksplit, float *workspace)
{
    return gemm2_impl(stream, ta, tb, m, n, k, alpha, A, lda, sa_out, sa_in, B, ldb, sb_out, sb_in,
                      beta, C, ldc, sc_out, sc_in, batch, batch_in, bias, act, pre, nullptr, precision,
                      ksplit, workspace);
}

extern "C" int nchip_gemm_add(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                              const float *A, int64_t lda, int64_t stride_a,
                              const float *B, int64_t ldb, int64_t stride_b,
                              float *C, int64_t ldc, int64_t stride_c, int batch,
                              const float *bias, int act, float *pre, const float *addend,
                              int precision, int ksplit, float *workspace)
{
    return gemm2_impl(stream, ta, tb, m, n, k, alpha, A, lda, stride_a, 0, B, ldb, stride_b, 0,
                      0.0f, C, ldc, stride_c, 0, batch, 1, bias, act, pre, addend, precision, ksplit,
                      workspace);
}

extern "C" int nchip_gemm_dact(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                               const float *A, int64_t lda, const float *B, int64_t ldb,
                               float *C, int64_t ldc, const float *pre_act, int act,
                               int precision, int ksplit, float *workspace)
{
    return gemm2_impl(stream, ta, tb, m, n, k, alpha, A, lda, 0, 0, B, ldb, 0, 0, 0.0f, C, ldc, 0, 0, 1, 1,
                      nullptr, 0, nullptr, nullptr, precision, ksplit, workspace, pre_act, act);
}

// nchip_gemm_dact that also leaves partial row sums of C: rowsum holds nchip_gemm_rowsum_rows(n)
// rows of m floats, of which *rows_written are written (row p = the sum over 16 columns of C;
// 0 when this product's kernel does not write them: the caller then sums C itself)
extern "C" int nchip_gemm_rowsum_rows(int n) { return (n + 127) / 128 * 8; }

extern "C" int nchip_gemm_dact_rowsum(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                                      const float *A, int64_t lda, const float *B, int64_t ldb,
                                      float *C, int64_t ldc, const float *pre_act, int act,
                                      int precision, int ksplit, float *workspace,
                                      float *rowsum, int *rows_written)
{
    return gemm2_impl(stream, ta, tb, m, n, k, alpha, A, lda, 0, 0, B, ldb, 0, 0, 0.0f, C, ldc, 0, 0, 1, 1,
                      nullptr, 0, nullptr, nullptr, precision, ksplit, workspace, pre_act, act, rowsum, rows_written);
}

extern "C" int nchip_gemm(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                          const float *A, int64_t lda, int64_t stride_a,
                          const float *B, int64_t ldb, int64_t stride_b,
                          float beta, float *C, int64_t ldc, int64_t stride_c, int batch,
                          const float *bias, int act, float *pre, int precision,
                          int ksplit, float *workspace)
{
    return nchip_gemm2(stream, ta, tb, m, n, k, alpha, A, lda, stride_a, 0, B, ldb, stride_b, 0,
                       beta, C, ldc, stride_c, 0, batch, 1, bias, act, pre, precision, ksplit,
                       workspace);
}

// tuning aid: forces tile configuration `cfg` for every later call (0 = automatic)
extern "C" void nchip_gemm_force_config(int cfg)
{
    g_force_cfg = cfg;
}

// testing aid: 0 sends width-invariant products of a few columns through the tile
// kernel again, 1 through the 32x32x2 MFMA few-column kernel, 2 through the vector-ALU
// kernel, 3 (default) through the 16x16x4 MFMA kernel (same bits, by construction: the
// tests compare the four)
extern "C" void nchip_gemm_few_columns_kernel(int on)
{
    g_skinny = on;
}

// Two width-invariant few-column products with one operand in common, in ONE launch:
// C0 (m0 x n) = A0 B + bias0 and C1 (m1 x n) = A1 B + bias1 (bias pointers may be NULL),
// the decoder's query and key/value projections of a timestep.  Same kernel and the same
// bits as two nchip_gemm calls in width-invariant mode.  Returns 1 when the shapes are not
// the few-column kernel's (nothing launched: the caller issues the two products itself).
extern "C" int nchip_gemm_pair_few_columns(void *stream, int m0, int m1, int n, int k,
                                           const float *A0, int64_t lda0, const float *A1, int64_t lda1,
                                           const float *B, int64_t ldb,
                                           float *C0, int64_t ldc0, float *C1, int64_t ldc1,
                                           const float *bias0, const float *bias1, int a_k_major)
{
    if (m0 <= 0 || m1 <= 0 || n <= 0 || !A0 || !A1 || !B || !C0 || !C1) return -1;
    if (a_k_major && g_skinny != 3) return 1;
    if (!g_skinny || g_prof_on || n > 64 || k < 32 || k % 32 || m0 % 32 || m1 % 32 || lda0 % 4 || lda1 % 4 || ldb % 4 ||
        lda0 < (a_k_major ? k : m0) || lda1 < (a_k_major ? k : m1) || ldb < k || ldc0 < m0 || ldc1 < m1 ||
        (((uintptr_t)A0 | (uintptr_t)A1 | (uintptr_t)B) & 15) != 0)
        return 1;
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = A0; g.B = B; g.C = C0; g.bias = bias0; g.lda = lda0; g.ldb = ldb; g.ldc = ldc0;
    g.M = m0; g.N = n; g.K = k; g.batch = 1; g.batch_in = 1; g.ksplit = 1; g.alpha = 1.0f;
    g.A_1 = A1; g.C_1 = C1; g.bias_1 = bias1; g.lda_1 = lda1; g.ldc_1 = ldc1; g.M_1 = m1;
    const int mmax = m0 > m1 ? m0 : m1;
    if (g_skinny == 3)
        launch_fewcol_mfma(g, mmax, 2, (hipStream_t)stream, a_k_major != 0);
    else if (g_skinny == 2)
        launch_fewcol_fma(g, dim3(mmax / 8, (n + 7) / 8, 2), (hipStream_t)stream);
    else
        hipLaunchKernelGGL(gemm_skinny_nn<16>, dim3(mmax / 32, (n + 31) / 32, 2), dim3(256), 0, (hipStream_t)stream, g);
    if (hipGetLastError() != hipSuccess) {
        fprintf(stderr, "nchip_gemm_pair_few_columns: launch failed\n");
        return -2;
    }
    return 0;
}

// One or two width-invariant few-column products of the layer norm (avg = 1) or RMS norm
// (avg = 0) of B's columns, in ONE launch: C0 (m0 x n) = act0(A0 norm(B) + bias0) and, when
// m1 > 0, C1 (m1 x n) = A1 norm(B) + bias1.  B holds k = 128, 256 or 512 raw features per
// column; ln_w / ln_b are the gain and bias (both or neither); the normalised columns are
// also written to ln_out (leading dimension ld_ln) when it is not NULL.  The bits are those
// of nchip_norm_fwd followed by the products in width-invariant mode.  Returns 1 when the
// shapes are not this kernel's (nothing launched: the caller issues the steps itself).
extern "C" int nchip_norm_gemm_few_columns(void *stream, const float *ln_w, const float *ln_b, float eps, int avg,
                                           float *ln_out, int64_t ld_ln, int m0, int m1, int n, int k,
                                           const float *A0, int64_t lda0, const float *A1, int64_t lda1,
                                           const float *B, int64_t ldb, float *C0, int64_t ldc0,
                                           float *C1, int64_t ldc1, const float *bias0, const float *bias1, int act0,
                                           int a_k_major)
{
    if (m0 <= 0 || m1 < 0 || n <= 0 || !A0 || !B || !C0 || (m1 > 0 && (!A1 || !C1)) || (ln_w == nullptr) != (ln_b == nullptr))
        return -1;
    if (g_skinny != 3 || g_prof_on || n > 64 || (k != 128 && k != 256 && k != 512) || m0 % 32 || m1 % 32 || lda0 % 4 ||
        (m1 > 0 && lda1 % 4) || lda0 < (a_k_major ? k : m0) || (m1 > 0 && lda1 < (a_k_major ? k : m1)) || ldb < k || ldc0 < m0 || (m1 > 0 && ldc1 < m1) ||
        (ln_out && ld_ln < k) || (((uintptr_t)A0 | (uintptr_t)A1) & 15) != 0 ||
        (act0 != NCHIP_ACT_NONE && act0 != NCHIP_ACT_GELU && act0 != NCHIP_ACT_RELU))
        return 1;
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = A0; g.B = B; g.C = C0; g.bias = bias0; g.lda = lda0; g.ldb = ldb; g.ldc = ldc0; g.act = act0;
    g.M = m0; g.N = n; g.K = k; g.batch = 1; g.batch_in = 1; g.ksplit = 1; g.alpha = 1.0f;
    g.A_1 = A1; g.C_1 = C1; g.bias_1 = bias1; g.lda_1 = lda1; g.ldc_1 = ldc1; g.M_1 = m1;
    g.ln_w = ln_w; g.ln_b = ln_b; g.ln_out = ln_out; g.ld_ln = ld_ln; g.ln_eps = eps; g.ln_avg = avg;
    const int mmax = m0 > m1 ? m0 : m1;
    const dim3 grid(mmax / 16, (n + 15) / 16, m1 > 0 ? 2 : 1);
    hipStream_t st = (hipStream_t)stream;
    if (a_k_major) {
        if (k == 128) hipLaunchKernelGGL((gemm_fewcol_mfma<2, 2, 16, 1>), grid, dim3(256), 0, st, g);
        else if (k == 256) hipLaunchKernelGGL((gemm_fewcol_mfma<2, 4, 16, 1>), grid, dim3(256), 0, st, g);
        else hipLaunchKernelGGL((gemm_fewcol_mfma<2, 8, 16, 1>), grid, dim3(256), 0, st, g);
    } else if (k == 128) hipLaunchKernelGGL((gemm_fewcol_mfma<2, 2>), grid, dim3(256), 0, st, g);
    else if (k == 256) hipLaunchKernelGGL((gemm_fewcol_mfma<2, 4>), grid, dim3(256), 0, st, g);
    else hipLaunchKernelGGL((gemm_fewcol_mfma<2, 8>), grid, dim3(256), 0, st, g);
    if (hipGetLastError() != hipSuccess) {
        fprintf(stderr, "nchip_norm_gemm_few_columns: launch failed\n");
        return -2;
    }
    return 0;
}

// 0: bf16 products always round their operands inside the tile loader;
// 1: large ones go through bf16 copies of the operands (default);
// 2: every unbatched bf16 product does (testing aid)
extern "C" void nchip_gemm_bf16_source(int mode)
{
    g_bf16src = mode;
}

extern "C" void nchip_gemm_force_band(int gm)
{
    g_force_gm = gm;
}

extern "C" int nchip_cast_bf16(void *stream, const float *src, uint16_t *dst, int64_t n)
{
    if (n <= 0) return 0;
    if (!src || !dst || (((uintptr_t)src | (uintptr_t)dst) & 15) != 0) {
        fprintf(stderr, "nchip_cast_bf16: 16-byte aligned buffers expected\n");
        return -1;
    }
    int64_t nb = (n / 8 + 255) / 256;
    if (nb < 1) nb = 1;
    if (nb > 4096) nb = 4096;
    hipLaunchKernelGGL(cast_bf16_flat_kernel, dim3((unsigned)nb), dim3(256), 0, (hipStream_t)stream, src, dst, n);
    if (hipGetLastError() != hipSuccess) { fprintf(stderr, "nchip_cast_bf16: launch failed\n"); return -2; }
    return 0;
}

extern "C" int nchip_widen_bf16(void *stream, const uint16_t *src, float *dst, int64_t n)
{
    if (n <= 0) return 0;
    int64_t nb = (n + 255) / 256;
    if (nb > 8192) nb = 8192;
    hipLaunchKernelGGL(widen_bf16_flat_kernel, dim3((unsigned)nb), dim3(256), 0, (hipStream_t)stream, src, dst, n);
    if (hipGetLastError() != hipSuccess) { fprintf(stderr, "nchip_widen_bf16: launch failed\n"); return -2; }
    return 0;
}

// Product whose operands are already bf16 in memory (the rounded copies of the fp32 matrices,
// element for element in the same column-major layout: no padding).  Unguarded 16-byte loads
// throughout, so the shapes must fit: k a multiple of 64; an operand whose long axis is
// contiguous (A with ta = 0, B with tb = 1) must fill whole tiles (m resp. n a multiple of
// 128: every tile class divides it); leading dimensions multiples of 8 elements; 16-byte
// aligned bases.  Returns 1 when they do not (nothing launched: the caller takes another
// route).  Epilogue options as in the fp32-operand calls; c16, when given, receives the
// result rounded to bf16 next to C.
extern "C" int nchip_gemm_bf16_operands(void *stream, const NchipGemmBf16Args *a)
{
    if (a->rows_written) *a->rows_written = 0;
    const int m = a->m, n = a->n, k = a->k, ta = a->ta != 0, tb = a->tb != 0;
    if (m <= 0 || n <= 0) return 0;
    if (!a->A16 || !a->B16 || !a->C || k <= 0 || a->lda < (ta ? k : m) || a->ldb < (tb ? n : k) || a->ldc < m) {
        fprintf(stderr, "nchip_gemm_bf16_operands: bad arguments (m=%d n=%d k=%d)\n", m, n, k);
        return -1;
    }
    if (k % 64 || a->lda % 8 || a->ldb % 8 || (((uintptr_t)a->A16 | (uintptr_t)a->B16) & 15) != 0)
        return 1;
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = reinterpret_cast<const float *>(a->A16); g.B = reinterpret_cast<const float *>(a->B16);
    g.C = a->C; g.c16 = a->C16; g.bias = a->bias; g.add = a->addend; g.pre = a->pre;
    g.dpre = a->dpre; g.dact = act_for_precision(a->dact, 2);
    g.lda = a->lda; g.ldb = a->ldb; g.ldc = a->ldc;
    g.batch_in = 1; g.M = m; g.N = n; g.K = k; g.batch = 1; g.ksplit = 1; g.kchunk = k;
    g.alpha = a->alpha; g.beta = 0.0f; g.act = act_for_precision(a->act, 2);
    hipStream_t st = (hipStream_t)stream;
    // tile class from the tile counts: the largest tile that still gives every CU a workgroup
    const int64_t t128 = (int64_t)((m + 127) / 128) * ((n + 127) / 128);
    const int64_t t128x64 = (int64_t)((m + 127) / 128) * ((n + 63) / 64);
    int cls = g_bf16ops_cls;
    if (cls < 1 || cls > 3) cls = t128 >= 224 ? 1 : (t128x64 >= 224 && m >= 128 ? 2 : 3);
    {
        const int bm = cls == 3 ? 64 : 128, bn = cls == 1 ? 128 : 64;
        if ((!ta && m % bm) || (tb && n % bn)) return 1; // row-contiguous operands need whole tiles
    }
    if (a->rowsum && a->rows_written && a->dpre) {
        const int bn = cls == 1 ? 128 : 64;
        g.rowsum = a->rowsum;
        *a->rows_written = (n + bn - 1) / bn * bn / 16;
    }
    ProfRec rec;
    if (g_prof_on) {
        (void)hipEventCreate(&rec.start);
        (void)hipEventCreate(&rec.stop);
        rec.flops = 2.0 * m * n * (double)k;
        rec.variant = 32 + cls * 4 + ta * 2 + tb; // the bf16-operand classes
    }
    ProfRec *pr = g_prof_on ? &rec : nullptr;
    // (measured on the C3 and C4 shapes: deeper prefetch - 3 or 4 register sets - changes nothing
    // once the loop waits for its oldest set only; 256 x 128 tiles with 8 wavefronts run at the
    // rate of the 128 x 128 class, 256 x 256 tiles spill)
    if (cls == 1) launch_tile<128, 128, 64, 2, 2, 2, 1>(st, ta, tb, g, pr);
    else if (cls == 2) launch_tile<128, 64, 64, 2, 2, 2, 1>(st, ta, tb, g, pr);
    else launch_tile<64, 64, 64, 2, 2, 2, 1>(st, ta, tb, g, pr);
    if (g_prof_on) g_prof.push_back(rec);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fprintf(stderr, "nchip_gemm_bf16_operands: launch failed: %s\n", hipGetErrorString(e));
        return -2;
    }
    return 0;
}

// tuning aid: 0 = choose the bf16-operand tile class from the shape, 1 = 128x128, 2 = 128x64, 3 = 64x64
extern "C" void nchip_gemm_bf16_operands_class(int cls) { g_bf16ops_cls = cls; }

// ---- profiling entry points ---------------------------------------------------
extern "C" void nchip_gemm_profile_enable(int on)
{
    g_prof_on = on != 0;
}

extern "C" int nchip_gemm_profile_read(int max_variants, char (*names)[48], int64_t *launches,
                                       double *flops, double *seconds)
{
    constexpr int NVAR = 64;
    double fl[NVAR] = { 0 }, sec[NVAR] = { 0 };
    int64_t cnt[NVAR] = { 0 };
    for (ProfRec &r : g_prof) {
        float ms = 0.0f;
        (void)hipEventSynchronize(r.stop);
        (void)hipEventElapsedTime(&ms, r.start, r.stop);
        if (r.variant >= 0 && r.variant < NVAR) {
            fl[r.variant] += r.flops;
            sec[r.variant] += ms * 1e-3;
            cnt[r.variant]++;
        }
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    g_prof.clear();
    static const char *tiles_f32[4] = { "64,64,16,2,2", "128,64,32,4,2", "128,128,32,4,2", "64,64,32,2,2" };
    static const char *tiles_bf16[4] = { "64,64,32,2,2", "128,64,32,4,2", "128,128,32,4,2", "64,64,32,2,2" };
    static const char *tiles_ops[4] = { "128,128,64,2,2", "128,128,64,2,2", "128,64,64,2,2", "64,64,64,2,2" }; // 0: the grouped launch
    int n = 0;
    for (int v = 0; v < NVAR && n < max_variants; v++) {
        if (!cnt[v]) continue;
        if (v >= 32) { // operands read as bf16: gemm_kernel<tile, ta, tb, 2>
            snprintf(names[n], 48, "gemm_kernel<%s,%d,%d,2%s>", tiles_ops[(v - 32) / 4], (v >> 1) & 1, v & 1,
                     v < 36 ? ",grouped" : "");
        } else {
            const bool two_groups = v / 8 == 3 || ((v & 1) && v / 8 == 0);
            snprintf(names[n], 48, "gemm_kernel<%s,%d,%d,%d%s>", (v & 1) ? tiles_bf16[v / 8] : tiles_f32[v / 8],
                     (v >> 2) & 1, (v >> 1) & 1, v & 1, two_groups ? ",2" : "");
        }
        launches[n] = cnt[v]; flops[n] = fl[v]; seconds[n] = sec[v];
        n++;
    }
    return n;
}

// ---- grouped launch ---------------------------------------------------------------
extern "C" int nchip_gemm_grouped_tiles(int m, int n)
{
    return ((m + 127) / 128) * ((n + 127) / 128);
}

extern "C" int nchip_gemm_grouped(void *stream, int ta, int tb, const NchipGemmProblem *dev_table,
                                  int n_problems, int total_tiles, int precision, double total_flops)
{
    if (n_problems <= 0 || total_tiles <= 0) return 0;
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.grp = dev_table; g.n_grp = n_problems;
    // 16 tiles per turn: measured at C3 (1156 tiles), FETCH_SIZE of the launch 3.18 GB at 1 (plain
    // round robin), 2.67 at 8, 2.13 at 16, duration 1574 / 1555 / 1563 us; from 32 on the runs
    // are long enough for the XCDs to finish apart (1692 us)
    { static const int gc = getenv("NCHIP_GRP_CHUNK") ? atoi(getenv("NCHIP_GRP_CHUNK")) : 16; g.grp_chunk = gc; }
    g.batch = 1; g.batch_in = 1; g.ksplit = 1;
    g.beta = 0.0f; g.act = 0;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(total_tiles, 1), block(precision == 2 ? 256 : 512);
    ProfRec rec;
    if (g_prof_on) {
        (void)hipEventCreate(&rec.start);
        (void)hipEventCreate(&rec.stop);
        rec.variant = precision == 2 ? 32 + (ta ? 2 : 0) + (tb ? 1 : 0)
                                     : 2 * 8 + (ta ? 4 : 0) + (tb ? 2 : 0) + (precision == 1 ? 1 : 0);
        rec.flops = total_flops;
    }
#define GRP_LAUNCH(KERNEL, BK_, TA, TB, BF)                                                                \
    do {                                                                                                   \
        constexpr size_t dyn = lds_dynamic_bytes<128, 128, BK_, TA, TB, BF>();                             \
        if (dyn) {                                                                                         \
            static const bool ok = hipFuncSetAttribute(reinterpret_cast<const void *>(KERNEL),             \
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) == hipSuccess;                       \
            if (!ok) { fprintf(stderr, "nchip_gemm_grouped: cannot reserve %zu bytes of LDS\n", dyn); return -2; } \
        }                                                                                                  \
        if (g_prof_on) hipExtLaunchKernelGGL(KERNEL, grid, block, dyn, st, rec.start, rec.stop, 0, g);     \
        else hipLaunchKernelGGL(KERNEL, grid, block, dyn, st, g);                                          \
    } while (0)
#define GRP(TA, TB, BF) GRP_LAUNCH((gemm_kernel<128, 128, 32, 4, 2, TA, TB, BF, 1, 2, 0, 1, (BF == 0)>), 32, TA, TB, BF)
#define GRP16(TA, TB) GRP_LAUNCH((gemm_kernel<128, 128, 64, 2, 2, TA, TB, 2, 1>), 64, TA, TB, 2)
    if (precision == 2) {
        if (!ta && !tb) GRP16(0, 0); else if (ta && !tb) GRP16(1, 0); else if (!ta && tb) GRP16(0, 1); else GRP16(1, 1);
    } else if (precision == 1) {
        if (!ta && !tb) GRP(0, 0, 1); else if (ta && !tb) GRP(1, 0, 1); else if (!ta && tb) GRP(0, 1, 1); else GRP(1, 1, 1);
    } else {
        if (!ta && !tb) GRP(0, 0, 0); else if (ta && !tb) GRP(1, 0, 0); else if (!ta && tb) GRP(0, 1, 0); else GRP(1, 1, 0);
    }
#undef GRP
#undef GRP16
#undef GRP_LAUNCH
    if (g_prof_on) g_prof.push_back(rec);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fprintf(stderr, "nchip_gemm_grouped: launch failed: %s\n", hipGetErrorString(e));
        return -2;
    }
    return 0;
}
