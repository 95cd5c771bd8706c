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

// floor(num / den) for num < 2^56, den < 2^41 and a quotient below 2^16: a
// double-precision estimate (relative error < 2^-50, so at most one off after
// truncation) corrected by the exact 64-bit remainder.
__device__ __forceinline__ unsigned int div_floor(unsigned long long num, unsigned long long den, double inv)
{
    double d = fma((double)(unsigned int)(num >> 32), 4294967296.0, (double)(unsigned int)num);
    unsigned int q = (unsigned int)(d * inv);
    long long r = (long long)num - (long long)((unsigned long long)q * den);
    if (r < 0) q--;
    else if (r >= (long long)den) q++;
    return q;
}

__device__ __forceinline__ unsigned long long wave_scan_incl(unsigned long long v, int lane)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        unsigned long long o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}

// One workgroup of NT threads per column (NT == 64: one wave per column, four
// columns per workgroup).  The column is cut into chunks of 4*NT elements; in
// a chunk thread t owns the 4 consecutive elements starting at 4*t, so the
// loads and the uint16 stores of a wave cover one contiguous span, the logits
// are read once and stay in registers, and the exclusive prefix of an element
// is (chunks before) + (waves before, via LDS) + (lanes before, via shuffles)
// + (own earlier elements).  All sums are integers, so their grouping does
// not change the result.
//
// PATH: the caller knows each column's symbol and wants only what a coder reads for it - the CDF
// entry at the split point of every level of the balanced tree over [0, v) (cp_utils.c:299-323),
// `levels` 16-bit values per column, 0 below the leaf.  Nothing else is divided or stored: the
// kernel is then one read of the logits.  Whatever the symbol's value, the split points lie in [1, v).
// (eight waves per SIMD asked of the compiler: two 1024-thread workgroups share a CU only when the
// scalar registers allow all 32 waves, and with one the phases of a column have nothing to overlap)
template <int NT, int NC, bool KEEP, bool PATH>
__global__ __launch_bounds__(NT == 64 ? 256 : NT) __attribute__((amdgpu_waves_per_eu(NT >= 1024 ? 8 : 4))) void softmax_cdf16_kernel(const float *logits, uint16_t *cdf,
                                                                        int v, int64_t ncol, int vec,
                                                                        const int32_t *sym, uint16_t *path, int levels)
{
    constexpr int NW = NT / 64;
    constexpr int UNR = KEEP ? NC : 1; // chunk loops stay rolled when chunks are re-read
    __shared__ float smax[NW];
    __shared__ unsigned long long swave[NC][NW];
    __shared__ unsigned long long stot;
    const int lane = threadIdx.x & 63;
    const int wave = NT == 64 ? 0 : (int)threadIdx.x >> 6;
    const int t = NT == 64 ? lane : (int)threadIdx.x;
    const int64_t col = NT == 64 ? (int64_t)blockIdx.x * 4 + ((int)threadIdx.x >> 6) : (int64_t)blockIdx.x;
    if (NT == 64 && col >= ncol) return; // whole wave; this shape uses no workgroup barrier
    const float *x = logits + col * v;
    uint16_t *out = PATH ? nullptr : cdf + col * v;
    // the split points of the symbol's walk, the same for every thread of the column: two 16-bit
    // values per register (a split point is below v <= 65535; 0xffff = the walk ended above this level)
    unsigned int split2[PATH ? 8 : 1];
    auto split_at = [&](int l) -> int {
        const unsigned int s16 = (split2[l >> 1] >> ((l & 1) * 16)) & 0xffffu;
        return s16 == 0xffffu ? -1 : (int)s16;
    };
    if (PATH) {
        const int s = sym[col];
        int start = 0, len = v;
#pragma unroll
        for (int l = 0; l < 16; l++) {
            unsigned int here = 0xffffu;
            if (l < levels && len > 1) {
                const int n0 = len >> 1;
                here = (unsigned int)(start + n0);
                if (s >= start + n0) { start += n0; len -= n0; }
                else len = n0;
            }
            split2[l >> 1] = (l & 1) ? (split2[l >> 1] | here << 16) : here;
        }
    }

    // KEEP: the logits stay in registers from the first read on; otherwise
    // (columns too long for that) each pass reads its chunk again, from L2
    float xv[KEEP ? NC : 1][4];
    auto fetch = [&](int c, float (&f)[4]) {
        int i0 = (c * NT + t) * 4;
        if (vec && i0 < v) {
            float4 g = *reinterpret_cast<const float4 *>(x + i0);
            f[0] = g.x; f[1] = g.y; f[2] = g.z; f[3] = g.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) f[j] = i0 + j < v ? x[i0 + j] : -INFINITY;
        }
    };
    auto chunk = [&](int c, float (&f)[4]) {
        if (KEEP) {
#pragma unroll
            for (int j = 0; j < 4; j++) f[j] = xv[c][j];
        } else {
            fetch(c, f);
        }
    };
    float mx = -INFINITY;
#pragma unroll UNR
    for (int c = 0; c < NC; c++) {
        float f[4];
        fetch(c, f);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (KEEP) xv[c][j] = f[j];
            mx = fmaxf(mx, f[j]);
        }
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
    if (NT > 64) {
        if (lane == 0) smax[wave] = mx;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < NW; w++) mx = fmaxf(mx, smax[w]);
    }

    // pass 1: totals per (chunk, wave); the wave-level scan is redone in
    // pass 2 rather than kept, which holds the register count down
    unsigned long long wave_tot[NT == 64 ? NC : 1];
#pragma unroll UNR
    for (int c = 0; c < NC; c++) {
        int i0 = (c * NT + t) * 4;
        unsigned long long s = 0;
        float f[4];
        chunk(c, f);
#pragma unroll
        for (int j = 0; j < 4; j++) s += i0 + j < v ? quant(f[j], mx) : 0u;
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) s += __shfl_xor(s, d, 64);
        if (NT == 64) wave_tot[c] = s;
        if (NT > 64 && lane == 0) swave[c][wave] = s;
    }
    unsigned long long tot = 0;
    if (NT > 64) {
        __syncthreads();
        // wave 0 turns the wave totals of each chunk into exclusive prefixes
        // that run on through the chunks; the grand total goes to stot
        if (wave == 0) {
            unsigned long long run = 0;
#pragma unroll 1
            for (int c = 0; c < NC; c++) {
                unsigned long long w = lane < NW ? swave[c][lane] : 0ull;
                unsigned long long incl = wave_scan_incl(w, lane);
                if (lane < NW) swave[c][lane] = run + incl - w;
                run += __shfl(incl, 63, 64);
            }
            if (lane == 0) stot = run;
        }
        __syncthreads();
        tot = stot;
    } else {
#pragma unroll
        for (int c = 0; c < NC; c++) tot += wave_tot[c];
    }
    const unsigned long long scale = (unsigned long long)(65536 - v);
    const double inv = 1.0 / (double)tot;
    unsigned long long chunk_base = 0;
    if (PATH && t == 0) {
#pragma unroll
        for (int l = 0; l < 16; l++)
            if (split_at(l) < 0 && l < levels) path[col * levels + l] = 0; // below the leaf
    }
#pragma unroll UNR
    for (int c = 0; c < NC; c++) {
        int i0 = (c * NT + t) * 4;
        if (PATH) {
            // the 256 elements of this wave in this chunk hold a split point, or nothing here is needed
            // (NT == 64 adds the chunks up as it goes, so it passes through all of them)
            const int w0 = (c * NT + wave * 64) * 4;
            bool hit = NT == 64;
#pragma unroll
            for (int l = 0; l < 16; l++) hit = hit || (split_at(l) >= w0 && split_at(l) < w0 + 256);
            if (!hit) continue; // the same for the whole wave
        }
        unsigned int q[4];
        unsigned long long s = 0;
        float f[4];
        chunk(c, f);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            q[j] = i0 + j < v ? quant(f[j], mx) : 0u;
            s += q[j];
        }
        unsigned long long run = wave_scan_incl(s, lane) - s;
        if (NT > 64) {
            run += swave[c][wave];
        } else {
            run += chunk_base;
            chunk_base += wave_tot[c];
        }
        if (i0 >= v) continue;
        if (PATH) {
            uint16_t *po = path + col * levels;
            unsigned int own = 0; // the levels whose split point is one of this thread's four elements
#pragma unroll
            for (int l = 0; l < 16; l++) {
                const int dj = split_at(l) - i0;
                own |= (unsigned int)(split_at(l) >= 0 && dj >= 0 && dj < 4) << l;
            }
            if (own) { // rare: at most 16 threads of a column divide at all
                unsigned int o[4];
                unsigned long long r = run;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    o[j] = div_floor(r * scale, tot, inv) + (unsigned int)(i0 + j);
                    r += q[j];
                }
#pragma unroll
                for (int l = 0; l < 16; l++)
                    if (own >> l & 1) {
                        const int dj = split_at(l) - i0;
                        po[l] = (uint16_t)(dj == 0 ? o[0] : dj == 1 ? o[1] : dj == 2 ? o[2] : o[3]);
                    }
            }
            continue;
        }
        unsigned int o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            o[j] = div_floor(run * scale, tot, inv) + (unsigned int)(i0 + j);
            run += q[j];
        }
        if (vec) {
            uint2 pk;
            pk.x = (o[0] & 0xffffu) | (o[1] << 16);
            pk.y = (o[2] & 0xffffu) | (o[3] << 16);
            *reinterpret_cast<uint2 *>(out + i0) = pk;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (i0 + j < v) out[i0 + j] = (uint16_t)o[j];
        }
    }
}

// Cumulative-frequency search: sym = the index with cdf[sym] <= target <
// cdf[sym + 1] (cdf[v] = 65536).  The column's CDF is staged in LDS when it
// fits; each thread then runs four searches side by side, with a fixed trip
// count of ceil(log2 v) and selects instead of branches, so four LDS reads
// are in flight per lane (once hi - lo is 1 a further step changes nothing).
template <bool LDS>
__global__ __launch_bounds__(TPB) void cdf_lookup_kernel(const uint16_t *cdf, const uint16_t *target,
                                                         uint16_t *sym, int v, int64_t m, int steps)
{
    __shared__ uint16_t sc[LDS ? 16384 : 1];
    const uint16_t *c = cdf + (int64_t)blockIdx.y * v;
    if (LDS) {
        for (int i = threadIdx.x; i < v; i += TPB) sc[i] = c[i];
        __syncthreads();
    }
    const uint16_t *tp = target + (int64_t)blockIdx.y * m;
    uint16_t *sp = sym + (int64_t)blockIdx.y * m;
    const int64_t stride = (int64_t)gridDim.x * TPB;
    for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < m; i += 4 * stride) {
        unsigned int tv[4];
        int lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int64_t ij = i + j * stride;
            tv[j] = tp[ij < m ? ij : i];
            lo[j] = 0;
            hi[j] = v;
        }
        for (int s = 0; s < steps; s++) {
            unsigned int cv[4];
            int mid[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                mid[j] = (lo[j] + hi[j]) >> 1;
                cv[j] = LDS ? sc[mid[j]] : c[mid[j]];
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                bool le = cv[j] <= tv[j];
                lo[j] = le ? mid[j] : lo[j];
                hi[j] = le ? hi[j] : mid[j];
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int64_t ij = i + j * stride;
            if (ij < m) sp[ij] = (uint16_t)lo[j];
        }
    }
}

// Many targets per column: first turn the column's CDF into the full inverse
// table inv[t] = symbol of target value t (65536 uint16 entries, 128 KiB of
// LDS; each entry by the same search, read from the cached CDF), after which
// a lookup is one LDS read.  Entry t depends on the CDF alone, so the result
// is the one the search gives.
constexpr int INV_NT = 1024;
__global__ __launch_bounds__(INV_NT) void cdf_lookup_table_kernel(const uint16_t *cdf, const uint16_t *target,
                                                                  uint16_t *sym, int v, int64_t m, int steps,
                                                                  int vec)
{
    extern __shared__ __attribute__((aligned(16))) uint16_t inv[];
    __shared__ uint16_t coarse[INV_NT + 1];
    const uint16_t *c = cdf + (int64_t)blockIdx.y * v;
    {   // the symbol of every 64th target value, by the full search
        int lo = 0, hi = v;
        unsigned int tv = threadIdx.x * 64;
        for (int s = 0; s < steps; s++) {
            int mid = (lo + hi) >> 1;
            bool le = c[mid] <= tv;
            lo = le ? mid : lo;
            hi = le ? hi : mid;
        }
        coarse[threadIdx.x] = (uint16_t)lo;
        if (threadIdx.x == 0) coarse[INV_NT] = (uint16_t)(v - 1);
    }
    __syncthreads();
    // the symbols of target values 64 b .. 64 b + 63 lie between coarse[b] and
    // coarse[b + 1], at most 65 candidates (every symbol has frequency >= 1):
    // 7 halvings finish each of them; eight run side by side
    for (int t0 = threadIdx.x; t0 < 65536; t0 += 8 * INV_NT) {
        int lo[8], hi[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            int bkt = (t0 + j * INV_NT) >> 6;
            lo[j] = coarse[bkt];
            hi[j] = coarse[bkt + 1] + 1;
        }
#pragma unroll
        for (int s = 0; s < 7; s++) {
            unsigned int cv[8];
            int mid[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                mid[j] = (lo[j] + hi[j]) >> 1;
                cv[j] = c[mid[j]];
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                bool le = cv[j] <= (unsigned int)(t0 + j * INV_NT);
                lo[j] = le ? mid[j] : lo[j];
                hi[j] = le ? hi[j] : mid[j];
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) inv[t0 + j * INV_NT] = (uint16_t)lo[j];
    }
    __syncthreads();
    const uint16_t *tp = target + (int64_t)blockIdx.y * m;
    uint16_t *sp = sym + (int64_t)blockIdx.y * m;
    // this workgroup's share of the column, cut at multiples of 4 targets
    int64_t quads = (m + 3) >> 2;
    int64_t per = (quads + gridDim.x - 1) / gridDim.x;
    int64_t q0 = per * blockIdx.x, q1 = q0 + per < quads ? q0 + per : quads;
    if (vec) {
        // four 8-byte loads in flight per lane (index clamped, store guarded)
        for (int64_t q = q0 + threadIdx.x; q < q1; q += 4 * INV_NT) {
            uint2 tv[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                int64_t qj = q + j * INV_NT;
                tv[j] = *reinterpret_cast<const uint2 *>(tp + 4 * (qj < q1 ? qj : q));
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                int64_t qj = q + j * INV_NT;
                uint2 r;
                r.x = (unsigned int)inv[tv[j].x & 0xffffu] | ((unsigned int)inv[tv[j].x >> 16] << 16);
                r.y = (unsigned int)inv[tv[j].y & 0xffffu] | ((unsigned int)inv[tv[j].y >> 16] << 16);
                if (qj < q1) *reinterpret_cast<uint2 *>(sp + 4 * qj) = r;
            }
        }
    } else {
        int64_t i1 = 4 * q1 < m ? 4 * q1 : m;
        for (int64_t i = 4 * q0 + threadIdx.x; i < i1; i += INV_NT) sp[i] = inv[tp[i]];
    }
}

bool allow_table_lds()
{
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(cdf_lookup_table_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 65536 * 2) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return true;
}

// Integer probabilities of libnc's nc_soft_max_int: y[i] = max(floor(q[i] * mult / Q), 1)
// with the same 24-bit integer exponentials q and their exact sum Q as the CDF above.
// q[i] * mult is exact in double (25 + 24 significant bits), the division is the one
// correctly rounded IEEE operation, so the CPU checker computes the same integers.  One
// workgroup per column, three passes over the column (maximum, sum, values): the second and
// third read it from cache.  Not on the coder's path (nncp.c does not call it).
__global__ __launch_bounds__(TPB) void softmax_int_kernel(const float *logits, int32_t *out, int v, float mult)
{
    __shared__ float s_max[TPB];
    __shared__ unsigned long long s_sum[TPB];
    const float *x = logits + (int64_t)blockIdx.x * v;
    int32_t *y = out + (int64_t)blockIdx.x * v;
    const int t = threadIdx.x;
    float mx = x[0];
    for (int i = t; i < v; i += TPB) mx = x[i] > mx ? x[i] : mx;
    s_max[t] = mx;
    __syncthreads();
    for (int d = TPB / 2; d > 0; d >>= 1) {
        if (t < d) s_max[t] = s_max[t + d] > s_max[t] ? s_max[t + d] : s_max[t];
        __syncthreads();
    }
    mx = s_max[0];
    unsigned long long tot = 0;
    for (int i = t; i < v; i += TPB) tot += quant(x[i], mx);
    s_sum[t] = tot;
    __syncthreads();
    for (int d = TPB / 2; d > 0; d >>= 1) {
        if (t < d) s_sum[t] += s_sum[t + d];
        __syncthreads();
    }
    const double q_total = (double)s_sum[0], m = (double)mult;
    for (int i = t; i < v; i += TPB) {
        double p = (double)quant(x[i], mx) * m / q_total;
        y[i] = p >= 2147483647.0 ? 2147483647 : (p >= 1.0 ? (int32_t)p : 1);
    }
}

} // namespace

extern "C" int nchip_softmax_int(void *stream, const float *logits, int32_t *out, int v, int64_t n, float mult)
{
    if (n <= 0) return 0;
    if (v < 1 || n > 0x7fffffff || !(mult >= 0.0f) || mult > 4294967296.0f) {
        fprintf(stderr, "nchip_softmax_int: v %d, n %lld or mult %g outside what the kernel takes\n", v, (long long)n, (double)mult);
        return -1;
    }
    hipLaunchKernelGGL(softmax_int_kernel, dim3((unsigned)n), dim3(TPB), 0, (hipStream_t)stream, logits, out, v, mult);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { fprintf(stderr, "nchip_softmax_int: %s\n", hipGetErrorString(e)); return -2; }
    return 0;
}

template <bool PATH>
static void launch_softmax_cdf16(hipStream_t st, const float *logits, uint16_t *cdf, int v, int64_t n, int vec,
                                 const int32_t *sym, uint16_t *path, int levels)
{
    if (v <= 256)
        hipLaunchKernelGGL((softmax_cdf16_kernel<64, 1, true, PATH>), dim3((unsigned)((n + 3) / 4)), dim3(256), 0, st, logits, cdf, v, n, vec, sym, path, levels);
    else if (v <= 1024)
        hipLaunchKernelGGL((softmax_cdf16_kernel<256, 1, true, PATH>), dim3((unsigned)n), dim3(256), 0, st, logits, cdf, v, n, vec, sym, path, levels);
    else if (v <= 4096)
        hipLaunchKernelGGL((softmax_cdf16_kernel<256, 4, true, PATH>), dim3((unsigned)n), dim3(256), 0, st, logits, cdf, v, n, vec, sym, path, levels);
    else if (v <= 16384)
        hipLaunchKernelGGL((softmax_cdf16_kernel<1024, 4, true, PATH>), dim3((unsigned)n), dim3(1024), 0, st, logits, cdf, v, n, vec, sym, path, levels);
    else
        hipLaunchKernelGGL((softmax_cdf16_kernel<1024, 16, false, PATH>), dim3((unsigned)n), dim3(1024), 0, st, logits, cdf, v, n, vec, sym, path, levels);
}

extern "C" int nchip_softmax_cdf16(void *stream, const float *logits, uint16_t *cdf, int v, int64_t n)
{
    if (n <= 0) return 0;
    if (v < 1 || v > 65535) { fprintf(stderr, "nchip_softmax_cdf16: vocabulary %d outside [1, 65535]\n", v); return -1; }
    // 16-byte loads and 8-byte stores need every column to start aligned
    int vec = (v & 3) == 0 && ((uintptr_t)logits & 15) == 0 && ((uintptr_t)cdf & 7) == 0;
    launch_softmax_cdf16<false>((hipStream_t)stream, logits, cdf, v, n, vec, nullptr, nullptr, 0);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { fprintf(stderr, "nchip_softmax_cdf16: %s\n", hipGetErrorString(e)); return -2; }
    return 0;
}

extern "C" int nchip_softmax_cdf16_path(void *stream, const float *logits, const int32_t *sym, uint16_t *path,
                                        int v, int64_t n, int levels)
{
    if (n <= 0 || levels <= 0) return 0;
    if (v < 1 || v > 65535) { fprintf(stderr, "nchip_softmax_cdf16_path: vocabulary %d outside [1, 65535]\n", v); return -1; }
    if (levels > 16 || (1 << levels) < v) { fprintf(stderr, "nchip_softmax_cdf16_path: %d levels for %d symbols\n", levels, v); return -1; }
    int vec = (v & 3) == 0 && ((uintptr_t)logits & 15) == 0;
    launch_softmax_cdf16<true>((hipStream_t)stream, logits, nullptr, v, n, vec, sym, path, levels);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { fprintf(stderr, "nchip_softmax_cdf16_path: %s\n", hipGetErrorString(e)); return -2; }
    return 0;
}

// What a binary-tree coder reads of a column when it knows the symbol: at every level of the
// balanced tree over [0, v) (cp_utils.c:299-323) the CDF entry at the split point.  One thread per
// column walks the tree for its symbol; whatever the symbol's value, start + n0 < v.
__global__ __launch_bounds__(TPB) void cdf_path_kernel(const uint16_t *cdf, const int32_t *sym, uint16_t *path,
                                                        int v, int64_t ncol, int levels)
{
    const int64_t c = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (c >= ncol) return;
    const uint16_t *col = cdf + c * v;
    uint16_t *out = path + c * levels;
    const int s = sym[c];
    int start = 0, n = v;
    for (int l = 0; l < levels; l++) {
        uint16_t mid = 0;
        if (n > 1) {
            const int n0 = n >> 1;
            mid = col[start + n0];
            if (s >= start + n0) { start += n0; n -= n0; }
            else n = n0;
        }
        out[l] = mid;
    }
}

extern "C" int nchip_cdf_path(void *stream, const uint16_t *cdf, const int32_t *sym, uint16_t *path,
                              int v, int64_t n, int levels)
{
    if (n <= 0 || levels <= 0) return 0;
    if (v <= 0 || (levels < 31 && (1 << levels) < v)) { fprintf(stderr, "nchip_cdf_path: %d levels do not reach %d symbols\n", levels, v); return -1; }
    hipLaunchKernelGGL(cdf_path_kernel, dim3((unsigned)((n + TPB - 1) / TPB)), dim3(TPB), 0, (hipStream_t)stream, cdf, sym, path, v, n, levels);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { fprintf(stderr, "nchip_cdf_path: %s\n", hipGetErrorString(e)); return -2; }
    return 0;
}

extern "C" int nchip_cdf_lookup(void *stream, const uint16_t *cdf, const uint16_t *target,
                                uint16_t *sym, int v, int64_t m, int64_t n)
{
    if (n <= 0 || m <= 0) return 0;
    if (n > 65535) { fprintf(stderr, "nchip_cdf_lookup: too many columns\n"); return -1; }
    // every workgroup of a column stages that column's CDF in LDS first, so
    // use only as many per column as fill the chip a few times over
    int steps = 0;
    while ((1 << steps) < v) steps++;
    int64_t bx = (m + TPB * 16 - 1) / (TPB * 16);
    int64_t cap = (4096 + n - 1) / n;
    if (bx > cap) bx = cap;
    // the table costs 65536 searches per workgroup: worth it from a few times
    // that many targets per workgroup on
    static const bool table_ok = allow_table_lds();
    if (table_ok && m >= 4 * 65536) {
        int64_t split = (256 + n - 1) / n; // workgroups per column: one per CU (the table fills its LDS)
        if (split > m / (2 * 65536)) split = m / (2 * 65536);
        if (split < 1) split = 1;
        // 8-byte accesses need every column (m targets apart) to start aligned
        int vec = (m & 3) == 0 && ((uintptr_t)target & 7) == 0 && ((uintptr_t)sym & 7) == 0;
        hipLaunchKernelGGL(cdf_lookup_table_kernel, dim3((unsigned)split, (unsigned)n), dim3(INV_NT), 65536 * 2,
                           (hipStream_t)stream, cdf, target, sym, v, m, steps, vec);
    } else {
        dim3 grid((unsigned)bx, (unsigned)n);
        if (v <= 16384)
            hipLaunchKernelGGL(cdf_lookup_kernel<true>, grid, dim3(TPB), 0, (hipStream_t)stream, cdf, target, sym, v, m, steps);
        else
            hipLaunchKernelGGL(cdf_lookup_kernel<false>, grid, dim3(TPB), 0, (hipStream_t)stream, cdf, target, sym, v, m, steps);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { fprintf(stderr, "nchip_cdf_lookup: %s\n", hipGetErrorString(e)); return -2; }
    return 0;
}
