/*
 * Single-precision GEMM of the CPU checker (test infrastructure only).
 * Column-major, C = alpha*op(A)*op(B) + beta*C.  Each output element is one
 * sequential dot product over k = 0..K-1 (no k-splitting), so the result does
 * not depend on the thread count or on where the element sits in a tile.
 * Packed 16x6 register tile with GCC vector extensions, OpenMP over column
 * panels: fast enough to serve as the timed CPU baseline.
 */
#include <omp.h>
#include "nc_ref_internal.h"

#define MR 16
#define NR 6

typedef float v8f __attribute__((vector_size(32), aligned(4)));

static void pack_a(int ta, int m, int k, const float *a, int lda, float *ap)
{
    /* panels of MR rows: ap[p][kk][r] = op(A)[p*MR + r][kk] */
    int np = (m + MR - 1) / MR;
    #pragma omp parallel for
    for (int p = 0; p < np; p++) {
        float *dst = ap + (size_t)p * MR * k;
        for (int kk = 0; kk < k; kk++)
            for (int r = 0; r < MR; r++) {
                int i = p * MR + r;
                float v = 0.0f;
                if (i < m)
                    v = ta ? a[(size_t)i * lda + kk] : a[(size_t)kk * lda + i];
                dst[kk * MR + r] = v;
            }
    }
}

static void pack_b(int tb, int n0, int nr, int k, const float *b, int ldb, float *bp)
{
    /* bp[kk][c] = op(B)[kk][n0 + c], zero padded to NR columns */
    for (int kk = 0; kk < k; kk++)
        for (int c = 0; c < NR; c++) {
            float v = 0.0f;
            if (c < nr)
                v = tb ? b[(size_t)kk * ldb + (n0 + c)] : b[(size_t)(n0 + c) * ldb + kk];
            bp[kk * NR + c] = v;
        }
}

static inline void ukernel(int k, const float *ap, const float *bp, float *acc)
{
    v8f c[NR][2];
    for (int j = 0; j < NR; j++)
        c[j][0] = c[j][1] = (v8f){ 0, 0, 0, 0, 0, 0, 0, 0 };
    for (int kk = 0; kk < k; kk++) {
        v8f a0 = *(const v8f *)(ap), a1 = *(const v8f *)(ap + 8);
        for (int j = 0; j < NR; j++) {
            float bv = bp[j];
            v8f b = { bv, bv, bv, bv, bv, bv, bv, bv };
            c[j][0] += a0 * b;
            c[j][1] += a1 * b;
        }
        ap += MR;
        bp += NR;
    }
    for (int j = 0; j < NR; j++) {
        *(v8f *)(acc + j * MR) = c[j][0];
        *(v8f *)(acc + j * MR + 8) = c[j][1];
    }
}

void ref_sgemm(int ta, int tb, int m, int n, int k, float alpha,
               const float *a, int lda, const float *b, int ldb,
               float beta, float *c, int ldc)
{
    int mp = (m + MR - 1) / MR, np = (n + NR - 1) / NR;
    float *ap;
    if (m <= 0 || n <= 0)
        return;
    ap = nc_malloc(sizeof(float) * (size_t)mp * MR * (k > 0 ? k : 1) + 64);
    pack_a(ta, m, k, a, lda, ap);
    #pragma omp parallel
    {
        float *bp = nc_malloc(sizeof(float) * NR * (k > 0 ? k : 1) + 64);
        float acc[MR * NR];
        #pragma omp for schedule(static)
        for (int q = 0; q < np; q++) {
            int n0 = q * NR, nr = n - n0 < NR ? n - n0 : NR;
            pack_b(tb, n0, nr, k, b, ldb, bp);
            for (int p = 0; p < mp; p++) {
                int m0 = p * MR, mr = m - m0 < MR ? m - m0 : MR;
                ukernel(k, ap + (size_t)p * MR * k, bp, acc);
                for (int j = 0; j < nr; j++)
                    for (int i = 0; i < mr; i++) {
                        float *dst = &c[(size_t)(n0 + j) * ldc + m0 + i];
                        float v = alpha * acc[j * MR + i];
                        *dst = beta == 0.0f ? v : v + beta * *dst;
                    }
            }
        }
        free(bp);
    }
    free(ap);
}
