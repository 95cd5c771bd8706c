/*
 * nchip_kernels.h - the thin C ABI over the hand-written gfx950 kernels of
 * libnc_hip.so.  Plain device pointers and sizes, no C++ or torch types; every
 * entry point enqueues on `stream` (a hipStream_t passed as void*) and returns
 * 0, or a negative value after printing the reason when the arguments do not
 * fit what the kernel assumes.  Matrices are column-major as in libnc
 * (libnc.h:106-115): element (i, j) of an m x n matrix with leading dimension
 * ld lives at base[i + j*ld].  The libnc-level ops of nc_api.h / nc_ext.h are
 * thin wrappers over these.
 */
#ifndef NCHIP_KERNELS_H
#define NCHIP_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NCHIP_ACT_NONE 0
#define NCHIP_ACT_GELU 1
#define NCHIP_ACT_RELU 2

/* or-ed into `precision`: use the tile class and reduction order that do not
   depend on m or n (64x64 tiles, two interleaved k chains, no split-K), so a
   column computed alone is bit-identical to the same column of a wide product */
#define NCHIP_GEMM_WIDTH_INVARIANT 0x100

/* C = act(alpha * op(A) * op(B) + beta * C + bias), batched.
   Replaces nc_matmul / nc_matmul_add (libnc.h:365-373, call sites
   nncp.c:659-1004).  op(A) is m x k: A is (m,k) when ta == 0, (k,m) when
   ta == 1; likewise B is (k,n) or (n,k).  bias (m) may be NULL.  When `pre`
   is not NULL the value before the activation is stored there too (same
   layout as C).  precision 0: fp32 MFMA; 1: operands rounded to bf16
   (nearest-even) on load, fp32 accumulation on the bf16 MFMA units.
   ksplit > 1 splits the reduction over that many workgroups whose partial
   tiles are summed in a fixed order by a second kernel; it needs
   `workspace` of at least batch*ksplit*m*n floats.  Every output element is a
   sequential MFMA accumulation chain over k = 0..K-1 that does not depend on
   m, n or the tile shape. */
int nchip_gemm(void *stream, int ta, int tb, int m, int n, int k, float alpha,
               const float *A, int64_t lda, int64_t stride_a,
               const float *B, int64_t ldb, int64_t stride_b,
               float beta, float *C, int64_t ldc, int64_t stride_c, int batch,
               const float *bias, int act, float *pre, int precision,
               int ksplit, float *workspace);

/* C = act(alpha * op(A) * op(B) + bias) + addend, with addend laid out like C
   (ldc, stride_c; may alias nothing written by the call).  Used for residual
   connections (nncp.c:803, 975) and to add an incoming gradient in the same
   pass instead of a separate element-wise sum. */
int nchip_gemm_add(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                   const float *A, int64_t lda, int64_t stride_a,
                   const float *B, int64_t ldb, int64_t stride_b,
                   float *C, int64_t ldc, int64_t stride_c, int batch,
                   const float *bias, int act, float *pre, const float *addend,
                   int precision, int ksplit, float *workspace);

/* C = (alpha * op(A) * op(B)) .* act'(pre_act): the input gradient of a linear
   layer whose input came out of an activation (pre_act = the values before
   that activation, laid out like C).  One GEMM instead of a GEMM and an
   element-wise pass; the product is rounded to fp32 before the multiplication,
   as the two-pass form does. */
int nchip_gemm_dact(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                    const float *A, int64_t lda, const float *B, int64_t ldb,
                    float *C, int64_t ldc, const float *pre_act, int act,
                    int precision, int ksplit, float *workspace);

/* Same with two-level batching: batch index z addresses
   A + (z / batch_in)*sa_out + (z % batch_in)*sa_in (likewise B and C).  Lets
   per-(stream, head) products read the (features, streams, time) activations
   in place, without the split_head / concat_head copies of nncp.c:554-579. */
int nchip_gemm2(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                const float *A, int64_t lda, int64_t sa_out, int64_t sa_in,
                const float *B, int64_t ldb, int64_t sb_out, int64_t sb_in,
                float beta, float *C, int64_t ldc, int64_t sc_out, int64_t sc_in,
                int batch, int batch_in,
                const float *bias, int act, float *pre, int precision,
                int ksplit, float *workspace);

/* Many independent GEMMs C_p = alpha_p * op(A_p) * op(B_p) in ONE launch (same
   transposition flags, 128x128 tiles, no bias/activation, beta = 0).  The
   weight-gradient GEMMs dW = dY X^T of a whole backward pass are issued this
   way: each is too small to fill 256 CUs on its own.  dev_table lives in
   device memory; tile_start is the running sum of
   nchip_gemm_grouped_tiles(m, n) over the preceding problems.  total_flops
   (sum of 2*m*n*k) is only recorded by the optional launch timing. */
typedef struct {
    const float *A, *B;
    float *C;
    const float *A2, *B2; /* optional second k range: C = alpha*(op(A)op(B) + op(A2)op(B2)) */
    int m, n, k, k2;      /* k2 = 0 without A2/B2; with them k must be a multiple of 64 */
    int lda, ldb, ldc;    /* A2 / B2 use lda / ldb too */
    int tile_start;
    float alpha;
} NchipGemmProblem;
int nchip_gemm_grouped_tiles(int m, int n);
/* precision 0: fp32; 1: fp32 operands rounded to bf16 in the tile loader; 2: the operand
   pointers of the table address bf16 copies (2 bytes per element, same layout and leading
   dimensions as the fp32 matrices they were rounded from), read with unguarded 16-byte
   loads - every k and k2 a multiple of 64, every row-contiguous operand extent (m with
   ta = 0, n with tb = 1) a multiple of 128, leading dimensions multiples of 8, bases 16-byte
   aligned; the caller checks.  C is fp32 in all three. */
int nchip_gemm_grouped(void *stream, int ta, int tb, const NchipGemmProblem *dev_table,
                       int n_problems, int total_tiles, int precision, double total_flops);

/* One product C = act(alpha op(A) op(B) + bias) [+ addend] whose operands are read as bf16
   from memory: A16 / B16 address the bf16 copies of the fp32 matrices (element for element,
   same column-major layout and leading dimensions, no padding), accumulation in fp32 on
   v_mfma_f32_32x32x16_bf16.  The values are those of nchip_gemm with precision 1 up to the
   order of the k sum inside a tile class.  Unguarded 16-byte loads throughout: k a multiple
   of 64, leading dimensions multiples of 8, bases 16-byte aligned, and an operand whose long
   axis is contiguous (A with ta = 0, B with tb = 1) must fill whole tiles of the class the
   shape selects (128 or 64 rows / columns).  Returns 1 when the shape does not fit (nothing
   launched: the caller takes another route), 0 when launched, negative on error.
     pre / addend / dpre+dact / rowsum+rows_written: as in nchip_gemm_add, nchip_gemm_dact and
     nchip_gemm_dact_rowsum (all optional);
     C16: when not NULL, the result once more, rounded to bf16 (nearest even), laid out like
     C with the same ldc - the operand copy of a later product, so that C is never cast. */
typedef struct {
    int ta, tb, m, n, k;
    float alpha;
    const uint16_t *A16, *B16;
    int64_t lda, ldb;
    float *C;
    int64_t ldc;
    uint16_t *C16;
    const float *bias;
    int act;
    float *pre;
    const float *addend;
    const float *dpre;
    int dact;
    float *rowsum;
    int *rows_written;
} NchipGemmBf16Args;
int nchip_gemm_bf16_operands(void *stream, const NchipGemmBf16Args *a);
/* tuning aid: 0 = tile class from the shape, 1 = 128x128, 2 = 128x64, 3 = 64x64 (all 64 deep) */
void nchip_gemm_bf16_operands_class(int cls);

/* Optional timing of every GEMM launch with HIP events on the launch stream.
   After nchip_gemm_profile_enable(1), each nchip_gemm* dispatch carries an
   event pair bound to its own start / stop timestamps (hipExtLaunchKernelGGL;
   a split-K reduction pass is not included); nchip_gemm_profile_read waits for them, sums
   launches / flops (2*m*n*k*batch) / seconds per kernel instantiation, fills up
   to max_variants rows and clears the records.  Returns the row count. */
void nchip_gemm_profile_enable(int on);
int nchip_gemm_profile_read(int max_variants, char (*names)[48], int64_t *launches,
                            double *flops, double *seconds);

/* Tuning aid: forces tile configuration `cfg` (an index into the table in
   k_gemm.hip) for every later nchip_gemm* call; 0 restores the automatic
   choice.  The environment variable NCHIP_GEMM_CFG sets the initial value. */
void nchip_gemm_force_config(int cfg);

/* nchip_gemm_dact that also leaves partial row sums of C (the bias gradient of the layer whose
   pre-activation gradient C is): `rowsum` holds nchip_gemm_rowsum_rows(n) rows of m floats;
   *rows_written of them are written.  Row p is the sum over 16 columns of C, the 16 that one lane
   of the epilogue holds: of the 32-column block p / 2, the columns c with c mod 8 in
   [4 (p mod 2), 4 (p mod 2) + 4) - four runs of 4 consecutive columns, 8 apart - added in
   increasing column order (columns past n count as zero).  Rows 2j and 2j + 1 together cover
   block j, so the sum of all rows in row order is the row sum of C.  *rows_written is 0
   when the kernel chosen for this product does not write them (split-K, bf16 operand copies):
   the caller then sums C itself. */
int nchip_gemm_rowsum_rows(int n);
int nchip_gemm_dact_rowsum(void *stream, int ta, int tb, int m, int n, int k, float alpha,
                           const float *A, int64_t lda, const float *B, int64_t ldb,
                           float *C, int64_t ldc, const float *pre_act, int act,
                           int precision, int ksplit, float *workspace,
                           float *rowsum, int *rows_written);

/* Two width-invariant fp32 products that share their right operand, in one launch:
   C0 (m0 x n) = A0 (m0 x k) B (k x n) + bias0 and C1 (m1 x n) = A1 (m1 x k) B + bias1, column
   major, untransposed, bias pointers may be NULL (the per-timestep query and key/value
   projections of the decoder, nncp.c:801-812, whose second result goes straight into its
   cache slot).  The bits are those of two nchip_gemm calls with NCHIP_GEMM_WIDTH_INVARIANT.
   a_k_major != 0: A0 and A1 are stored with k contiguous (element (i, kk) at A[kk + i * lda]: the
   transposed copy of a weight matrix), which a quarter of the cache lines serves; same bits.
   Returns 0, 1 when the shapes are not the few-column kernel's (n <= 64, k and both m
   multiples of 32, 16-byte aligned operands; nothing was launched), negative on error. */
int nchip_gemm_pair_few_columns(void *stream, int m0, int m1, int n, int k,
                                const float *A0, int64_t lda0, const float *A1, int64_t lda1,
                                const float *B, int64_t ldb,
                                float *C0, int64_t ldc0, float *C1, int64_t ldc1,
                                const float *bias0, const float *bias1, int a_k_major);

/* One or two width-invariant few-column products of the layer norm (avg = 1) or RMS norm
   (avg = 0) of B's columns, in one launch: C0 (m0 x n) = act0(A0 norm(B) + bias0) and, when
   m1 > 0, C1 (m1 x n) = A1 norm(B) + bias1.  B holds k = 128, 256 or 512 raw features per
   column; ln_w / ln_b are gain and bias (both or neither); the normalised columns are also
   written to ln_out (leading dimension ld_ln) when it is not NULL.  The decoder's timestep:
   the norm that ends one block (nncp.c:896-987, layer_norm of nncp.c:279-288) rides on the
   first product of the next.  The bits are those of nchip_norm_fwd followed by the products
   with NCHIP_GEMM_WIDTH_INVARIANT.  a_k_major as for nchip_gemm_pair_few_columns.  Returns 0, 1
   when the shapes are not this kernel's (nothing was launched), negative on error. */
int nchip_norm_gemm_few_columns(void *stream, const float *ln_w, const float *ln_b, float eps, int avg,
                                float *ln_out, int64_t ld_ln, int m0, int m1, int n, int k,
                                const float *A0, int64_t lda0, const float *A1, int64_t lda1,
                                const float *B, int64_t ldb, float *C0, int64_t ldc0,
                                float *C1, int64_t ldc1, const float *bias0, const float *bias1, int act0,
                                int a_k_major);

/* Testing aid: which kernel takes width-invariant fp32 products (NCHIP_GEMM_WIDTH_INVARIANT)
   with at most 64 columns, untransposed operands and beta = 0 (the decoder's per-timestep
   products).  3 (default): 16 x 16 tiles with v_mfma_f32_16x16x4_f32, the four wavefronts of a
   workgroup the four chains of the width-invariant class; 2: the vector-ALU kernel - an fp32
   MFMA accumulates its k values one after the other with fused multiply-adds, so the chains
   are formed by plain fma instructions, one chain per thread, 8 x 8 outputs per workgroup;
   1: 32-row tiles with v_mfma_f32_32x32x2_f32; 0: the tile kernel.  The results are the same
   bits in all four. */
void nchip_gemm_few_columns_kernel(int kernel);

/* Tuning aid: tiles are ordered, inside each XCD's run, in bands of `gm` tile
   rows (1 = plain column-major tile order; a negative value restores the
   default of 8). */
void nchip_gemm_force_band(int gm);

/* bf16 products (precision 1) and where the rounding happens: 0 = inside the
   tile loader, from the fp32 operands, always; 1 (default) = large unbatched
   products first write bf16 copies of both operands to a scratch buffer (one
   streaming pass each) and the tiles load those, half the bytes; 2 = every
   unbatched bf16 product takes that route (testing aid).  The rounded values
   and the accumulation order are the same on both routes.  The environment
   variable NCHIP_GEMM_BF16SRC sets the initial value. */
void nchip_gemm_bf16_source(int mode);

/* Chooses ksplit for nchip_gemm from the shape alone (never from data). */
int nchip_gemm_pick_ksplit(int m, int n, int k, int batch);

/* Relative-position causal attention, forward (nncp.c:722-800 fused).
   Layouts as in nc_relpos_attention (nc_ext.h): q (H*dk, B, T) with leading
   dimension ldq per token column, kv/kvm (H*dk+H*dv, B, T|M) with ldkv,
   w_r (dk, d_pos, H) or NULL, b_r (K, H) or NULL, out (H*dv, B, T) with ldo.
   probs (K, T, H, B) receives the attention probabilities (kept for the
   backward pass); rel (d_pos, T, H, B) is scratch for w_r^T q (unused when
   w_r is NULL).  precision as in nchip_gemm. */
int nchip_relpos_attn_fwd(void *stream, const float *q, int64_t ldq,
                          const float *kv, const float *kvm, int64_t ldkv,
                          const float *w_r, const float *b_r,
                          float *out, int64_t ldo, float *probs, float *rel,
                          int H, int dk, int dv, int B, int T, int M, int d_pos,
                          int attn_len, float b_r_scale, int precision);

/* The same for ONE query position t of the segment (the per-timestep step of a
   decoder, nncp.c:801-863): q and out are single token columns (H*dk, B) and
   (H*dv, B); kv is the segment's K/V cache (H*dk+H*dv, B, T) whose columns
   0..t are filled (later columns must hold finite values; they are masked).
   The result is bit-identical to column t of nchip_relpos_attn_fwd on the
   completed segment.  Only shapes of the single-kernel path (d_head 32 or 64,
   T <= 64, K <= 128, d_pos <= 128). */
int nchip_relpos_attn_fwd_step(void *stream, const float *q, int64_t ldq,
                               const float *kv, const float *kvm, int64_t ldkv,
                               const float *w_r, const float *b_r, float *out, int64_t ldo,
                               int H, int dk, int dv, int B, int T, int M, int d_pos,
                               int attn_len, float b_r_scale, int t);

/* Testing aid for the call above: 1 (default) runs the one-query kernel on the vector ALUs
   (fused multiply-add chains in the order the MFMAs of the whole-segment kernel accumulate),
   0 runs the whole-segment kernel with every query row the one query.  Same bits.  No
   counterpart in the reference. */
void nchip_relpos_attn_step_kernel(int scalar);

/* Heads of 128 features (nncp's enwik profile, nncp.c:2549): the forward is one kernel up to
   320 keys; the backward is one kernel up to 128 keys and the batched products beyond, where
   they are faster.  always = 1 makes the backward one kernel at every key count it holds
   (tests; shapes with many more (stream, head) pairs than CUs).  Same results to rounding.
   No counterpart in the reference. */
void nchip_relpos_attn_wide_backward(int always);

/* Kernel launches issued by the calling thread's last successful
   nchip_relpos_attn_fwd (1 when the head fits the single-kernel path). */
int nchip_relpos_attn_last_launches(void);

/* Backward of the above from the saved probs.  dq, dkv, dkvm are fully
   overwritten; dw_r (dk, d_pos, H) and db_r (K, H) are overwritten with the
   sums over streams, reduced in a fixed order (no atomics).  scratch needs
   nchip_relpos_attn_bwd_scratch() floats.  Returns 0, a negative error, or 1
   when keep_partials was set and the single-kernel path ran: then dw_r / db_r
   are NOT written and the per-stream partials stay in scratch for the caller
   to sum over the B rows: the dw_r partial of stream b at scratch[b*n_w + i]
   (n_w = dk*d_pos*H), the db_r partial at scratch[B*n_w + b*n_b + i]
   (n_b = K*H). */
size_t nchip_relpos_attn_bwd_scratch(int H, int dk, int B, int T, int M, int d_pos);
int nchip_relpos_attn_bwd(void *stream, const float *q, int64_t ldq,
                          const float *kv, const float *kvm, int64_t ldkv,
                          const float *w_r, const float *probs,
                          const float *dout, int64_t ldo,
                          float *dq, float *dkv, float *dkvm, float *dw_r, float *db_r,
                          int H, int dk, int dv, int B, int T, int M, int d_pos,
                          int attn_len, float b_r_scale, int precision, float *scratch,
                          int keep_partials);

/* The same attention on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16, fp32 accumulation,
   fp32 scores and softmax): every operand is the bf16 copy (nearest even) of the fp32 tensor
   of nchip_relpos_attn_fwd / _bwd, in the same layout with the same leading dimensions;
   probs16 is (K, T, H, B) bf16, written by the forward with the very values it multiplied
   with V and read by the backward; out16 / dq16 / dkv16 / dkvm16 (each may be NULL) receive
   bf16 copies of the fp32 results.  d_head 64 (keys and values), T <= 64, K = M + T <= 256 and
   a multiple of 8, d_pos <= K, leading dimensions multiples of 8: returns 1 (nothing
   launched) for anything else, 0 when launched, negative on error.  The backward writes
   per-stream dw_r / db_r partials to scratch (nchip_relpos_attn_bwd_scratch floats) and sums
   them over the streams in stream order.  No counterpart in the reference. */
int nchip_relpos_attn_fwd_bf16(void *stream, const uint16_t *q16, int64_t ldq, const uint16_t *kv16,
                               const uint16_t *kvm16, int64_t ldkv, const uint16_t *w_r16, const float *b_r,
                               float *out, uint16_t *out16, int64_t ldo, uint16_t *probs16, int H, int dk,
                               int dv, int B, int T, int M, int d_pos, int attn_len, float b_r_scale);
int nchip_relpos_attn_bwd_bf16(void *stream, const uint16_t *q16, int64_t ldq, const uint16_t *kv16,
                               const uint16_t *kvm16, int64_t ldkv, const uint16_t *w_r16,
                               const uint16_t *probs16, const uint16_t *dout16, int64_t ldo,
                               float *dq, uint16_t *dq16, float *dkv, uint16_t *dkv16, float *dkvm,
                               uint16_t *dkvm16, float *dw_r, float *db_r, int H, int dk, int dv, int B,
                               int T, int M, int d_pos, int attn_len, float b_r_scale, float *scratch);

/* LayerNorm / RMSNorm over axis 0 of (d, n) with optional affine
   (nncp.c:279-288; libnc.h:389-395).  xhat (d, n) and rstd (n) are saved for
   the backward.  w/b may be NULL (then y == xhat may alias). */
int nchip_norm_fwd(void *stream, const float *x, const float *w, const float *b,
                   float *y, float *xhat, float *rstd, int d, int64_t n,
                   float eps, int avg);
/* nchip_norm_fwd that also leaves y rounded to bf16 (nearest even) in y16 (d, n), the operand
   copy the bf16 products read; y16 NULL = nchip_norm_fwd.  No counterpart in the reference. */
int nchip_norm_fwd_bf16copy(void *stream, const float *x, const float *w, const float *b,
                            float *y, float *xhat, float *rstd, int d, int64_t n,
                            float eps, int avg, uint16_t *y16);
/* dx (d,n) = gradient of the input, plus dx_add (d,n) when that is not NULL;
   dw, db (d) overwritten (may be NULL when w is NULL).  partial needs
   nchip_norm_bwd_partial_rows(n) * 2 * d floats. */
int nchip_norm_bwd_partial_rows(int64_t n);
/* Rows of `partial` actually written for (d, n): row r holds the dw partial at
   partial[(2r)*d + i] and the db partial at partial[(2r+1)*d + i].  With
   partial given and dw == db == NULL the sums over the rows are left to the
   caller (they can be batched over many calls). */
int nchip_norm_bwd_rows(int d, int64_t n);
int nchip_norm_bwd(void *stream, const float *g, const float *xhat, const float *rstd,
                   const float *w, float *dx, const float *dx_add, float *dw, float *db,
                   float *partial, int d, int64_t n, int avg);

/* nchip_norm_bwd that also leaves partial row sums of the dx it writes (the bias gradient of
   a linear layer whose output went straight into this norm): dx_partial holds
   nchip_norm_bwd_rows(d, n) rows of d floats, their sum in row order is the sum of dx over
   its n columns.  Only for the widths nchip_norm_bwd_has_dx_rowsum() names; NULL = plain
   nchip_norm_bwd. */
#ifdef __cplusplus
bool nchip_norm_bwd_has_dx_rowsum(int d);
#else
_Bool nchip_norm_bwd_has_dx_rowsum(int d);
#endif
int nchip_norm_bwd_rowsum(void *stream, const float *g, const float *xhat, const float *rstd,
                          const float *w, float *dx, const float *dx_add, float *dw, float *db,
                          float *partial, int d, int64_t n, int avg, float *dx_partial);

/* nchip_norm_bwd_rowsum that also leaves dx rounded to bf16 in dx16 (d, n); NULL = none. */
int nchip_norm_bwd_bf16copy(void *stream, const float *g, const float *xhat, const float *rstd,
                            const float *w, float *dx, const float *dx_add, float *dw, float *db,
                            float *partial, int d, int64_t n, int avg, float *dx_partial, uint16_t *dx16);

/* nchip_norm_bwd for callers that cannot allocate device memory (code under HIP graph
   capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
   reference.  Same arguments without `partial`: the partial dw / db rows go to a buffer the
   library itself holds in device memory, nchip_norm_bwd_static_capacity() floats (8 MiB)
   per GPU for the life of the process, and the call allocates nothing.  The rows it holds
   are the nchip_norm_bwd_rows(d, n) rows the kernels actually write (never more than the
   nchip_norm_bwd_partial_rows(n) that size a caller's buffer for nchip_norm_bwd): (d, n) must
   satisfy nchip_norm_bwd_rows(d, n) * 2 * d <= that capacity - true for every n when d is 128, 256,
   512 or 1024, and for d <= 32768 otherwise - else the call returns -3 with a message and
   launches nothing.  The stream must belong to the current device.  All calls on one GPU
   share the buffer: calls that may overlap there (different streams, different threads)
   race; calls on one stream are ordered and safe.  Results are bit-identical to
   nchip_norm_bwd. */
size_t nchip_norm_bwd_static_capacity(void);
int nchip_norm_bwd_static(void *stream, const float *g, const float *xhat, const float *rstd,
                          const float *w, float *dx, const float *dx_add, float *dw, float *db,
                          int d, int64_t n, int avg);

/* softmax over axis 0 of (v, n) and its backward dx = y*(g - sum(g*y))
   (libnc.h:382; nncp.c:796, 1008). */
int nchip_softmax_fwd(void *stream, const float *x, float *y, int v, int64_t n);
int nchip_softmax_bwd(void *stream, const float *y, const float *g, float *dx, int v, int64_t n);

/* y[c] = log p[idx[c], c]; fused gradient dlogits = g[c]*(onehot - p)
   (libnc.h:385-388; nncp.c:1170). */
int nchip_indexed_log(void *stream, const float *p, const int32_t *idx, float *y, int v, int64_t n);
/* nchip_indexed_log and nchip_get_col index a table with the caller's data.  An index outside
   [0, v) reads nothing - the result is 0 - and raises a flag in pinned host memory.
   nchip_index_error() returns that flag and clears it; it is meaningful after a wait for the
   stream the kernels ran on (nc_synchronize and every other wait of the tensor library check
   it and end the process with a message, as libnc does on misuse). */
int nchip_index_error(void);
int nchip_nll_bwd(void *stream, const float *p, const int32_t *idx, const float *g,
                  float *dlogits, int v, int64_t n, int fused);

/* embedding gather y[:, c] = w[:, idx[c]] and its deterministic scatter-add
   backward (libnc.h:374-377; nncp.c:625): dw (d, v) overwritten; columns that
   share an index are summed in increasing c. */
int nchip_get_col(void *stream, const float *w, const int32_t *idx, float *y, int d, int v, int64_t n);
/* the same gather times a scale (nncp.c:625-630: the embedding and its multiplier in one
   launch; one rounding per element, as the separate product has) */
int nchip_get_col_scaled(void *stream, const float *w, const int32_t *idx, float *y, int d, int v, int64_t n, float scale);
int nchip_add_col(void *stream, const float *g, const int32_t *idx, float *dw, int d, int v, int64_t n);

/* fused optimiser step over one parameter (libnc.h:540-572 semantics as
   defined in nc_api.h): algo 0 SGD, 1 Adam (bias corrections c1, c2 passed
   in), 16 RMSProp. */
int nchip_opt_update(void *stream, int algo, float *w, float *m, float *v, const float *g,
                     int64_t n, float lr, float beta1, float beta2, float eps, float clip,
                     float c1, float c2);

/* The same update for many parameter tensors in ONE launch (the optimiser is
   pure bandwidth: 16 B per parameter for RMSProp).  dev_table[n_tensors] and
   dev_chunk_prefix[n_tensors + 1] live in device memory; tensor i owns the
   workgroups chunk_prefix[i] .. chunk_prefix[i+1]-1, each covering `chunk`
   consecutive elements.  m may be NULL (beta1 == 0), v may be NULL (SGD).  w16, when not
   NULL, receives the updated w rounded to bf16 (nearest even), element for element: the
   operand copy the bf16 products read, so that no weight is cast again after its update.
   wide, when not NULL, receives that rounded value widened to f32 again (parameters stored
   as bf16: w is their fp32 master, w16 the parameter itself, wide the copy that kernels
   reading f32 use). */
typedef struct {
    float *w, *m, *v;
    const float *g;
    int64_t n;
    float lr;
    int pad_;
    uint16_t *w16;
    float *wide;
} NchipOptTensor;
int nchip_opt_update_multi(void *stream, int algo, const NchipOptTensor *dev_table,
                           const int *dev_chunk_prefix, int n_tensors, int total_chunks, int chunk,
                           float beta1, float beta2, float eps, float clip, float c1, float c2);

/* dst[i] = src[i] rounded to bf16 (nearest even), i < n: one streaming pass. */
int nchip_cast_bf16(void *stream, const float *src, uint16_t *dst, int64_t n);
/* dst[i] = the f32 value of bf16 src[i] (exact), i < n. */
int nchip_widen_bf16(void *stream, const uint16_t *src, float *dst, int64_t n);

/* logits (v, n) f32 -> cdf (v, n) u16 as specified in nc_ext.h
   (nc_soft_max_cdf16); bit-identical to the CPU checker. */
int nchip_softmax_cdf16(void *stream, const float *logits, uint16_t *cdf, int v, int64_t n);
/* Integer probabilities per column (nc_soft_max_int, libnc.h:383-384): out[i] =
   max(floor(q[i] * mult / sum q), 1) as int32, q the 24-bit integer exponentials of the CDF
   above; 0 <= mult <= 2^32; bit-identical to the CPU checker. */
int nchip_softmax_int(void *stream, const float *logits, int32_t *out, int v, int64_t n, float mult);
/* path[l, c], l < levels: the entries of column c of cdf (v, n) that nncp_write_sym_cdf reads
   when it codes sym[c] - cdf[start + (len >> 1)] at each level of the balanced tree over [0, v)
   (cp_utils.c:299-323), 0 below the leaf.  levels >= ceil(log2 v).  No index leaves the column
   whatever sym[c] holds. */
int nchip_cdf_path(void *stream, const uint16_t *cdf, const int32_t *sym, uint16_t *path,
                   int v, int64_t n, int levels);
/* nchip_cdf_path of the table nchip_softmax_cdf16 would write, without the table: one read of the
   logits, `levels` entries per column out (ceil(log2 v) <= levels <= 16).  Same values. */
int nchip_softmax_cdf16_path(void *stream, const float *logits, const int32_t *sym, uint16_t *path,
                             int v, int64_t n, int levels);
/* sym[i, c] = largest s with cdf[s, c] <= target[i, c]; targets (m, n). */
int nchip_cdf_lookup(void *stream, const uint16_t *cdf, const uint16_t *target,
                     uint16_t *sym, int v, int64_t m, int64_t n);

#ifdef __cplusplus
}
#endif
#endif /* NCHIP_KERNELS_H */
