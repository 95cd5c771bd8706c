// Launchers of the small data-movement / element-wise kernels used by the
// libnc front end (k_elementwise.hip).  All enqueue on `st` and return nothing;
// argument checking is done by the callers in nc_ops.cpp.
#ifndef K_INTERNAL_H
#define K_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#define K_MAX_DIMS 8

// n-d descriptor: iterate over dims[], reading with stride sa/sb (0 = broadcast)
struct NdDesc {
    int nd;
    int64_t dims[K_MAX_DIMS];
    int64_t sa[K_MAX_DIMS];
    int64_t sb[K_MAX_DIMS];
};

enum KBinOp { KB_ADD = 0, KB_MUL = 1 };
enum KUnOp { KU_SIGMOID = 0, KU_TANH, KU_RELU, KU_GELU };

extern "C" {
// dst (strides d.sb) = src (strides d.sa); esize in {1,2,4}
void k_copy_nd(hipStream_t st, const void *src, void *dst, const NdDesc *d, int esize);
// i32/i8/u16 -> f32 style conversions are not needed on the device path
void k_fill_f32(hipStream_t st, float *p, float v, int64_t n);
// dst[i*k + kk] = src[kk*m + i]: the k-major copy of an m x k matrix stored with rows contiguous
void k_transpose_f32(hipStream_t st, const float *src, float *dst, int m, int k);
void k_fill_bytes(hipStream_t st, void *p, int v, int64_t nbytes);
// y[i] = a[i] op b[i % nb]   (b's shape is a prefix of a's)
void k_binary_prefix(hipStream_t st, int op, const float *a, const float *b, float *y,
                     int64_t n, int64_t nb);
// general broadcast: y contiguous over d.dims, a strides d.sa, b strides d.sb
void k_binary_nd(hipStream_t st, int op, const float *a, const float *b, float *y,
                 const NdDesc *d, int64_t n);
// y = mask[i % nm] (xor inv) ? c : x ;  backward: (mask ? 0 : g)
void k_masked_fill(hipStream_t st, const float *x, const int8_t *mask, float *y,
                   int64_t n, int64_t nm, float c, int inv);
void k_unary_fwd(hipStream_t st, int op, const float *x, float *y, int64_t n);
void k_unary_bwd(hipStream_t st, int op, const float *x, const float *g, float *dx, int64_t n);
// gated_swish: y = g*x*sigmoid(beta x); bwd writes dg, dx
void k_gated_swish_fwd(hipStream_t st, const float *g, const float *x, float *y, int64_t n, float beta);
void k_gated_swish_bwd(hipStream_t st, const float *g, const float *x, const float *gy,
                       float *dg, float *dx, int64_t n, float beta);
void k_lerp_fwd(hipStream_t st, const float *a, const float *b, const float *t, float *y, int64_t n);
void k_lerp_bwd(hipStream_t st, const float *a, const float *b, const float *t, const float *g,
                float *da, float *db, float *dt, int64_t n);
void k_lstm_clamped_fwd(hipStream_t st, const float *cp, const float *in, const float *fg,
                        const float *ig, float *y, int64_t n);
void k_lstm_clamped_bwd(hipStream_t st, const float *cp, const float *in, const float *fg,
                        const float *ig, const float *g, float *dcp, float *din, float *dfg,
                        float *dig, int64_t n);
// y = a * b * ... helpers for backward of mul: t = g * other[i % nb]
// (k_binary_prefix with KB_MUL covers it)

// out[i] = sum_o x[i + o*inner], o < outer, fixed order; tmp: nsplit*inner floats
int k_reduce_trailing_nsplit(int64_t inner, int64_t outer);
void k_reduce_trailing(hipStream_t st, const float *x, const float *y0, float *out, float *tmp,
                       int64_t inner, int64_t outer);
// stage 1 only: tmp[s][i] for s < k_reduce_trailing_nsplit(inner, outer); returns that count
int k_reduce_trailing_partials(hipStream_t st, const float *x, float *tmp, int64_t inner, int64_t outer);
// many row sums in one launch: dst[i] = sum_{r < rows} src[r*stride + i], i < n,
// per table entry (table in device memory); 4 interleaved row groups per
// element, sequential inside a group, combined in group order
struct KReduceRowsEntry {
    const float *src;
    float *dst;
    int64_t stride;
    int rows, n;
};
void k_reduce_rows_multi(hipStream_t st, const KReduceRowsEntry *dev_table, int n_entries, int max_n);
// out[0] = sum of all n elements (fixed tree); tmp: 1024 floats
void k_reduce_all(hipStream_t st, const float *x, float *out, float *tmp, int64_t n);
// general un-broadcast: out (numel nout, dims d.dims with strides d.sb over the
// REDUCED iteration) -- slow fallback, one thread per output element
void k_unbroadcast_nd(hipStream_t st, const float *g, float *out, const NdDesc *keep,
                      const NdDesc *red, int64_t nout, int64_t nred);
// y[j,i,o] = x[j - (pos + i*mult), i, o] or 0  (adjoint: + instead of -)
void k_rel_shift(hipStream_t st, const float *x, float *y, int64_t n0, int64_t n1,
                 int64_t outer, int64_t pos, int64_t mult, int adjoint);
// axis-0 pad/trim as in nc_pad; adjoint = backward (x gets the gradient)
void k_pad(hipStream_t st, const float *x, float *y, int64_t n_in, int64_t cols,
           int64_t left, int lop, int64_t right, int rop);
void k_pad_bwd(hipStream_t st, const float *gy, float *gx, int64_t n_in, int64_t cols,
               int64_t left, int lop, int64_t right, int rop);
}

// single-kernel rel-pos attention for heads that fit in LDS (k_attn_fused.hip)
struct FusedAttnFwdArgs {
    const float *q, *kv, *kvm, *w_r, *b_r;
    float *out, *probs;
    int64_t ldq, ldkv, ldo;
    int H, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
    int q_only; // >= 0: q and out are single (features, B) columns holding query position q_only
};
struct FusedAttnBwdArgs {
    const float *q, *kv, *kvm, *w_r, *probs, *dout;
    float *dq, *dkv, *dkvm, *dwp, *dbp; // dwp / dbp: per-stream partials in scratch
    int64_t ldq, ldkv, ldo;
    int H, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
};
bool k_attn_fused_shape_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr);
// the single-query (per-timestep) mode: heads of up to 128 keys only
bool k_attn_fused_step_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr);
int k_attn_fused_fwd(hipStream_t st, const FusedAttnFwdArgs &a, int dk);
// returns 0, -1 (path unavailable, nothing launched) or -2 (launch failed)
int k_attn_fused_bwd(hipStream_t st, const FusedAttnBwdArgs &a, int dk, float *dw_r, float *db_r,
                     int64_t n_w, int64_t n_b, int *launches, bool keep_partials);
// dw_r (n_w) and db_r (n_b) = sums over the B per-stream partials, in stream order (either may be NULL / 0)
int k_attn_param_grad_reduce(hipStream_t st, const float *dwp, float *dw, int64_t n_w,
                             const float *dbp, float *db, int64_t n_b, int B);

// k_attn_bf16.hip: the same attention on the bf16 matrix cores.  Operands are the bf16 copies
// of the fp32 tensors of FusedAttnFwdArgs / FusedAttnBwdArgs (same layouts, leading
// dimensions in elements); probs is (K, T, H, B) bf16; out16 / dq16 / dkv16 / dkvm16 (may be
// NULL) receive bf16 copies of the fp32 results, laid out like them.
struct Bf16AttnFwdArgs {
    const uint16_t *q, *kv, *kvm, *w_r;
    const float *b_r;
    float *out;
    uint16_t *out16, *probs;
    int64_t ldq, ldkv, ldo;
    int H, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
};
struct Bf16AttnBwdArgs {
    const uint16_t *q, *kv, *kvm, *w_r, *probs, *dout;
    float *dq, *dkv, *dkvm, *dwp, *dbp; // dwp / dbp: per-stream partials in scratch
    uint16_t *dq16, *dkv16, *dkvm16;
    int64_t ldq, ldkv, ldo;
    int H, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
};
bool k_attn_bf16_shape_ok(int dk, int dv, int T, int K, int d_pos, bool has_wr);
int k_attn_bf16_fwd(hipStream_t st, const Bf16AttnFwdArgs &a); // 0 or -2 (launch failed)
int k_attn_bf16_bwd(hipStream_t st, const Bf16AttnBwdArgs &a);

#endif
