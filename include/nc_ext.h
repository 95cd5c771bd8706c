/*
 * nc_ext.h - additive entry points beside the libnc-compatible ABI of
 * nc_api.h.  The reference API already carries fused ops of this kind
 * (nc_fused_layer_norm libnc.h:394, nc_geglu libnc.h:254, nc_apply
 * libnc.h:634); these follow the same ownership rules (NCTensor* arguments are
 * consumed, the result is owned by the caller) and take part in nc_backward().
 * libnc_hip.so implements them as single fused HIP kernels; libnc_ref.so (the
 * CPU checker) implements them as direct scalar loops.
 */
#ifndef NC_EXT_H
#define NC_EXT_H

#include "nc_api.h"

#ifdef __cplusplus
extern "C" {
#endif

/* activations for nc_linear() */
#define NC_ACT_NONE 0
#define NC_ACT_GELU 1 /* tanh form: 0.5x(1+tanh(0.7978845608(x+0.044715x^3))) */
#define NC_ACT_RELU 2

/* y = act(w * x + bias).  w (m,k), x (k,n), bias (m) or NULL -> (m,n).
   Replaces the nc_matmul + nc_add + nc_gelu triple of nncp.c:930-943 and
   the matmul + bias pairs at nncp.c:659-661, 970-972, 1002-1004. */
NCTensor *nc_linear(NCTensor *w, NCTensor *x, NCTensor *bias, int act);

/* y = act(w * x + bias) + res, res shaped like the result: the linear layer
   together with the residual connection that follows it (nncp.c:896, 979).
   Gradients flow to w, x, bias and res. */
NCTensor *nc_linear_add(NCTensor *w, NCTensor *x, NCTensor *bias, int act, NCTensor *res);

/* Relative-position causal attention over memory + current segment, all
   heads and streams in one call.  Replaces nncp.c:722-800 and the
   split_head/concat_head copies (nncp.c:554-579).
     q      (H*dk, B, T)            queries, head h owns rows h*dk..h*dk+dk-1
     kv     (H*dk + H*dv, B, T)     keys (first H*dk rows) and values, current
     kv_mem (H*dk + H*dv, B, M)     the same for the memory, or NULL (M = 0)
     w_r    (dk, d_pos, H) or NULL  relative-position vectors
     b_r    (K, H) or NULL          relative-position scalar bias, K = M+T
   With key j in [0,K), query i in [0,T), distance delta = i + M - j:
     S[j,i] = (k_j.q_i + w_r[:, max(d_pos-1-delta,0), h].q_i
               + b_r_scale * b_r[K-1-delta, h]) / sqrt(dk)
              for 0 <= delta < attn_len, else -inf
     out[:, i] = sum_j v_j softmax_j(S[:, i])
   Result (H*dv, B, T).  Gradients flow to q, kv, kv_mem, w_r and b_r. */
NCTensor *nc_relpos_attention(NCTensor *q, NCTensor *kv, NCTensor *kv_mem,
                              NCTensor *w_r, NCTensor *b_r, int n_head,
                              int d_key, int attn_len, float b_r_scale);

/* The two projections of one decoder timestep (nncp.c:801-812) in one launch: returns
   w0 x + bias0 (m0, n) and writes w1 x (m1, n) into slice `index` of the last axis of dst
   (m1, n, T), the key / value cache.  w0 (m0, k), w1 (m1, k), x (k, n); bias0 may be NULL.
   Consumes w0, bias0, w1 and x, not dst.  The values are those of nc_linear(w0, x, bias0)
   and nc_matmul(w1, x), bit for bit.  No gradient. */
NCTensor *nc_linear_pair_into(NCTensor *w0, NCTensor *bias0, NCTensor *w1, NCTensor *x,
                              NCTensor *dst, int index);

/* The layer norm (avg_flag 1) or RMS norm (0) of x (k, n) with gain g and bias b (both or
   neither), followed by y0 = act0(w0 norm(x) + bias0) and, when w1 and dst are given,
   w1 norm(x) written into slice `index` of the last axis of dst (m1, n, T) - one launch in
   width-invariant fp32 mode for k = 128, 256 or 512 and at most 64 columns (the decoder's
   timestep: the norm that ends one block rides on the first product of the next,
   nncp.c:896-987), the separate steps otherwise.  *pnormed, when pnormed is not NULL,
   receives norm(x) as a new tensor.  The values are those of nc_fused_layer_norm followed by
   nc_linear / nc_linear_pair_into, bit for bit.  Consumes x, g, b, w0, bias0 and w1, not
   dst.  With a pair act0 must be NC_ACT_NONE.  No gradient. */
NCTensor *nc_norm_linear_pair_into(NCTensor *x, NCTensor *g, NCTensor *b, float eps, BOOL avg_flag,
                                   NCTensor *w0, NCTensor *bias0, int act0,
                                   NCTensor *w1, NCTensor *dst, int index, NCTensor **pnormed);

/* Keeps a k-major copy of the weight matrix w (m, k) until nc_forget_k_major_weights: forward
   products with at most 64 columns in width-invariant fp32 mode whose left operand is w
   (nc_matmul, nc_matmul_add, nc_linear, nc_linear_add, nc_linear_pair_into,
   nc_norm_linear_pair_into) read the copy instead - the same arithmetic and the same bits;
   such a product is bound by the cache lines it brings in, one per k for a matrix stored with
   rows contiguous, a quarter of that for the copy.  The matrix is found by its address: w
   must neither be written nor freed while the copy is kept (the decoder keeps copies of its
   weights for the timesteps of a segment, between two training steps).  Does not consume w.
   No counterpart in the reference. */
void nc_keep_k_major_weight(NCTensor *w);
void nc_forget_k_major_weights(NCContext *m);

/* One query position of nc_relpos_attention: q (H*dk, B) is the query of
   position t, kv_cache (H*dk+H*dv, B, T) holds the keys / values of positions
   0..t of the current segment (later columns finite, e.g. zero), kv_mem, w_r,
   b_r as above.  Result (H*dv, B), bit-identical to column t of the
   whole-segment call once the segment is complete (the decoder's view of
   nncp.c:801-863).  No gradient. */
NCTensor *nc_relpos_attention_step(NCTensor *q, NCTensor *kv_cache, NCTensor *kv_mem,
                                   NCTensor *w_r, NCTensor *b_r, int n_head, int d_key,
                                   int attn_len, float b_r_scale, int t);

/* When non-zero, the forward products of nc_matmul / nc_matmul_add / nc_linear
   use one tile class and one reduction order whatever the number of columns,
   so evaluating a single token column reproduces, bit for bit, that column of a
   whole-segment evaluation (what a per-timestep decoder needs against a
   whole-segment encoder).  Returns the previous setting.  No effect in
   libnc_ref.so, whose products are column-independent by construction. */
int nc_set_matmul_width_invariant(NCContext *m, int enable);

/* Integer CDF for the arithmetic coder (anchor: nc_soft_max_int libnc.h:384).
   logits (V, n) f32 -> (V, n) NC_TYPE_U16 with, per column,
     cdf[0] = 0, cdf[i+1] - cdf[i] >= 1, implicit cdf[V] = 65536.
   Pure function of the logits, bit-identical between the two libraries:
     m = max_i x_i ;  e_i = nc_exp_det(max(x_i - m, -30)) ;
     q_i = (uint32)(e_i * 2^24) ;  Q_i = sum_{j<i} q_j (exact integers) ;
     cdf[i] = floor(Q_i * (65536 - V) / Q_V) + i.                          */
NCTensor *nc_soft_max_cdf16(NCTensor *logits);

/* nc_soft_max_cdf16 with the result on the host device, written there by the kernel itself
   (pinned memory): for a few columns - a decoder timestep - this saves the launch and the
   latency of a copy.  The contents are valid after the next nc_synchronize of the logits'
   device.  Same values.  No counterpart in the reference. */
NCTensor *nc_soft_max_cdf16_to_host(NCTensor *logits);

/* nc_get_col (libnc.h:374-375) with the contiguous i32 indices x on the host device, read
   by the kernel itself from pinned memory instead of being uploaded first (a decoder
   timestep's tokens), times `scale` (nncp.c:625-630: the embedding multiplier; the values are
   those of nc_mul(nc_get_col(w, x), scale)).  x must not change until the device has been
   synchronised.  Consumes w and x.  No gradient.  No counterpart in the reference. */
NCTensor *nc_get_col_host_indices(NCTensor *w, NCTensor *x, float scale);

/* cdf (V, n) U16, targets (m, n) U16 -> (m, n) U16 symbols: the largest s
   with cdf[s, col] <= target (cumulative-frequency search of a decoder). */
NCTensor *nc_cdf_lookup(NCTensor *cdf, NCTensor *targets);

/* cdf (V, n) U16, symbols: n contiguous I32 on the same device -> (L, n) U16, L = max(1,
   ceil(log2 V)): the entries of each column that nncp_write_sym_cdf reads when it codes that
   column's symbol (the split point of every level of its tree, 0 below the leaf), in the order
   it reads them - nncp_write_sym_cdf_path codes from them.  An encoder brings these L values
   per column to the host instead of the V of the column.  Consumes both.  No counterpart in
   the reference. */
NCTensor *nc_cdf_path(NCTensor *cdf, NCTensor *symbols);
/* nc_cdf_path(nc_soft_max_cdf16(logits), symbols) in one pass over the logits: the table itself is
   never written.  Same values.  Consumes both. */
NCTensor *nc_soft_max_cdf16_path(NCTensor *logits, NCTensor *symbols);
/* nc_soft_max_cdf16_path with the result on the host device, written there by the kernel itself
   (pinned memory), and nc_tensor_to_cpu_device without its wait: in both cases the contents are
   valid after the next nc_synchronize of the source's device.  An encoder queues everything it
   wants from an evaluation - these entries, the loss - and waits once.  No counterpart in the
   reference (libnc_ref.so: the plain forms). */
NCTensor *nc_soft_max_cdf16_path_to_host(NCTensor *logits, NCTensor *symbols);
NCTensor *nc_tensor_to_cpu_device_queued(NCTensor *x);

/* The deterministic exponential used by nc_soft_max_cdf16, for x <= 0:
   n = rint(x*log2e); r = x - n*ln2 (two fmaf steps); degree-6 polynomial in
   fmaf form; result scaled by 2^n through the exponent field.  Only IEEE
   single-precision operations that round identically on x86 and gfx950. */
float nc_exp_det(float x);

/* When non-zero, every nc_matmul / nc_linear on device tensors rounds both
   operands to bf16 (round-to-nearest-even) as it loads them and accumulates in
   fp32 on the bf16 MFMA units; parameters and activations stay fp32 in memory.
   Returns the previous setting.  libnc_ref.so emulates the same rounding. */
int nc_set_matmul_bf16(NCContext *m, int enable);

/* bf16 operand copies.  With nc_set_matmul_bf16 on, a product whose shape allows it reads
   both operands as bf16 from memory: every f32 device buffer can carry a bf16 copy of itself
   (same elements, rounded to nearest even), written by the kernel that produces the f32
   values where there is one (layer norms, the optimiser's weight update, product epilogues
   that feed another product) and by one cast pass otherwise, and dropped whenever the buffer
   is written in place.  nc_get_bf16_cast_count: how many copies were made by a cast of their
   own so far (the ones a producing kernel could still take over).  nc_set_bf16_shadow_check:
   testing aid, process-wide - when non-zero, every use of a copy first compares it with a
   fresh rounding of the buffer and ends the process if they differ (a writer that failed to
   drop the copy); returns the previous setting.  Both 0 / no effect in libnc_ref.so. */
int64_t nc_get_bf16_cast_count(NCContext *m);
int nc_set_bf16_shadow_check(int enable);
/* While non-zero (and nc_set_matmul_bf16 is on), the forward products nc_matmul / nc_matmul_add /
   nc_linear / nc_linear_add also leave the bf16 copy of their result: for results that go
   straight into another consumer of bf16 operands (the query and key / value projections in
   front of nc_relpos_attention), which then needs no cast of them.  Returns the previous
   setting.  No effect on values; no effect in libnc_ref.so. */
int nc_set_bf16_copy_of_results(NCContext *m, int enable);

/* When non-zero, nc_backward() postpones the weight-gradient GEMMs
   dW = dY X^T of plain linear layers (weight used once in the graph) and runs
   them all in one grouped launch just before it returns.  The gradient
   tensors passed to the NCParamUpdateFunc for those parameters then hold valid
   data only after nc_backward() has returned - fine for callbacks that just
   forward to sgd_opt_update_var (nncp.c:1078-1096).  Returns the previous
   setting.  No effect in libnc_ref.so. */
int nc_set_deferred_weight_grad(NCContext *m, int enable);

/* The optimiser's per-parameter state, for checkpoints and for tests that put two models
   into the same state: `which` 0 = first moment (Adam with beta1 != 0), 1 = second moment
   (Adam, RMSProp), 2 = the fp32 master values of a parameter stored as NC_TYPE_BF16 (the
   update works on them and leaves their rounding in the parameter; a caller that sets them
   sets the parameter to their rounding as well).  nc_sgd_opt_get_state returns a new 1-D f32 tensor on the host device
   holding a copy (NULL when the parameter has no optimiser or the algorithm keeps no such
   moment); nc_sgd_opt_set_state copies the values of v (f32, same element count, any device)
   into it.  nc_sgd_opt_get_step / nc_sgd_opt_set_step: the count of updates applied, which
   Adam's bias correction reads.  No counterpart in libnc.h (its optimiser state is opaque:
   libnc.h:561-571). */
NCTensor *nc_sgd_opt_get_state(NCParam *p, int which);
void nc_sgd_opt_set_state(NCParam *p, int which, const NCTensor *v);
int64_t nc_sgd_opt_get_step(NCSGDOptState *s);
void nc_sgd_opt_set_step(NCSGDOptState *s, int64_t step);

/* Number of kernel launches issued so far (0 in libnc_ref.so). */
int64_t nc_get_launch_count(NCContext *m);

/* The stream (a hipStream_t) on which this context enqueues all its device work, for callers
   that mix the raw kernel entry points of nchip_kernels.h with tensor calls: work they
   enqueue on it runs in order with the library's own, and nc_synchronize() waits for it.
   NULL before the device exists and in libnc_ref.so. */
void *nc_context_stream(NCContext *m);

#ifdef __cplusplus
}
#endif
#endif /* NC_EXT_H */
