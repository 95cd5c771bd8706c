/*
 * CPU checker versions of the fused entry points of nc_ext.h (test
 * infrastructure only).  nc_relpos_attention is written directly from the
 * index formula of the score matrix (nncp.c:728-800), as plain scalar loops,
 * and is itself checked against the unfused op sequence of nncp.c and
 * against textbook attention in tests/test_oracle_attention.py.
 */
#include "nc_ref_internal.h"

/* every op takes its operands through nc_operand (nc_ref_ops.c): contiguous, bf16 widened */
NCTensor *nc_operand(NCTensor *x);
#define nc_contig(x) nc_operand(x)

typedef struct {
    int H, dk, dv, B, T, M, K, d_pos, attn_len;
    float b_r_scale, scale;
    const float *q, *kv, *kvm, *w_r, *b_r;
    size_t ldq, ldkv;
} AttnDesc;

static inline const float *key_ptr(const AttnDesc *a, int b, int h, int j)
{
    if (j < a->M)
        return a->kvm + (size_t)a->ldkv * (b + (size_t)a->B * j) + h * a->dk;
    return a->kv + (size_t)a->ldkv * (b + (size_t)a->B * (j - a->M)) + h * a->dk;
}

static inline const float *val_ptr(const AttnDesc *a, int b, int h, int j)
{
    return key_ptr(a, b, 0, j) + a->H * a->dk + h * a->dv;
}

/* attention probabilities of one (b,h,i) column into A[0..K) */
static void attn_column(const AttnDesc *a, int b, int h, int i, float *A)
{
    const float *q = a->q + a->ldq * (b + (size_t)a->B * i) + h * a->dk;
    float mx = -INFINITY, s = 0;
    for (int j = 0; j < a->K; j++) {
        int delta = i + a->M - j;
        if (delta < 0 || delta >= a->attn_len) {
            A[j] = -INFINITY;
            continue;
        }
        const float *k = key_ptr(a, b, h, j);
        float acc = 0;
        for (int d = 0; d < a->dk; d++)
            acc += k[d] * q[d];
        if (a->w_r) {
            int p = a->d_pos - 1 - delta;
            const float *w = a->w_r + ((size_t)h * a->d_pos + (p > 0 ? p : 0)) * a->dk;
            float r = 0;
            for (int d = 0; d < a->dk; d++)
                r += w[d] * q[d];
            acc += r;
        }
        if (a->b_r)
            acc += a->b_r_scale * a->b_r[(size_t)h * a->K + (a->K - 1 - delta)];
        A[j] = acc * a->scale;
        mx = A[j] > mx ? A[j] : mx;
    }
    for (int j = 0; j < a->K; j++) {
        A[j] = (A[j] == -INFINITY) ? 0.0f : expf(A[j] - mx);
        s += A[j];
    }
    for (int j = 0; j < a->K; j++)
        A[j] /= s;
}

static void attn_desc(AttnDesc *a, const NCTensor *q, const NCTensor *kv, const NCTensor *kvm,
                      const NCTensor *w_r, const NCTensor *b_r, int n_head, int d_key,
                      int attn_len, float b_r_scale)
{
    memset(a, 0, sizeof(*a));
    if (q->n_dims != 3 || kv->n_dims != 3)
        nc_fatal("relpos_attention: q and kv must be (features, B, T)");
    a->H = n_head; a->dk = d_key;
    a->B = (int)q->dims[1]; a->T = (int)q->dims[2];
    a->M = kvm ? (int)kvm->dims[2] : 0;
    a->K = a->M + a->T;
    if ((int)q->dims[0] != n_head * d_key || kv->dims[1] != q->dims[1] || kv->dims[2] != q->dims[2])
        nc_fatal("relpos_attention: q/kv shape mismatch");
    if (kv->dims[0] <= q->dims[0] || (kv->dims[0] - q->dims[0]) % n_head)
        nc_fatal("relpos_attention: kv must hold H*dk key rows then H*dv value rows");
    a->dv = (int)(kv->dims[0] - q->dims[0]) / n_head;
    if (kvm && (kvm->dims[0] != kv->dims[0] || kvm->dims[1] != kv->dims[1]))
        nc_fatal("relpos_attention: kv_mem shape mismatch");
    a->ldq = q->dims[0]; a->ldkv = kv->dims[0];
    a->q = nc_f32(q); a->kv = nc_f32(kv); a->kvm = kvm ? nc_f32(kvm) : NULL;
    if (w_r) {
        if (w_r->n_dims != 3 || (int)w_r->dims[0] != d_key || (int)w_r->dims[2] != n_head)
            nc_fatal("relpos_attention: w_r must be (dk, d_pos, H)");
        a->d_pos = (int)w_r->dims[1];
        if (a->d_pos > a->K)
            nc_fatal("relpos_attention: d_pos > K is not supported");
        a->w_r = nc_f32(w_r);
    }
    if (b_r) {
        if (b_r->n_dims != 2 || (int)b_r->dims[0] != a->K || (int)b_r->dims[1] != n_head)
            nc_fatal("relpos_attention: b_r must be (K, H)");
        a->b_r = nc_f32(b_r);
    }
    a->attn_len = attn_len;
    a->b_r_scale = b_r_scale;
    a->scale = 1.0f / sqrtf((float)d_key);
}

NCTensor *nc_relpos_attention(NCTensor *q, NCTensor *kv, NCTensor *kv_mem,
                              NCTensor *w_r, NCTensor *b_r, int n_head,
                              int d_key, int attn_len, float b_r_scale)
{
    AttnDesc a;
    NCTensor *y, *args[5];
    NCNode *n;
    size_t dims[3];
    q = nc_contig(q); kv = nc_contig(kv);
    if (kv_mem) kv_mem = nc_contig(kv_mem);
    if (w_r) w_r = nc_contig(w_r);
    if (b_r) b_r = nc_contig(b_r);
    attn_desc(&a, q, kv, kv_mem, w_r, b_r, n_head, d_key, attn_len, b_r_scale);
    dims[0] = (size_t)a.H * a.dv; dims[1] = a.B; dims[2] = a.T;
    y = nc_alloc(q->dev, NC_TYPE_F32, 3, dims, 0);
    #pragma omp parallel for collapse(2)
    for (int b = 0; b < a.B; b++)
        for (int h = 0; h < a.H; h++) {
            float *A = nc_malloc(sizeof(float) * a.K);
            for (int i = 0; i < a.T; i++) {
                float *o = nc_f32(y) + dims[0] * (b + (size_t)a.B * i) + h * a.dv;
                attn_column(&a, b, h, i, A);
                for (int d = 0; d < a.dv; d++)
                    o[d] = 0;
                for (int j = 0; j < a.K; j++) {
                    const float *v = val_ptr(&a, b, h, j);
                    for (int d = 0; d < a.dv; d++)
                        o[d] += v[d] * A[j];
                }
            }
            free(A);
        }
    args[0] = q; args[1] = kv; args[2] = kv_mem; args[3] = w_r;
    /* b_r is the 5th argument; nodes carry shape info for 4, which is all the
       backward needs here because it allocates from the saved tensors */
    {
        NCTensor *all[5] = { q, kv, kv_mem, w_r, b_r };
        n = nc_new_node(q->dev->ctx, OP_RELPOS_ATTN, 5, all);
        for (int i = 0; i < 5; i++)
            if (all[i])
                n->saved[i] = nc_view(all[i]);
        n->ia[0] = n_head; n->ia[1] = d_key; n->ia[2] = attn_len;
        n->fa[0] = b_r_scale;
        if (nc_needs_grad(all, 5)) nc_attach(y, n); else nc_free_node(n);
    }
    nc_free_tensor(q); nc_free_tensor(kv); nc_free_tensor(kv_mem);
    nc_free_tensor(w_r); nc_free_tensor(b_r);
    return y;
}

/* one query position: the whole-segment routine on a query tensor that holds
   the query in column t, then that column of the result (see nc_ext.h) */
/* nc_ext.h: the decoder's two projections of a timestep, stated with the plain ops: the first
   result is nc_matmul + bias, the second goes into slice `index` of dst. */
NCTensor *nc_linear_pair_into(NCTensor *w0, NCTensor *bias0, NCTensor *w1, NCTensor *x,
                              NCTensor *dst, int index)
{
    NCTensor *y0, *y1;
    if (dst->n_dims != 3 || index < 0 || (size_t)index >= dst->dims[2])
        nc_fatal("nc_linear_pair_into: dst must be (m1, n, T) and 0 <= index < T");
    y0 = nc_matmul(w0, nc_dup_tensor(x));
    if (bias0)
        y0 = nc_add(y0, bias0);
    y1 = nc_matmul(w1, x);
    y1 = nc_reshape_3d(y1, y1->dims[0], y1->dims[1], 1);
    nc_tensor_copy_slice(dst, y1, 2, index, index + 1, 0);
    nc_free_tensor(y1);
    return y0;
}

/* nc_ext.h: forms of nc_soft_max_cdf16 / nc_get_col that spare the GPU library a copy; every
   tensor of this library is on the host already */
NCTensor *nc_soft_max_cdf16_to_host(NCTensor *logits)
{
    return nc_soft_max_cdf16(logits);
}

NCTensor *nc_get_col_host_indices(NCTensor *w, NCTensor *x, float scale)
{
    NCTensor *y = nc_get_col(w, x);
    return nc_mul(y, nc_new_f32(y->dev, scale));
}

/* nc_ext.h: a layout hint for the GPU library's few-column products; nothing to do here */
void nc_keep_k_major_weight(NCTensor *w)
{
    (void)w;
}

void nc_forget_k_major_weights(NCContext *m)
{
    (void)m;
}

/* nc_ext.h: the norm that ends one block together with the first product(s) of the next,
   stated with the plain ops */
NCTensor *nc_norm_linear_pair_into(NCTensor *x, NCTensor *g, NCTensor *b, float eps, BOOL avg_flag,
                                   NCTensor *w0, NCTensor *bias0, int act0,
                                   NCTensor *w1, NCTensor *dst, int index, NCTensor **pnormed)
{
    NCTensor *normed, *y0;
    if ((w1 == NULL) != (dst == NULL))
        nc_fatal("nc_norm_linear_pair_into: w1 and dst go together");
    normed = nc_fused_layer_norm(x, g, b, eps, avg_flag);
    if (w1) {
        if (act0 != NC_ACT_NONE)
            nc_fatal("nc_norm_linear_pair_into: no activation on the first product of a pair");
        y0 = nc_linear_pair_into(w0, bias0, w1, nc_dup_tensor(normed), dst, index);
    } else {
        y0 = nc_linear(w0, nc_dup_tensor(normed), bias0, act0);
    }
    if (pnormed)
        *pnormed = normed;
    else
        nc_free_tensor(normed);
    return y0;
}

NCTensor *nc_relpos_attention_step(NCTensor *q, NCTensor *kv_cache, NCTensor *kv_mem,
                                   NCTensor *w_r, NCTensor *b_r, int n_head, int d_key,
                                   int attn_len, float b_r_scale, int t)
{
    size_t dims[3], B, T;
    NCTensor *qf, *y;
    q = nc_contig(q);
    if (q->n_dims != 2 || kv_cache->n_dims != 3)
        nc_fatal("relpos_attention_step: q (H*dk, B) and kv_cache (.., B, T) expected");
    B = kv_cache->dims[1]; T = kv_cache->dims[2];
    if (q->dims[1] != B || t < 0 || (size_t)t >= T)
        nc_fatal("relpos_attention_step: stream count or position out of range");
    dims[0] = q->dims[0]; dims[1] = B; dims[2] = T;
    qf = nc_alloc(q->dev, NC_TYPE_F32, 3, dims, 1);
    memcpy(nc_f32(qf) + (size_t)t * dims[0] * B, nc_f32(q), sizeof(float) * dims[0] * B);
    nc_free_tensor(q);
    y = nc_relpos_attention(qf, kv_cache, kv_mem, w_r, b_r, n_head, d_key, attn_len, b_r_scale);
    y = nc_contig(nc_slice(y, 2, t, t + 1));
    return nc_reshape_2d(y, y->dims[0], B);
}


/* gradients exactly as the chain rule gives them for the formula above:
   dA[j] = v_j.do ; dS[j] = A[j](dA[j] - sum_j A dA) * scale ;
   dq += (k_j + w_r[pi]) dS[j] ; dk_j += q dS[j] ; dw_r[pi] += q dS[j] ;
   db_r[K-1-delta] += b_r_scale dS[j] ; dv_j += do A[j].                     */
void nc_relpos_attention_bw(NCNode *nd, NCTensor *g, NCTensor **ga)
{
    AttnDesc a;
    NCTensor *q = nd->saved[0], *kv = nd->saved[1], *kvm = nd->saved[2];
    NCTensor *w_r = nd->saved[3], *b_r = nd->saved[4];
    NCTensor *dq, *dkv, *dkvm = NULL, *dwr = NULL, *dbr = NULL;
    attn_desc(&a, q, kv, kvm, w_r, b_r, nd->ia[0], nd->ia[1], nd->ia[2], nd->fa[0]);
    g = nc_contig(nc_dup_tensor(g));
    dq = nc_alloc(q->dev, NC_TYPE_F32, 3, q->dims, 1);
    dkv = nc_alloc(q->dev, NC_TYPE_F32, 3, kv->dims, 1);
    if (kvm) dkvm = nc_alloc(q->dev, NC_TYPE_F32, 3, kvm->dims, 1);
    if (w_r) dwr = nc_alloc(q->dev, NC_TYPE_F32, 3, w_r->dims, 1);
    if (b_r) dbr = nc_alloc(q->dev, NC_TYPE_F32, 2, b_r->dims, 1);
    float *A = nc_malloc(sizeof(float) * a.K), *dS = nc_malloc(sizeof(float) * a.K);
    size_t ldo = (size_t)a.H * a.dv;
    for (int b = 0; b < a.B; b++)
        for (int h = 0; h < a.H; h++)
            for (int i = 0; i < a.T; i++) {
                const float *go = nc_f32(g) + ldo * (b + (size_t)a.B * i) + h * a.dv;
                const float *qv = a.q + a.ldq * (b + (size_t)a.B * i) + h * a.dk;
                float *dqv = nc_f32(dq) + a.ldq * (b + (size_t)a.B * i) + h * a.dk;
                float dot = 0;
                attn_column(&a, b, h, i, A);
                for (int j = 0; j < a.K; j++) {
                    const float *v = val_ptr(&a, b, h, j);
                    float da = 0;
                    for (int d = 0; d < a.dv; d++)
                        da += v[d] * go[d];
                    dS[j] = da;
                    dot += A[j] * da;
                }
                for (int j = 0; j < a.K; j++) {
                    int delta = i + a.M - j;
                    float ds = A[j] * (dS[j] - dot) * a.scale;
                    size_t col = (j < a.M) ? (b + (size_t)a.B * j) : (b + (size_t)a.B * (j - a.M));
                    float *dkvp = (j < a.M ? nc_f32(dkvm) : nc_f32(dkv)) + a.ldkv * col;
                    /* value gradient */
                    for (int d = 0; d < a.dv; d++)
                        dkvp[a.H * a.dk + h * a.dv + d] += go[d] * A[j];
                    if (delta < 0 || delta >= a.attn_len)
                        continue;
                    const float *k = key_ptr(&a, b, h, j);
                    for (int d = 0; d < a.dk; d++) {
                        dqv[d] += k[d] * ds;
                        dkvp[h * a.dk + d] += qv[d] * ds;
                    }
                    if (w_r) {
                        int p = a.d_pos - 1 - delta;
                        size_t off = ((size_t)h * a.d_pos + (p > 0 ? p : 0)) * a.dk;
                        for (int d = 0; d < a.dk; d++) {
                            dqv[d] += a.w_r[off + d] * ds;
                            nc_f32(dwr)[off + d] += qv[d] * ds;
                        }
                    }
                    if (b_r)
                        nc_f32(dbr)[(size_t)h * a.K + (a.K - 1 - delta)] += a.b_r_scale * ds;
                }
            }
    free(A); free(dS);
    nc_free_tensor(g);
    NCTensor *out[5] = { dq, dkv, dkvm, dwr, dbr };
    for (int i = 0; i < 5; i++) {
        if (out[i] && nd->parents[i]) ga[i] = out[i];
        else nc_free_tensor(out[i]);
    }
}

/* ---- integer CDF path ---------------------------------------------------- */

float nc_exp_det(float x)
{
    const float log2e = 0x1.715476p+0f;   /* 1.44269502 */
    const float ln2_hi = 0x1.63p-1f;      /* 0.693359375 */
    const float ln2_lo = -0x1.bd0106p-13f; /* -2.12194440e-4 */
    float n = rintf(x * log2e);
    float r = fmaf(-n, ln2_hi, x);
    r = fmaf(-n, ln2_lo, r);
    float p = 0x1.6c16c2p-10f;            /* 1/720 */
    p = fmaf(p, r, 0x1.111112p-7f);       /* 1/120 */
    p = fmaf(p, r, 0x1.555556p-5f);       /* 1/24 */
    p = fmaf(p, r, 0x1.555556p-3f);       /* 1/6 */
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    union { float f; uint32_t u; } v = { p };
    v.u += (uint32_t)((int32_t)n * (1 << 23));
    return v.f;
}

NCTensor *nc_soft_max_cdf16(NCTensor *logits)
{
    NCTensor *y;
    size_t V, cols;
    logits = nc_contig(logits);
    if (logits->type != NC_TYPE_F32 || logits->n_dims < 1)
        nc_fatal("soft_max_cdf16: f32 logits expected");
    V = logits->dims[0];
    if (V < 1 || V > 65535)
        nc_fatal("soft_max_cdf16: vocabulary size %zu outside [1, 65535]", V);
    cols = nc_numel(logits) / V;
    y = nc_alloc(logits->dev, NC_TYPE_U16, logits->n_dims, logits->dims, 0);
    uint32_t *qv = nc_malloc(sizeof(uint32_t) * V);
    for (size_t c = 0; c < cols; c++) {
        const float *x = nc_f32(logits) + c * V;
        uint16_t *cdf = (uint16_t *)y->buf->data + c * V;
        float mx = x[0];
        uint64_t tot = 0, run = 0;
        for (size_t i = 1; i < V; i++)
            mx = x[i] > mx ? x[i] : mx;
        for (size_t i = 0; i < V; i++) {
            float d = x[i] - mx;
            d = d < -30.0f ? -30.0f : d;
            qv[i] = (uint32_t)(nc_exp_det(d) * 16777216.0f);
            tot += qv[i];
        }
        for (size_t i = 0; i < V; i++) {
            cdf[i] = (uint16_t)(run * (65536 - V) / tot + i);
            run += qv[i];
        }
    }
    free(qv);
    nc_free_tensor(logits);
    return y;
}

/* libnc.h:383-384, "max(soft_max[i] * mult, 1) converted to int32".  Build-defined where the
   header is silent: the probabilities are the 24-bit integer exponentials of the CDF above over
   their exact sum, and the conversion is a floor; q * mult is exact in double and the division
   is one correctly rounded operation, so the GPU kernel computes the same integers. */
NCTensor *nc_soft_max_int(NCTensor *x, float mult)
{
    NCTensor *y;
    size_t V, cols;
    x = nc_contig(x);
    if (x->type != NC_TYPE_F32 || x->n_dims < 1)
        nc_fatal("soft_max_int: f32 input expected");
    if (!(mult >= 0.0f) || mult > 4294967296.0f)
        nc_fatal("soft_max_int: mult %g outside [0, 2^32]", (double)mult);
    V = x->dims[0];
    cols = nc_numel(x) / V;
    y = nc_alloc(x->dev, NC_TYPE_I32, x->n_dims, x->dims, 0);
    for (size_t c = 0; c < cols; c++) {
        const float *in = nc_f32(x) + c * V;
        int32_t *out = (int32_t *)y->buf->data + c * V;
        float mx = in[0];
        uint64_t tot = 0;
        for (size_t i = 1; i < V; i++)
            mx = in[i] > mx ? in[i] : mx;
        for (size_t i = 0; i < V; i++) {
            float d = in[i] - mx;
            d = d < -30.0f ? -30.0f : d;
            tot += (uint32_t)(nc_exp_det(d) * 16777216.0f);
        }
        for (size_t i = 0; i < V; i++) {
            float d = in[i] - mx;
            d = d < -30.0f ? -30.0f : d;
            double p = (double)(uint32_t)(nc_exp_det(d) * 16777216.0f) * (double)mult / (double)tot;
            out[i] = p >= 2147483647.0 ? 2147483647 : (p >= 1.0 ? (int32_t)p : 1);
        }
    }
    nc_free_tensor(x);
    return y;
}

/* nc_ext.h: the walk of nncp_write_sym_cdf (cp_utils.c:299-323 on integer counts), keeping what it reads */
NCTensor *nc_cdf_path(NCTensor *cdf, NCTensor *symbols)
{
    NCTensor *y;
    size_t V, cols, dims[2];
    int levels = 1;
    cdf = nc_contig(cdf); symbols = nc_contig(symbols);
    if (cdf->type != NC_TYPE_U16 || symbols->type != NC_TYPE_I32)
        nc_fatal("cdf_path: a u16 cdf and i32 symbols expected");
    V = cdf->dims[0];
    cols = V ? nc_numel(cdf) / V : 0;
    if (V == 0 || nc_numel(symbols) != cols)
        nc_fatal("cdf_path: one symbol per column of the cdf expected");
    while (((size_t)1 << levels) < V) levels++;
    dims[0] = (size_t)levels; dims[1] = cols;
    y = nc_alloc(cdf->dev, NC_TYPE_U16, 2, dims, 1);
    for (size_t c = 0; c < cols; c++) {
        const uint16_t *cp = (const uint16_t *)cdf->buf->data + cdf->off + c * V;
        uint16_t *yp = (uint16_t *)y->buf->data + c * (size_t)levels;
        long sym = ((const int32_t *)symbols->buf->data + symbols->off)[c];
        size_t start = 0, n = V;
        for (int l = 0; l < levels && n > 1; l++) {
            size_t n0 = n >> 1;
            yp[l] = cp[start + n0];
            if (sym >= (long)(start + n0)) { start += n0; n -= n0; }
            else n = n0;
        }
    }
    nc_free_tensor(cdf); nc_free_tensor(symbols);
    return y;
}

NCTensor *nc_soft_max_cdf16_path(NCTensor *logits, NCTensor *symbols) /* nc_ext.h: by its definition */
{
    return nc_cdf_path(nc_soft_max_cdf16(logits), symbols);
}

NCTensor *nc_soft_max_cdf16_path_to_host(NCTensor *logits, NCTensor *symbols) { return nc_soft_max_cdf16_path(logits, symbols); }
NCTensor *nc_tensor_to_cpu_device_queued(NCTensor *x) { return nc_tensor_to_cpu_device(x); }

NCTensor *nc_cdf_lookup(NCTensor *cdf, NCTensor *targets)
{
    NCTensor *y;
    size_t V, cols, m;
    cdf = nc_contig(cdf); targets = nc_contig(targets);
    if (cdf->type != NC_TYPE_U16 || targets->type != NC_TYPE_U16)
        nc_fatal("cdf_lookup: u16 tensors expected");
    V = cdf->dims[0];
    cols = nc_numel(cdf) / V;
    m = targets->dims[0];
    if (nc_numel(targets) != m * cols)
        nc_fatal("cdf_lookup: targets must be (m, n) for a (V, n) cdf");
    y = nc_alloc(cdf->dev, NC_TYPE_U16, targets->n_dims, targets->dims, 0);
    for (size_t c = 0; c < cols; c++) {
        const uint16_t *cp = (const uint16_t *)cdf->buf->data + cdf->off + c * V;
        const uint16_t *tp = (const uint16_t *)targets->buf->data + targets->off + c * m;
        uint16_t *yp = (uint16_t *)y->buf->data + c * m;
        for (size_t i = 0; i < m; i++) {
            size_t lo = 0, hi = V; /* invariant: cdf[lo] <= t < cdf[hi] (cdf[V] = 65536) */
            while (hi - lo > 1) {
                size_t mid = (lo + hi) >> 1;
                if (cp[mid] <= tp[i]) lo = mid; else hi = mid;
            }
            yp[i] = (uint16_t)lo;
        }
    }
    nc_free_tensor(cdf); nc_free_tensor(targets);
    return y;
}
