/*
 * Transformer-XL model of NNCP on top of the libnc ABI: the `trf` model class
 * (nncp.c:263-1562) restated as a library.  Two evaluation paths issue
 * exactly the tensor ops the reference issues:
 *   - reference path (cfg.fused = 0): the op-by-op sequence of trf_eval,
 *     including the per-timestep (seq_eval) variant with its K/V caches and the
 *     graph surgery of trf_eval_gradient;
 *   - fused path (cfg.fused = 1): the same mathematics through nc_linear,
 *     nc_relpos_attention and nc_fused_layer_norm (full-segment evaluation).
 * Not supported (as in no BASELINE configuration): rotary position embedding,
 * dropout / retrain, tied input-output embedding, sparse gradients.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "model_internal.h"

static void die(const char *msg)
{
    fprintf(stderr, "nncp_host: %s\n", msg);
    abort();
}

void nncp_config_default(NNCPConfig *c) /* the "default" profile, nncp.c:2471-2513 */
{
    memset(c, 0, sizeof(*c));
    c->seed = 123;
    c->batch_size = 16; c->seg_len = 32; c->n_symbols = 256;
    c->n_layer = 4; c->d_model = 256; c->n_head = 8;
    c->d_key = c->d_value = c->d_model / c->n_head;
    c->d_inner = c->d_model * 2;
    c->d_pos = 32; c->mem_len = 32;
    for (int i = 0; i < c->n_layer; i++)
        c->attn_len[i] = c->mem_len + c->seg_len;
    c->init_range = 1.0f; c->embed_mult = 1.0f;
    c->use_bias = 1; c->use_w_r = 1; c->tied_w_r = 1; c->tied_b_r = 1;
    c->ln_flags = NNCP_LN_POST;
    c->ff_act = NNCP_FF_GELU;
    c->sgd_opt.algo = SGD_OPT_ADAM;
    c->sgd_opt.u.adam.beta1 = 0.0f; c->sgd_opt.u.adam.beta2 = 0.9999f;
    c->sgd_opt.u.adam.eps = 1e-8f; c->sgd_opt.u.adam.gradient_clip = 0.1f;
    c->sgd_opt.lr = 3e-4f;
    c->use_device = 1; c->fused = 0; c->nb_threads = 1;
}

static NCTensor *new_param(NNCPModel *s, NCTensor **slot, NCTensor *t, float init, const char *fmt, int idx)
{
    *slot = t;
    nc_new_param(&s->params, slot, fmt, idx);
    if (init > 0.0f)
        nc_tensor_set_rnd_unif(t, 0, init, s->rnd);
    return t;
}

static void new_layer_norm(NNCPModel *s, NCTensor **g, NCTensor **b, int idx) /* nncp.c:268-277 */
{
    new_param(s, g, nc_new_tensor_1d(s->dev, s->param_type, s->cfg.d_model), 0, "ln_g_%d", idx);
    nc_tensor_set_f32(*g, 1.0f);
    new_param(s, b, nc_new_tensor_1d(s->dev, s->param_type, s->cfg.d_model), 0, "ln_b_%d", idx);
}

NNCPModel *nncp_model_new(const NNCPConfig *cfg)
{
    NNCPModel *s = nc_mallocz(sizeof(*s));
    const NNCPConfig *c;
    s->cfg = *cfg;
    c = &s->cfg;
    if (c->model_type == NNCP_MODEL_LSTM) {
        /* nncp_init, nncp.c:2770-2779, then lstm_init */
        s->ctx = nc_context_init(c->nb_threads);
        s->cpu = nc_new_cpu_device(s->ctx);
        s->dev = c->use_device ? nc_new_cuda_device(s->ctx, 0) : s->cpu;
        s->rnd = nc_rnd_init(s->dev, c->seed);
        s->param_type = c->param_bf16 ? NC_TYPE_BF16 : NC_TYPE_F32; /* nncp.c:1727-1730 */
        if (c->param_bf16)
            nc_set_matmul_bf16(s->ctx, 1);
        s->cls = &nncp_lstm_class;
        lstm_init(s);
        return s;
    }
    s->cls = &nncp_trf_class;
    if (c->n_layer < 1 || c->n_layer > NNCP_N_LAYER_MAX || c->d_model != c->d_key * c->n_head)
        die("bad configuration (need d_model == d_key * n_head, 1 <= n_layer <= 32)");
    int T = c->seg_len, M = c->mem_len, K = T + M, B = c->batch_size, H = c->n_head, D = c->d_model;
    int gated = c->ff_act == NNCP_FF_GEGLU || c->ff_act == NNCP_FF_GATED_SILU;
    /* nncp_init, nncp.c:2770-2779 */
    s->ctx = nc_context_init(c->nb_threads);
    s->cpu = nc_new_cpu_device(s->ctx);
    s->dev = c->use_device ? nc_new_cuda_device(s->ctx, 0) : s->cpu;
    s->rnd = nc_rnd_init(s->dev, c->seed);
    s->param_type = c->param_bf16 ? NC_TYPE_BF16 : NC_TYPE_F32; /* nncp.c:343-346 */
    if (c->param_bf16)
        nc_set_matmul_bf16(s->ctx, 1);
    s->fused_now = c->fused;
    if (c->fused)
        nc_set_deferred_weight_grad(s->ctx, 1); /* backward_cb only forwards to sgd_opt_update_var */
    /* trf_init, nncp.c:304-520 */
    s->embed_mult = sqrtf((float)D) * c->embed_mult;
    nc_param_list_init(s->ctx, &s->params);
    float init = c->init_range / sqrtf((float)D);
    s->layers = nc_mallocz(sizeof(Layer) * c->n_layer);
    for (int l = 0; l < c->n_layer; l++) {
        Layer *tl = &s->layers[l];
        /* mask[j,i] = !(0 <= (i+M)-j < attn_len), nncp.c:352-365 */
        NCTensor *mask = nc_new_tensor_2d(s->cpu, NC_TYPE_I8, K, T);
        for (int i = 0; i < T; i++)
            for (int j = 0; j < K; j++) {
                int pos = i + M - j;
                nc_set1_i32_2d(mask, j, i, !(pos >= 0 && pos < c->attn_len[l]));
            }
        tl->attn_mask = nc_tensor_to_device(mask, s->dev);
        if (l == 0 || !c->tied_b_r)
            new_param(s, &tl->b_r, nc_new_tensor_2d(s->dev, s->param_type, K, H), 0, "b_r_%d", l);
        if (c->use_w_r && (l == 0 || !c->tied_w_r))
            new_param(s, &tl->w_r, nc_new_tensor_3d(s->dev, s->param_type, c->d_key, c->d_pos, H), init, "w_r_%d", l);
        new_param(s, &tl->w_q, nc_new_tensor_2d(s->dev, s->param_type, H * c->d_key, D), init, "w_q_%d", l);
        if (c->query_bias)
            new_param(s, &tl->b_q, nc_new_tensor_1d(s->dev, s->param_type, H * c->d_key), 0, "b_q_%d", l);
        new_param(s, &tl->w_kv, nc_new_tensor_2d(s->dev, s->param_type, H * c->d_key + H * c->d_value, D), init, "w_kv_%d", l);
        if (c->d_value != D)
            new_param(s, &tl->w_o, nc_new_tensor_2d(s->dev, s->param_type, D, H * c->d_value), init, "w_o_%d", l);
        int n1 = gated ? c->d_inner * 2 : c->d_inner;
        new_param(s, &tl->ff1, nc_new_tensor_2d(s->dev, s->param_type, n1, D), init, "ff1_%d", l);
        if (c->use_bias)
            new_param(s, &tl->ff_bias1, nc_new_tensor_1d(s->dev, s->param_type, n1), 0, "ff_bias1_%d", l);
        new_param(s, &tl->ff2, nc_new_tensor_2d(s->dev, s->param_type, D, c->d_inner),
                  init * sqrtf((float)D / (float)c->d_inner), "ff2_%d", l);
        if (c->use_bias)
            new_param(s, &tl->ff_bias2, nc_new_tensor_1d(s->dev, s->param_type, D), 0, "ff_bias2_%d", l);
        if (c->ln_flags & (NNCP_LN_POST | NNCP_LN_PRE)) {
            new_layer_norm(s, &tl->ln_g1, &tl->ln_b1, l * 2);
            new_layer_norm(s, &tl->ln_g2, &tl->ln_b2, l * 2 + 1);
        }
        if (c->ln_flags & NNCP_LN_COEF)
            new_param(s, &tl->alpha, nc_new_scalar(s->dev, s->param_type), 0, "alpha_%d", l);
        /* caches and node tables of the per-timestep path, nncp.c:439-452 */
        tl->mem_key = nc_new_tensor_4d(s->dev, NC_TYPE_F32, c->d_key, K, H, B);
        tl->mem_value = nc_new_tensor_4d(s->dev, NC_TYPE_F32, c->d_value, K, H, B);
        tl->key_nodes = nc_mallocz(sizeof(NCNode *) * (T + 1));
        tl->kq_nodes = nc_mallocz(sizeof(NCNode *) * T);
        tl->value_nodes = nc_mallocz(sizeof(NCNode *) * (T + 1));
        tl->va_nodes = nc_mallocz(sizeof(NCNode *) * T);
    }
    if (c->ln_flags & NNCP_LN_FINAL)
        new_layer_norm(s, &s->ln_g, &s->ln_b, c->n_layer * 2);
    new_param(s, &s->embed, nc_new_tensor_2d(s->dev, s->param_type, D, c->n_symbols), init, "embed", 0);
    new_param(s, &s->embed_out, nc_new_tensor_2d(s->dev, s->param_type, c->n_symbols, D), init, "embed_out", 0);
    if (c->use_bias)
        new_param(s, &s->out_bias, nc_new_tensor_1d(s->dev, s->param_type, c->n_symbols), 0, "out_bias", 0);
    s->mem_h = nc_mallocz(sizeof(NCTensor *) * c->n_layer);
    s->train_h = nc_mallocz(sizeof(NCTensor *) * c->n_layer);
    s->mem_store = nc_mallocz(sizeof(NCTensor *) * c->n_layer);
    s->mem_pos = nc_mallocz(sizeof(int) * c->n_layer);
    s->mem_cap = 0;
    if (c->use_device && M > T) {
        /* room for the window to move: up to 8 segments, at most 256 MiB, behind the memory */
        size_t seg_bytes = (size_t)D * B * T * sizeof(float);
        size_t slack = ((size_t)256 << 20) / seg_bytes;
        slack = slack < 1 ? 1 : (slack > 8 ? 8 : slack);
        const char *e = getenv("NNCP_MEM_SLACK_SEGMENTS"); /* tests: 1 makes the window start over at every other update */
        if (e && atoi(e) >= 1 && atoi(e) <= 64) slack = (size_t)atoi(e);
        s->mem_cap = M + (int)slack * T;
    }
    for (int l = 0; l < c->n_layer; l++) {
        if (s->mem_cap) {
            s->mem_store[l] = nc_new_tensor_3d(s->dev, NC_TYPE_F32, D, B, s->mem_cap);
            s->mem_h[l] = nc_slice_alias(s->mem_store[l], 2, 0, M);
        } else {
            s->mem_h[l] = nc_new_tensor_3d(s->dev, NC_TYPE_F32, D, B, M);
        }
        s->train_h[l] = nc_new_tensor_3d(s->dev, NC_TYPE_F32, D, B, T);
    }
    s->outputs = nc_mallocz(sizeof(NCTensor *) * T);
    s->opt = nc_sgd_opt_init(s->ctx, &c->sgd_opt);
    nc_sgd_opt_set_all(&s->params, s->opt);
    return s;
}

void nncp_model_free(NNCPModel *s) /* trf_end nncp.c:522-550, nncp_end nncp.c:2802-2809 */
{
    nc_free(s->retrain.buf);
    if (s->cfg.model_type == NNCP_MODEL_LSTM) {
        lstm_end(s);
        nc_rnd_end(s->rnd);
        nc_context_end(s->ctx);
        nc_free(s);
        return;
    }
    trf_eval_end(s);
    for (int l = 0; l < s->cfg.n_layer; l++) {
        Layer *tl = &s->layers[l];
        nc_free_tensor(s->mem_h[l]); nc_free_tensor(s->mem_store[l]); nc_free_tensor(s->train_h[l]);
        nc_free_tensor(tl->mem_key); nc_free_tensor(tl->mem_value); nc_free_tensor(tl->attn_mask);
        nc_free(tl->key_nodes); nc_free(tl->kq_nodes); nc_free(tl->value_nodes); nc_free(tl->va_nodes);
    }
    trf_step_end(s);
    nc_free(s->step_kv); nc_free(s->step_kvm);
    nc_free(s->mem_h); nc_free(s->mem_store); nc_free(s->mem_pos); nc_free(s->train_h); nc_free(s->outputs);
    nc_sgd_opt_set_all(&s->params, NULL);
    nc_sgd_opt_end(s->opt);
    nc_param_list_end(&s->params);
    nc_free(s->layers);
    nc_rnd_end(s->rnd);
    nc_context_end(s->ctx);
    nc_free(s);
}

const NNCPConfig *nncp_model_config(NNCPModel *s) { return &s->cfg; }
NCContext *nncp_model_context(NNCPModel *s) { return s->ctx; }
NCDevice *nncp_model_device(NNCPModel *s) { return s->dev; }
NCDevice *nncp_model_cpu_device(NNCPModel *s) { return s->cpu; }
int64_t nncp_model_train_step(NNCPModel *s) { return s->train_step; }

NCTensor **nncp_model_param(NNCPModel *s, const char *name)
{
    for (struct list_head *el = s->params.param_list.next; el != &s->params.param_list; el = el->next) {
        NCParam *p = (NCParam *)el;
        if (!strcmp(p->name, name))
            return p->pval;
    }
    return NULL;
}

int nncp_model_param_count(NNCPModel *s)
{
    int n = 0;
    for (struct list_head *el = s->params.param_list.next; el != &s->params.param_list; el = el->next)
        n++;
    return n;
}

const char *nncp_model_param_name(NNCPModel *s, int index)
{
    int n = 0;
    for (struct list_head *el = s->params.param_list.next; el != &s->params.param_list; el = el->next)
        if (n++ == index)
            return ((NCParam *)el)->name;
    return NULL;
}

static NCParam *find_param_entry(NNCPModel *s, const char *name)
{
    NCParam *p = nc_find_param(&s->params, name);
    if (!p)
        die("no parameter of that name");
    return p;
}

NCTensor *nncp_model_opt_state(NNCPModel *s, const char *name, int which)
{
    return nc_sgd_opt_get_state(find_param_entry(s, name), which);
}

void nncp_model_set_opt_state(NNCPModel *s, const char *name, int which, const NCTensor *v)
{
    nc_sgd_opt_set_state(find_param_entry(s, name), which, v);
}

NCTensor *nncp_model_memory(NNCPModel *s, int l)
{
    if (s->cfg.model_type == NNCP_MODEL_LSTM || s->cfg.mem_len <= 0 || l < 0 || l >= s->cfg.n_layer)
        return NULL;
    return s->mem_h[l];
}

/* parameter files: what --load_coefs names (nncp.c:3149, 3761; its use at nncp.c:3439-3442 and
   3604-3607 is compiled out in the reference, the calls are libnc.h:530, 536) */
void nncp_model_save_coefs(NNCPModel *s, const char *filename) { nc_save_coefs(&s->params, filename); }
void nncp_model_load_coefs(NNCPModel *s, const char *filename) { nc_load_coefs(&s->params, filename); }

/* ---- pieces shared by the evaluation paths ----------------------------------- */

static NCTensor *scalar(NNCPModel *s, float v) { return nc_new_f32(s->dev, v); }

/* nncp.c:290-298: a fresh mask of 0 / 1/(1-prob) from the model's random stream */
static NCTensor *dropout_mul(NNCPModel *s, NCTensor *x, float prob)
{
    NCTensor *mask;
    if (!s->dropout_enabled || prob == 0)
        return x;
    mask = nc_new_tensor_from_tensor_nz(x);
    nc_tensor_set_dropout(mask, prob, s->rnd);
    return nc_mul(x, mask);
}

static NCTensor *layer_norm(NNCPModel *s, NCTensor *x, NCTensor *g, NCTensor *b) /* nncp.c:279-288 */
{
    int rms = s->cfg.ln_flags & NNCP_LN_RMSNORM;
    if (s->cfg.fused)
        return nc_fused_layer_norm(x, nc_dup_tensor(g), nc_dup_tensor(b), 1e-5f, !rms);
    x = rms ? nc_rms_norm(x, 1e-5f) : nc_layer_norm(x, 1e-5f);
    return nc_add(nc_mul(x, nc_dup_tensor(g)), nc_dup_tensor(b));
}

static NCTensor *split_head(NCTensor *x, int n_head) /* nncp.c:554-565 */
{
    size_t d[NC_N_DIMS_MAX];
    nc_tensor_get_dims(x, d);
    x = nc_reshape_4d(x, d[0] / n_head, n_head, d[1], d[2]);
    return nc_permute_4d(x, 0, 3, 1, 2);
}

static NCTensor *concat_head(NCTensor *x) /* nncp.c:569-579 */
{
    size_t d[NC_N_DIMS_MAX];
    x = nc_permute_4d(x, 0, 2, 3, 1);
    nc_tensor_get_dims(x, d);
    return nc_reshape_2d(x, d[0] * d[1], d[2] * d[3]);
}

/* store layer input into train_h (whole segment or one timestep), nncp.c:647-657 */
static void save_layer_input(NNCPModel *s, int l, int output_index, NCTensor *x, int seg_len)
{
    if (s->fused_now && output_index < 0) {
        /* whole segment on the fused path: train_h keeps the layer input itself (a view
           of its storage outside the graph) instead of a copy of it */
        NCTensor *v = nc_slice_alias(x, 1, 0, (size_t)s->cfg.batch_size * seg_len);
        nc_free_tensor(s->train_h[l]);
        s->train_h[l] = nc_reshape_3d(v, s->cfg.d_model, s->cfg.batch_size, seg_len);
        return;
    }
    NCTensor *dst = output_index < 0 ? nc_dup_tensor(s->train_h[l])
                                     : nc_slice_alias(s->train_h[l], 2, output_index, output_index + 1);
    NCTensor *src = nc_reshape_3d(nc_dup_tensor(x), s->cfg.d_model, s->cfg.batch_size, seg_len);
    nc_tensor_copy(dst, src);
    nc_free_tensor(src);
    nc_free_tensor(dst);
}

/* position tensors of the reference path, built at the first timestep, nncp.c:728-761 */
static void build_position_tensors(NNCPModel *s, int l)
{
    const NNCPConfig *c = &s->cfg;
    Layer *tl = &s->layers[l];
    if (c->use_w_r) {
        if (l == 0 || !c->tied_w_r) {
            NCTensor *w = nc_dup_tensor(tl->w_r);
            w = c->batch_size > 1 ? nc_repeat_1d(w, c->batch_size)
                                  : nc_reshape_4d(w, c->d_key, c->d_pos, c->n_head, 1);
            tl->tmp_w_r = w;
        } else {
            tl->tmp_w_r = nc_dup_tensor(s->layers[0].tmp_w_r);
        }
    }
    if (l == 0 || !c->tied_b_r) {
        NCTensor *b = nc_mul(nc_dup_tensor(tl->b_r), scalar(s, sqrtf((float)(c->d_key * c->d_model))));
        b = nc_repeat_2d(b, c->seg_len, c->batch_size);
        tl->tmp_b_r = nc_permute_4d(b, 0, 2, 1, 3);
    } else {
        tl->tmp_b_r = nc_dup_tensor(s->layers[0].tmp_b_r);
    }
}

/* reference attention, whole segment: nncp.c:763-800 */
static NCTensor *attention_segment_ref(NNCPModel *s, int l, NCTensor *query, NCTensor *key, NCTensor *value)
{
    const NNCPConfig *c = &s->cfg;
    Layer *tl = &s->layers[l];
    NCTensor *t0 = nc_matmul_add(key, nc_dup_tensor(query), NULL, 1, 0, 1.0f), *rd;
    if (c->use_w_r) {
        rd = nc_matmul_add(nc_dup_tensor(tl->tmp_w_r), query, NULL, 1, 0, 1.0f);
        rd = nc_pad(rd, c->mem_len + c->seg_len - c->d_pos, NC_PAD_DUP, 0, NC_PAD_ZERO);
        rd = nc_add(rd, nc_dup_tensor(tl->tmp_b_r));
    } else {
        nc_free_tensor(query);
        rd = nc_dup_tensor(tl->tmp_b_r);
    }
    rd = nc_rel_shift(rd, -(c->seg_len - 1), 1);
    t0 = nc_add(rd, t0);
    t0 = nc_mul(t0, scalar(s, 1.0f / sqrtf((float)c->d_key)));
    t0 = nc_masked_fill(t0, nc_dup_tensor(tl->attn_mask), -INFINITY, 0);
    t0 = nc_soft_max(t0);
    t0 = dropout_mul(s, t0, c->dropout_att_prob); /* nncp.c:797-799 */
    return nc_matmul(value, t0);
}

/* reference attention, one timestep against the K/V caches: nncp.c:801-863 */
static NCTensor *attention_timestep_ref(NNCPModel *s, int l, int t, NCTensor *query, NCTensor *key, NCTensor *value)
{
    const NNCPConfig *c = &s->cfg;
    Layer *tl = &s->layers[l];
    int row = c->mem_len + t;
    NCTensor *slot, *t0, *t1, *rd;
    NCNode *node;

    tl->key_nodes[t + 1] = nc_dup_node(nc_get_node(key));
    slot = nc_slice_alias(tl->mem_key, 1, row, row + 1);
    nc_tensor_copy(slot, key);
    nc_free_tensor(key); nc_free_tensor(slot);
    key = nc_dup_tensor(tl->mem_key);

    tl->value_nodes[t + 1] = nc_dup_node(nc_get_node(value));
    slot = nc_slice_alias(tl->mem_value, 1, row, row + 1);
    nc_tensor_copy(slot, value);
    nc_free_tensor(value); nc_free_tensor(slot);
    value = nc_dup_tensor(tl->mem_value);

    t0 = nc_matmul_add(key, nc_dup_tensor(query), NULL, 1, 0, 1.0f);
    node = nc_get_node(t0);
    nc_node_set_arg(node, 1, query);
    tl->kq_nodes[t] = node;
    if (c->use_w_r) {
        rd = nc_matmul_add(nc_dup_tensor(tl->tmp_w_r), query, NULL, 1, 0, 1.0f);
        rd = nc_pad(rd, c->mem_len + c->seg_len - c->d_pos, NC_PAD_DUP, 0, NC_PAD_ZERO);
        rd = nc_add(rd, nc_slice(nc_dup_tensor(tl->tmp_b_r), 1, t, t + 1));
    } else {
        nc_free_tensor(query);
        rd = nc_slice(nc_dup_tensor(tl->tmp_b_r), 1, t, t + 1);
    }
    rd = nc_rel_shift(rd, -(c->seg_len - 1 - t), 1);
    t0 = nc_add(rd, t0);
    t0 = nc_mul(t0, scalar(s, 1.0f / sqrtf((float)c->d_key)));
    t1 = nc_slice_alias(tl->attn_mask, 1, t, t + 1);
    t0 = nc_masked_fill(t0, t1, -INFINITY, 0);
    t1 = nc_soft_max(t0);
    t0 = nc_matmul(value, nc_dup_tensor(t1));
    node = nc_get_node(t0);
    nc_node_set_arg(node, 1, t1);
    nc_free_tensor(t1);
    tl->va_nodes[t] = node;
    return t0;
}

/* self-attention block of the reference path: nncp.c:659-890 */
static NCTensor *attention_ref(NNCPModel *s, int l, int output_index, NCTensor *x, int seg_len)
{
    const NNCPConfig *c = &s->cfg;
    Layer *tl = &s->layers[l];
    int H = c->n_head, HDk = H * c->d_key, HDv = H * c->d_value, B = c->batch_size;
    NCTensor *query, *key, *value, *t0;

    query = nc_matmul(nc_dup_tensor(tl->w_q), nc_dup_tensor(x));
    if (c->query_bias)
        query = nc_add(query, nc_dup_tensor(tl->b_q));
    t0 = nc_matmul(nc_dup_tensor(tl->w_kv), x);
    key = nc_slice(nc_dup_tensor(t0), 0, 0, HDk);
    value = nc_slice(t0, 0, HDk, HDk + HDv);
    query = nc_reshape_3d(query, HDk, B, seg_len);
    key = nc_reshape_3d(key, HDk, B, seg_len);
    value = nc_reshape_3d(value, HDv, B, seg_len);

    if (output_index <= 0) { /* keys / values of the memory, nncp.c:673-711 */
        NCTensor *key0, *value0;
        t0 = nc_reshape_2d(nc_dup_tensor(s->mem_h[l]), c->d_model, c->mem_len * B);
        t0 = nc_matmul(nc_dup_tensor(tl->w_kv), t0);
        key0 = nc_slice(nc_dup_tensor(t0), 0, 0, HDk);
        value0 = nc_slice(t0, 0, HDk, HDk + HDv);
        key0 = nc_reshape_3d(key0, HDk, B, c->mem_len);
        value0 = nc_reshape_3d(value0, HDv, B, c->mem_len);
        if (output_index < 0) {
            NCTensor *tab[2];
            tab[0] = key0; tab[1] = key;
            key = nc_concat(tab, 2, 2);
            tab[0] = value0; tab[1] = value;
            value = nc_concat(tab, 2, 2);
        } else {
            NCTensor *slot = nc_slice_alias(tl->mem_key, 1, 0, c->mem_len);
            key0 = split_head(key0, H);
            tl->key_nodes[0] = nc_dup_node(nc_get_node(key0));
            nc_tensor_copy(slot, key0);
            nc_free_tensor(key0); nc_free_tensor(slot);
            slot = nc_slice_alias(tl->mem_value, 1, 0, c->mem_len);
            value0 = split_head(value0, H);
            tl->value_nodes[0] = nc_dup_node(nc_get_node(value0));
            nc_tensor_copy(slot, value0);
            nc_free_tensor(value0); nc_free_tensor(slot);
        }
    }
    query = dropout_mul(s, query, c->dropout_prob); /* nncp.c:713-717; none on the keys */
    value = dropout_mul(s, value, c->dropout_prob);
    key = split_head(key, H);
    query = split_head(query, H);
    value = split_head(value, H);
    if (output_index <= 0)
        build_position_tensors(s, l);
    if (output_index < 0)
        t0 = attention_segment_ref(s, l, query, key, value);
    else
        t0 = attention_timestep_ref(s, l, output_index, query, key, value);
    if (tl->w_o) {
        t0 = nc_matmul(nc_dup_tensor(tl->w_o), concat_head(t0));
        t0 = dropout_mul(s, t0, c->dropout_prob); /* nncp.c:873-874 */
    } else { /* sum of the heads, nncp.c:875-890 */
        int axis[4] = { 0, 3, 1, 2 };
        t0 = nc_permute(t0, 4, axis);
        t0 = nc_reduce_sum(NULL, t0, 3);
        t0 = nc_mul(t0, scalar(s, 1.0f / sqrtf((float)H)));
        t0 = nc_reshape_2d(t0, c->d_value, (size_t)seg_len * B);
    }
    return t0;
}

/* the same block through the fused entry points (full segment) */
/* res (or NULL) is the residual input, added by the output projection itself */
static NCTensor *attention_fused(NNCPModel *s, int l, NCTensor *x, NCTensor *res)
{
    const NNCPConfig *c = &s->cfg;
    Layer *tl = &s->layers[l];
    int H = c->n_head, HDk = H * c->d_key, HDv = H * c->d_value, B = c->batch_size, T = c->seg_len;
    NCTensor *q, *kv, *kvm = NULL, *att;
    Layer *pr = &s->layers[c->tied_w_r ? 0 : l], *pb = &s->layers[c->tied_b_r ? 0 : l];

    /* (bf16 products: the attention reads bf16 operands too, so these three products leave the
       bf16 copies of their results) */
    int copies = nc_set_bf16_copy_of_results(s->ctx, 1);
    q = nc_linear(nc_dup_tensor(tl->w_q), nc_dup_tensor(x), c->query_bias ? nc_dup_tensor(tl->b_q) : NULL, NC_ACT_NONE);
    kv = nc_matmul(nc_dup_tensor(tl->w_kv), x);
    if (c->mem_len > 0) {
        kvm = nc_reshape_2d(nc_dup_tensor(s->mem_h[l]), c->d_model, (size_t)c->mem_len * B);
        kvm = nc_matmul(nc_dup_tensor(tl->w_kv), kvm);
        kvm = nc_reshape_3d(kvm, HDk + HDv, B, c->mem_len);
    }
    nc_set_bf16_copy_of_results(s->ctx, copies);
    att = nc_relpos_attention(nc_reshape_3d(q, HDk, B, T), nc_reshape_3d(kv, HDk + HDv, B, T), kvm,
                              c->use_w_r ? nc_dup_tensor(pr->w_r) : NULL, nc_dup_tensor(pb->b_r),
                              H, c->d_key, c->attn_len[l], sqrtf((float)(c->d_key * c->d_model)));
    att = nc_reshape_2d(att, HDv, (size_t)B * T);
    if (!tl->w_o)
        die("the fused path needs d_value != d_model (an output projection)");
    return nc_matmul_add(nc_dup_tensor(tl->w_o), att, res, 0, 0, 1.0f);
}

/* feed-forward block: nncp.c:930-977; res (fused path only, or NULL) is the
   residual input, added by the second linear layer itself */
static NCTensor *feed_forward(NNCPModel *s, int l, NCTensor *x, NCTensor *res)
{
    const NNCPConfig *c = &s->cfg;
    Layer *tl = &s->layers[l];
    NCTensor *t0, *tab[2];
    int act = c->ff_act;
    if (s->fused_now && (act == NNCP_FF_GELU || act == NNCP_FF_RELU)) {
        t0 = nc_linear(nc_dup_tensor(tl->ff1), x, tl->ff_bias1 ? nc_dup_tensor(tl->ff_bias1) : NULL,
                       act == NNCP_FF_GELU ? NC_ACT_GELU : NC_ACT_RELU);
        if (res)
            return nc_linear_add(nc_dup_tensor(tl->ff2), t0, tl->ff_bias2 ? nc_dup_tensor(tl->ff_bias2) : NULL,
                                 NC_ACT_NONE, res);
        return nc_linear(nc_dup_tensor(tl->ff2), t0, tl->ff_bias2 ? nc_dup_tensor(tl->ff_bias2) : NULL, NC_ACT_NONE);
    }
    if (res)
        die("feed_forward: the residual is fused only on the fused GELU/ReLU path");
    t0 = nc_matmul(nc_dup_tensor(tl->ff1), x);
    if (tl->ff_bias1)
        t0 = nc_add(t0, nc_dup_tensor(tl->ff_bias1));
    t0 = dropout_mul(s, t0, c->dropout_prob); /* before the activation, nncp.c:933-934 */
    switch (act) {
    case NNCP_FF_RELU: t0 = nc_relu(t0); break;
    case NNCP_FF_GELU: t0 = nc_gelu(t0); break;
    case NNCP_FF_GEGLU:
        nc_split(tab, t0, 2, NULL, 0);
        t0 = nc_mul(nc_gelu(tab[0]), tab[1]);
        break;
    case NNCP_FF_GATED_SILU:
        nc_split(tab, t0, 2, NULL, 0);
        t0 = nc_gated_swish(tab[1], tab[0], 1.0f);
        break;
    default: die("unknown ff_act");
    }
    t0 = nc_matmul(nc_dup_tensor(tl->ff2), t0);
    if (tl->ff_bias2)
        t0 = nc_add(t0, nc_dup_tensor(tl->ff_bias2));
    return dropout_mul(s, t0, c->dropout_prob); /* nncp.c:973-974 */
}

static void free_position_tensors(NNCPModel *s)
{
    for (int l = 0; l < s->cfg.n_layer; l++) {
        nc_free_tensor(s->layers[l].tmp_w_r); s->layers[l].tmp_w_r = NULL;
        nc_free_tensor(s->layers[l].tmp_b_r); s->layers[l].tmp_b_r = NULL;
    }
}

NCTensor *trf_eval(NNCPModel *s, int output_index, const NCTensor *input)
{
    const NNCPConfig *c = &s->cfg;
    int seg_len, B = c->batch_size;
    NCTensor *t0, *x, *output;

    prof_start(PROF_EVAL); /* nncp.c:606 */
    /* dropout masks sit between steps that the fused entry points merge, so a
       retrain pass goes through the op-by-op sequence */
    s->fused_now = c->fused && !s->dropout_enabled;
    const int fused = s->fused_now;
    if (fused && output_index >= 0)
        die("the fused path evaluates whole segments only (output_index < 0)");
    if (output_index < 0) { /* nncp.c:612-623 */
        /* a copy of the caller's tokens that ends with its upload: the library can leave
           that transfer queued instead of waiting for it (the caller may rewrite `input`) */
        t0 = nc_new_tensor_from_tensor_nz(input);
        nc_tensor_copy(t0, (NCTensor *)input);
        s->seq_eval = 0;
        seg_len = c->seg_len;
    } else {
        t0 = nc_slice_alias(input, 1, output_index, output_index + 1);
        s->seq_eval = 1;
        seg_len = 1;
    }
    t0 = nc_tensor_to_device(t0, s->dev);
    t0 = nc_reshape_1d(t0, (size_t)B * seg_len);
    x = nc_get_col(nc_dup_tensor(s->embed), t0);
    x = nc_mul(x, scalar(s, s->embed_mult));
    x = dropout_mul(s, x, c->dropout_prob); /* nncp.c:631-633 */

    for (int l = 0; l < c->n_layer; l++) {
        Layer *tl = &s->layers[l];
        NCTensor *x1 = nc_dup_tensor(x), *ff_in;
        if (c->ln_flags & NNCP_LN_PRE)
            x1 = layer_norm(s, x1, tl->ln_g1, tl->ln_b1);
        save_layer_input(s, l, output_index, x1, seg_len);
        /* the fused path folds the residual sums (nncp.c:896, 979) into the
           GEMMs that produce their other operand */
        int fold = fused && !(c->ln_flags & NNCP_LN_COEF);
        int fold_ff = fold && (c->ff_act == NNCP_FF_GELU || c->ff_act == NNCP_FF_RELU);
        if (fold) {
            t0 = attention_fused(s, l, x1, x);
        } else {
            t0 = fused ? attention_fused(s, l, x1, NULL) : attention_ref(s, l, output_index, x1, seg_len);
            if (c->ln_flags & NNCP_LN_COEF)
                t0 = nc_mul(t0, nc_dup_tensor(tl->alpha));
            t0 = nc_add(t0, x); /* residual, nncp.c:896 */
        }
        if (c->ln_flags & NNCP_LN_POST)
            t0 = layer_norm(s, t0, tl->ln_g1, tl->ln_b1);
        ff_in = nc_dup_tensor(t0);
        if (c->ln_flags & NNCP_LN_PRE)
            t0 = layer_norm(s, t0, tl->ln_g2, tl->ln_b2);
        if (fold_ff) {
            t0 = feed_forward(s, l, t0, ff_in);
        } else {
            t0 = feed_forward(s, l, t0, NULL);
            if (c->ln_flags & NNCP_LN_COEF)
                t0 = nc_mul(t0, nc_dup_tensor(tl->alpha));
            t0 = nc_add(t0, ff_in); /* nncp.c:979 */
        }
        if (c->ln_flags & NNCP_LN_POST)
            t0 = layer_norm(s, t0, tl->ln_g2, tl->ln_b2);
        x = t0;
    }
    if (c->ln_flags & NNCP_LN_FINAL)
        x = layer_norm(s, x, s->ln_g, s->ln_b);
    x = dropout_mul(s, x, c->dropout_prob); /* nncp.c:997-999 */
    /* logits and probabilities, nncp.c:1001-1009 */
    if (fused) {
        t0 = nc_linear(nc_dup_tensor(s->embed_out), x, s->out_bias ? nc_dup_tensor(s->out_bias) : NULL, NC_ACT_NONE);
    } else {
        t0 = nc_matmul(nc_dup_tensor(s->embed_out), x);
        if (s->out_bias)
            t0 = nc_add(t0, nc_dup_tensor(s->out_bias));
    }
    t0 = nc_reshape_3d(t0, c->n_symbols, B, seg_len);
    nc_free_tensor(s->logits);
    s->logits = nc_dup_tensor(t0);
    output = nc_soft_max(t0);
    if (s->outputs[output_index < 0 ? 0 : output_index])
        die("trf_eval: previous evaluation not consumed (call trf_eval_gradient or trf_eval_end)");
    s->outputs[output_index < 0 ? 0 : output_index] = nc_dup_tensor(output);
    if (!fused && (output_index < 0 || output_index == c->seg_len - 1))
        free_position_tensors(s);
    prof_end(PROF_EVAL); /* nncp.c:1027 */
    return output;
}

NCTensor *trf_last_logits(NNCPModel *s) { return s->logits; }

/* ---- per-timestep evaluation with K/V caches (the decoder's view, nncp.c:801-863,
   through the fused entry points) ------------------------------------------------
   trf_step_begin once per segment, then trf_eval_step(t) for t = 0, 1, ...: each
   call evaluates ONE token column (the symbols of position t-1 of every stream)
   against the memory and the columns seen so far.  With
   nc_set_matmul_width_invariant() on in both the encoder and the decoder its
   logits are bit-identical to column t of the whole-segment trf_eval. */
void trf_step_end(NNCPModel *s)
{
    if (!s->step_kv) return;
    for (int l = 0; l < s->cfg.n_layer; l++) {
        nc_free_tensor(s->step_kv[l]); s->step_kv[l] = NULL;
        nc_free_tensor(s->step_kvm[l]); s->step_kvm[l] = NULL;
    }
    nc_free_tensor(s->step_embed_mult); s->step_embed_mult = NULL;
    s->step_logits_only = 0;
    nc_forget_k_major_weights(s->ctx);
}

void trf_step_begin(NNCPModel *s)
{
    const NNCPConfig *c = &s->cfg;
    if (!c->fused)
        die("per-timestep cached evaluation needs the fused path (cfg.fused = 1)");
    if (s->dropout_enabled)
        die("per-timestep cached evaluation is a decoding path: not during a retrain pass");
    s->fused_now = 1;
    if (!s->step_kv) {
        s->step_kv = nc_mallocz(sizeof(NCTensor *) * c->n_layer);
        s->step_kvm = nc_mallocz(sizeof(NCTensor *) * c->n_layer);
    }
    trf_step_end(s);
    for (int l = 0; l < c->n_layer; l++) /* zero: columns not yet reached are masked but must be finite */
        s->step_kv[l] = nc_new_tensor_3d(s->dev, NC_TYPE_F32, (size_t)c->n_head * (c->d_key + c->d_value),
                                         c->batch_size, c->seg_len);
    s->step_embed_mult = scalar(s, s->embed_mult);
    /* the weights do not change until the training step that follows the last timestep: the
       products of a timestep (a few token columns each) read k-major copies of them */
    for (int l = 0; l < c->n_layer; l++) {
        Layer *tl = &s->layers[l];
        nc_keep_k_major_weight(tl->w_q);
        nc_keep_k_major_weight(tl->w_kv);
        if (tl->w_o) nc_keep_k_major_weight(tl->w_o);
        nc_keep_k_major_weight(tl->ff1);
        nc_keep_k_major_weight(tl->ff2);
    }
    nc_keep_k_major_weight(s->embed_out);
}

void trf_step_logits_only(NNCPModel *s, int on)
{
    s->step_logits_only = on;
}

NCTensor *trf_eval_step(NNCPModel *s, int t, const NCTensor *input)
{
    const NNCPConfig *c = &s->cfg;
    int B = c->batch_size, H = c->n_head, HDk = H * c->d_key, HDv = H * c->d_value;
    NCTensor *t0, *x;
    if (!s->step_kv || !s->step_kv[0])
        die("trf_eval_step: call trf_step_begin first");
    if (t < 0 || t >= c->seg_len)
        die("trf_eval_step: position outside the segment");
    t0 = nc_slice_alias(input, 1, t, t + 1);
    t0 = nc_reshape_1d(t0, (size_t)B);
    if (s->dev != s->cpu && nc_get_tensor_device(input) == s->cpu) {
        /* the kernel reads the tokens where they are and applies the multiplier */
        x = nc_get_col_host_indices(nc_dup_tensor(s->embed), t0, s->embed_mult);
    } else {
        x = nc_get_col(nc_dup_tensor(s->embed), nc_tensor_to_device(t0, s->dev));
        x = nc_mul(x, nc_dup_tensor(s->step_embed_mult));
    }
    /* Post-norm blocks with a plain activation (nncp's default structure, nncp.c:2489-2513):
       a norm is followed by a product, so it rides on that product's launch
       (nc_norm_linear_pair_into) - the norm after the attention on the first feed-forward
       product, the norm that ends a block on the projections of the next block or on the
       output product.  `pend` is the block whose closing norm x still waits for. */
    const int ride = (c->ln_flags & (NNCP_LN_PRE | NNCP_LN_POST | NNCP_LN_FINAL | NNCP_LN_COEF)) == NNCP_LN_POST &&
                     (c->ff_act == NNCP_FF_GELU || c->ff_act == NNCP_FF_RELU);
    const int is_ln = !(c->ln_flags & NNCP_LN_RMSNORM);
    Layer *pend = NULL;
    for (int l = 0; l < c->n_layer; l++) {
        Layer *tl = &s->layers[l];
        Layer *pr = &s->layers[c->tied_w_r ? 0 : l], *pb = &s->layers[c->tied_b_r ? 0 : l];
        NCTensor *x1 = NULL, *ff_in, *q, *att;
        if (!pend) {
            x1 = nc_dup_tensor(x);
            if (c->ln_flags & NNCP_LN_PRE)
                x1 = layer_norm(s, x1, tl->ln_g1, tl->ln_b1);
        }
        if (t == 0 && c->mem_len > 0) { /* K/V of the memory: once per segment */
            NCTensor *m2 = nc_reshape_2d(nc_dup_tensor(s->mem_h[l]), c->d_model, (size_t)c->mem_len * B);
            m2 = nc_matmul(nc_dup_tensor(tl->w_kv), m2);
            s->step_kvm[l] = nc_reshape_3d(m2, HDk + HDv, B, c->mem_len);
        }
        /* query and key / value of this position in one launch; the latter goes straight into
           column t of the cache */
        if (pend) {
            NCTensor *xn;
            q = nc_norm_linear_pair_into(x, nc_dup_tensor(pend->ln_g2), nc_dup_tensor(pend->ln_b2), 1e-5f, is_ln,
                                         nc_dup_tensor(tl->w_q), c->query_bias ? nc_dup_tensor(tl->b_q) : NULL, NC_ACT_NONE,
                                         nc_dup_tensor(tl->w_kv), s->step_kv[l], t, &xn);
            x = xn;
            pend = NULL;
        } else {
            q = nc_linear_pair_into(nc_dup_tensor(tl->w_q), c->query_bias ? nc_dup_tensor(tl->b_q) : NULL,
                                    nc_dup_tensor(tl->w_kv), x1, s->step_kv[l], t);
        }
        att = nc_relpos_attention_step(q, nc_dup_tensor(s->step_kv[l]),
                                       c->mem_len > 0 ? nc_dup_tensor(s->step_kvm[l]) : NULL,
                                       c->use_w_r ? nc_dup_tensor(pr->w_r) : NULL, nc_dup_tensor(pb->b_r),
                                       H, c->d_key, c->attn_len[l], sqrtf((float)(c->d_key * c->d_model)), t);
        if (!tl->w_o)
            die("the fused path needs d_value != d_model (an output projection)");
        if (ride) {
            NCTensor *h;
            int act = c->ff_act == NNCP_FF_GELU ? NC_ACT_GELU : NC_ACT_RELU;
            t0 = nc_matmul_add(nc_dup_tensor(tl->w_o), att, x, 0, 0, 1.0f);
            h = nc_norm_linear_pair_into(t0, nc_dup_tensor(tl->ln_g1), nc_dup_tensor(tl->ln_b1), 1e-5f, is_ln,
                                         nc_dup_tensor(tl->ff1), tl->ff_bias1 ? nc_dup_tensor(tl->ff_bias1) : NULL, act,
                                         NULL, NULL, 0, &ff_in);
            x = nc_linear_add(nc_dup_tensor(tl->ff2), h, tl->ff_bias2 ? nc_dup_tensor(tl->ff_bias2) : NULL,
                              NC_ACT_NONE, ff_in);
            pend = tl;
            continue;
        }
        int fold = !(c->ln_flags & NNCP_LN_COEF);
        int fold_ff = fold && (c->ff_act == NNCP_FF_GELU || c->ff_act == NNCP_FF_RELU);
        if (fold) {
            t0 = nc_matmul_add(nc_dup_tensor(tl->w_o), att, x, 0, 0, 1.0f);
        } else {
            t0 = nc_matmul_add(nc_dup_tensor(tl->w_o), att, NULL, 0, 0, 1.0f);
            t0 = nc_mul(t0, nc_dup_tensor(tl->alpha));
            t0 = nc_add(t0, x);
        }
        if (c->ln_flags & NNCP_LN_POST)
            t0 = layer_norm(s, t0, tl->ln_g1, tl->ln_b1);
        ff_in = nc_dup_tensor(t0);
        if (c->ln_flags & NNCP_LN_PRE)
            t0 = layer_norm(s, t0, tl->ln_g2, tl->ln_b2);
        if (fold_ff) {
            t0 = feed_forward(s, l, t0, ff_in);
        } else {
            t0 = feed_forward(s, l, t0, NULL);
            if (c->ln_flags & NNCP_LN_COEF)
                t0 = nc_mul(t0, nc_dup_tensor(tl->alpha));
            t0 = nc_add(t0, ff_in);
        }
        if (c->ln_flags & NNCP_LN_POST)
            t0 = layer_norm(s, t0, tl->ln_g2, tl->ln_b2);
        x = t0;
    }
    if (c->ln_flags & NNCP_LN_FINAL)
        x = layer_norm(s, x, s->ln_g, s->ln_b);
    if (pend)
        t0 = nc_norm_linear_pair_into(x, nc_dup_tensor(pend->ln_g2), nc_dup_tensor(pend->ln_b2), 1e-5f, is_ln,
                                      nc_dup_tensor(s->embed_out), s->out_bias ? nc_dup_tensor(s->out_bias) : NULL,
                                      NC_ACT_NONE, NULL, NULL, 0, NULL);
    else
        t0 = nc_linear(nc_dup_tensor(s->embed_out), x, s->out_bias ? nc_dup_tensor(s->out_bias) : NULL, NC_ACT_NONE);
    t0 = nc_reshape_3d(t0, c->n_symbols, B, 1);
    nc_free_tensor(s->logits);
    s->logits = nc_dup_tensor(t0);
    if (s->step_logits_only)
        return t0;
    return nc_soft_max(t0);
}

void trf_eval_end(NNCPModel *s) /* nncp.c:1032-1060 */
{
    free_position_tensors(s);
    for (int l = 0; l < s->cfg.n_layer; l++) {
        Layer *tl = &s->layers[l];
        for (int i = 0; i <= s->cfg.seg_len; i++) {
            nc_free_node(tl->key_nodes[i]); tl->key_nodes[i] = NULL;
            nc_free_node(tl->value_nodes[i]); tl->value_nodes[i] = NULL;
        }
    }
    for (int i = 0; i < s->cfg.seg_len; i++) {
        nc_free_tensor(s->outputs[i]);
        s->outputs[i] = NULL;
    }
    nc_free_tensor(s->logits);
    s->logits = NULL;
    nc_free_tensor(s->pending_loss); nc_free_tensor(s->pending_loss_host);
    s->pending_loss = s->pending_loss_host = NULL;
}

void nncp_backward_cb(void *opaque, NCTensor *yg, NCTensor *get_col_index) /* nncp.c:1078-1096 */
{
    sgd_opt_update_var(opaque, yg, get_col_index);
}

/* route the gradients of the T per-timestep products into one concatenated
   key (value) tensor: nncp.c:1116-1158 */
static NCNode *merge_timestep_nodes(NNCPModel *s, NCNode **src, NCNode **consumers)
{
    int T = s->cfg.seg_len;
    size_t *ones = nc_malloc(sizeof(size_t) * T), two[2] = { (size_t)s->cfg.mem_len, (size_t)T };
    NCNode *n, *n1, *pair[2];
    for (int i = 0; i < T; i++)
        ones[i] = 1;
    n = nc_concat_node(s->ctx, src + 1, T, 1, ones);
    pair[0] = src[0]; pair[1] = n;
    n1 = nc_concat_node(s->ctx, pair, 2, 1, two);
    for (int i = 0; i <= T; i++) {
        nc_free_node(src[i]);
        src[i] = NULL;
    }
    for (int i = 0; i < T; i++)
        nc_node_set_parent(consumers[i], 0, n1);
    nc_free_node(n);
    nc_free_node(n1);
    nc_free(ones);
    return n;
}

/* NNCPModelClass.queue_loss: the first half of trf_eval_gradient for a whole-segment
   evaluation, queued behind it without a wait */
static void trf_queue_loss(NNCPModel *s, NCTensor *expected)
{
    if (s->seq_eval || !s->outputs[0] || s->pending_loss) {
        nc_free_tensor(expected);
        return;
    }
    NCTensor *output = s->outputs[0];
    s->outputs[0] = NULL;
    NCTensor *loss = nc_sum(nc_indexed_log(output, expected));
    s->pending_loss_host = nc_tensor_to_cpu_device_queued(nc_dup_tensor(loss));
    s->pending_loss = loss;
}

float trf_eval_gradient(NNCPModel *s, const NCTensor *expected_output1) /* nncp.c:1099-1193 */
{
    const NNCPConfig *c = &s->cfg;
    NCTensor *expected, *output, *loss;
    float ret;
    if (s->pending_loss) { /* queued by trf_queue_loss; the caller has waited since */
        prof_start(PROF_GRAD);
        nc_synchronize(s->dev); /* (no cost on a drained stream; a guard for a caller that has not) */
        loss = s->pending_loss;
        ret = ((const float *)nc_tensor_get_ptr(s->pending_loss_host, NULL))[0];
        nc_free_tensor(s->pending_loss_host);
        s->pending_loss = s->pending_loss_host = NULL;
        goto backward;
    }
    expected = nc_tensor_to_device(nc_dup_tensor(expected_output1), s->dev);
    prof_start(PROF_GRAD); /* nncp.c:1108 */
    if (s->seq_eval) {
        NCNode **tab = nc_malloc(sizeof(NCNode *) * (c->n_layer * 2 + 1));
        int count = 0;
        for (int l = 0; l < c->n_layer; l++) {
            Layer *tl = &s->layers[l];
            tab[count++] = merge_timestep_nodes(s, tl->key_nodes, tl->kq_nodes);
            tab[count++] = merge_timestep_nodes(s, tl->value_nodes, tl->va_nodes);
        }
        output = nc_concat(s->outputs, c->seg_len, 2);
        for (int i = 0; i < c->seg_len; i++)
            s->outputs[i] = NULL;
        tab[count++] = nc_get_node(output);
        nc_concat_optimization(s->ctx, tab, count);
        nc_free(tab);
    } else {
        output = s->outputs[0];
        s->outputs[0] = NULL;
    }
    loss = nc_indexed_log(output, nc_dup_tensor(expected));
    nc_free_tensor(expected);
    loss = nc_sum(loss);
    ret = nc_get_scalar_f32(loss);
backward:
    loss = nc_mul(loss, nc_new_f32(nc_get_tensor_device(loss), -1.0f / (float)(c->seg_len * c->batch_size)));
    nc_backward(loss, nc_new_f32(s->dev, 1.0f), nncp_backward_cb, 0);
    nc_free_tensor(loss);
    nc_free_tensor(s->logits);
    s->logits = NULL;
    prof_end(PROF_GRAD); /* nncp.c:1191 */
    return ret;
}

void trf_reset(NNCPModel *s) /* nncp.c:1195-1203 */
{
    for (int l = 0; l < s->cfg.n_layer; l++)
        nc_tensor_set_zero(s->mem_h[l]);
}

void trf_update(NNCPModel *s) /* nncp.c:1224-1235 with mem_update nncp.c:1205-1221 */
{
    int M = s->cfg.mem_len, T = s->cfg.seg_len;
    prof_start(PROF_UPDATE); /* nncp.c:1227 */
    nc_sgd_opt_update(s->opt);
    for (int l = 0; l < s->cfg.n_layer && M > 0; l++) {
        if (M > T && s->mem_cap) {
            /* the same memory as below, at a new place: the segment goes behind the window
               and the window moves on by T; at the end of the store the rows that stay go
               back to its start (once in mem_cap / T - M / T + 1 updates) */
            NCTensor *store = s->mem_store[l];
            int pos = s->mem_pos[l];
            if (pos + M + T <= s->mem_cap) {
                nc_tensor_copy_slice(store, s->train_h[l], 2, pos + M, pos + M + T, 0);
                pos += T;
            } else {
                nc_tensor_copy_slice(store, store, 2, 0, M - T, pos + T);
                nc_tensor_copy_slice(store, s->train_h[l], 2, M - T, M, 0);
                pos = 0;
            }
            s->mem_pos[l] = pos;
            nc_free_tensor(s->mem_h[l]);
            s->mem_h[l] = nc_slice_alias(store, 2, pos, pos + M);
        } else if (M > T) {
            nc_tensor_copy_slice(s->mem_h[l], s->mem_h[l], 2, 0, M - T, T);
            nc_tensor_copy_slice(s->mem_h[l], s->train_h[l], 2, M - T, M, 0);
        } else if (M == T) {
            /* the memory becomes exactly the saved layer inputs: the two tensors trade
               places (train_h is rewritten in full before it is read again) */
            NCTensor *tmp = s->mem_h[l];
            s->mem_h[l] = s->train_h[l];
            s->train_h[l] = tmp;
        } else {
            nc_tensor_copy_slice(s->mem_h[l], s->train_h[l], 2, 0, M, T - M);
        }
    }
    s->train_step++;
    prof_end(PROF_UPDATE); /* nncp.c:1234 */
}

void trf_set_lr(NNCPModel *s, float lr) { nc_sgd_opt_set_lr(s->opt, lr); }

void trf_set_retrain(NNCPModel *s, int enabled) /* nncp.c:1237-1241 */
{
    s->dropout_enabled = enabled && s->cfg.dropout_prob != 0;
}

NNCPRetrainState *nncp_model_retrain_state(NNCPModel *s) { return &s->retrain; }
void nncp_model_set_train_step(NNCPModel *s, int64_t step) { s->train_step = step; }

const NNCPModelClass nncp_trf_class = { /* nncp.c:1544-1562 */
    trf_eval, trf_eval_end, trf_eval_gradient, trf_reset, trf_update, trf_set_lr, trf_set_retrain, trf_last_logits,
    trf_eval_end, /* no state is handed on before trf_update */
    trf_queue_loss,
};

const NNCPModelClass *nncp_model_class(NNCPModel *s) { return s->cls; }
NCTensor *nncp_model_last_logits(NNCPModel *s) { return s->cls->last_logits(s); }
