/*
 * lstm_model.c - the `lstm` model class of the reference (nncp.c:1565-2330)
 * over the libnc ABI: stacked LSTM cells (normal / clamped / tied memory
 * update), sparse input embedding per layer (ws), optional connection of
 * every layer to all layers below (full_connect), RMS layer norm with a
 * scalar gain per gate, optional projection, and one output layer over the
 * (grouped) sum of the layer outputs.  Same entry points and ownership rules
 * as the reference's lstm_eval / lstm_eval_gradient / lstm_update, called by
 * the block loop through NNCPModelClass.
 *
 * Restrictions of this mirror: n_states = seg_len (no overlapping states), no
 * dropout (the reference's dropout2_init returns NULL, nncp.c:1657-1681, and
 * its decoder asserts dropout off), GRU cells are not built (the reference
 * marks them unsupported, nncp.c:1969), fp32 parameters.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "model_internal.h"

#define MAT_MAX 4
#define FORGET_GATE 0 /* nncp.c:1571-1574 */
#define INPUT_NODE 1
#define OUTPUT_GATE 2
#define INPUT_GATE 3

typedef struct { /* LSTMCell, nncp.c:1580-1596 */
    int mat_count;
    NCTensor *u, *w, *ws, *b[MAT_MAX], *g[MAT_MAX], *p;
    NCTensor *c0, *h0; /* state carried to the next segment */
    NCTensor *c0_prev, *h0_prev; /* what they held before the last segment evaluation */
    NCTensor *c, *h;   /* state inside the segment (with its graph) */
} Cell;

struct LstmState {
    Cell *cells;
    NCTensor **outputs;
    NCTensor *fc_b, *fc_w, *logits;
    int seq_eval;
};

static void die(const char *msg)
{
    fprintf(stderr, "nncp_host (lstm): %s\n", msg);
    abort();
}

static NCTensor *param(NNCPModel *s, NCTensor **slot, NCTensor *t, float range, const char *fmt, int a, int b)
{
    *slot = t;
    nc_new_param(&s->params, slot, fmt, a, b);
    if (range != 0)
        nc_tensor_set_rnd_unif(t, 0, range, s->rnd); /* var_init_rnd, nncp.c:1650 */
    return t;
}

void nncp_config_default_lstm(NNCPConfig *c) /* nncp.c:2574-2603 */
{
    memset(c, 0, sizeof(*c));
    c->model_type = NNCP_MODEL_LSTM;
    c->batch_size = 32; c->seg_len = 20; c->n_symbols = 256;
    c->n_layer = 4;
    c->lstm_n_cells = 352; c->lstm_n_cells2 = 352; c->lstm_n_embed_out = 4;
    c->lstm_type = NNCP_LSTM_CLAMPED;
    c->lstm_full_connect = 1; c->lstm_use_layer_norm = 1; c->lstm_forget_bias = 0;
    c->sgd_opt.algo = SGD_OPT_ADAM;
    c->sgd_opt.u.adam.beta1 = 0; c->sgd_opt.u.adam.beta2 = 0.9999f; c->sgd_opt.u.adam.eps = 1e-10f;
    c->sgd_opt.u.adam.gradient_clip = 0;
    c->sgd_opt.lr = 4e-3f;
    c->seed = 123; c->use_device = 1; c->nb_threads = 1;
}

void lstm_init(NNCPModel *s) /* nncp.c:1701-1813 */
{
    const NNCPConfig *c = &s->cfg;
    const int L = c->n_layer, C1 = c->lstm_n_cells, C2 = c->lstm_n_cells2, V = c->n_symbols, B = c->batch_size;
    if (L < 1 || L > NNCP_N_LAYER_MAX || C1 < 1 || C2 < C1 || c->lstm_n_embed_out < 1 || c->lstm_n_embed_out > L ||
        c->lstm_type < NNCP_LSTM_NORMAL || c->lstm_type > NNCP_LSTM_TIED)
        die("bad configuration (1 <= n_layer <= 32, n_cells2 >= n_cells >= 1, 1 <= n_embed_out <= n_layer, type normal/clamped/tied)");
    struct LstmState *ls = nc_mallocz(sizeof(*ls));
    s->lstm = ls;
    nc_param_list_init(s->ctx, &s->params);
    ls->cells = nc_mallocz(sizeof(Cell) * L);
    for (int l = 0; l < L; l++) {
        Cell *lc = &ls->cells[l];
        const int n_in = c->lstm_full_connect ? C1 * l : (l != 0 ? C1 : 0);
        lc->mat_count = c->lstm_type == NNCP_LSTM_TIED ? 3 : 4;
        const size_t rows = (size_t)C2 * lc->mat_count;
        param(s, &lc->u, nc_new_tensor_2d(s->dev, s->param_type, rows, C1), 1.0f / sqrtf((float)C1), "u%d", l, 0);
        if (n_in != 0)
            param(s, &lc->w, nc_new_tensor_2d(s->dev, s->param_type, rows, n_in), 1.0f / sqrtf((float)n_in), "w%d", l, 0);
        param(s, &lc->ws, nc_new_tensor_2d(s->dev, s->param_type, rows, V), 0.75f, "ws%d", l, 0);
        for (int j = 0; j < lc->mat_count; j++) {
            param(s, &lc->b[j], nc_new_tensor_1d(s->dev, s->param_type, C2), 0, "b%d_%d", l, j);
            if (c->lstm_use_layer_norm) {
                param(s, &lc->g[j], nc_new_scalar(s->dev, s->param_type), 0, "g%d_%d", l, j);
                nc_tensor_set_f32(lc->g[j], 1.0f);
            }
        }
        nc_tensor_set_f32(lc->b[FORGET_GATE], c->lstm_forget_bias);
        if (C2 != C1)
            param(s, &lc->p, nc_new_tensor_2d(s->dev, s->param_type, C1, C2), sqrtf(1.0f / (float)C2), "p%d", l, 0);
        /* lstm_set_batch_size, nncp.c:1815-1832 */
        lc->h0 = nc_new_tensor_2d(s->dev, NC_TYPE_F32, C1, B);
        lc->c0 = nc_new_tensor_2d(s->dev, NC_TYPE_F32, C2, B);
        lc->h0_prev = nc_new_tensor_2d(s->dev, NC_TYPE_F32, C1, B);
        lc->c0_prev = nc_new_tensor_2d(s->dev, NC_TYPE_F32, C2, B);
    }
    param(s, &ls->fc_b, nc_new_tensor_1d(s->dev, s->param_type, V), 0, "fc_b", 0, 0);
    param(s, &ls->fc_w, nc_new_tensor_2d(s->dev, s->param_type, V, (size_t)C1 * c->lstm_n_embed_out),
          sqrtf(12.0f / (float)(C1 * L)), "fc_w", 0, 0);
    ls->outputs = nc_mallocz(sizeof(NCTensor *) * c->seg_len);
    s->opt = nc_sgd_opt_init(s->ctx, &c->sgd_opt);
    nc_sgd_opt_set_all(&s->params, s->opt);
    lstm_reset(s);
}

void lstm_end(NNCPModel *s) /* nncp.c:1834-1857 */
{
    struct LstmState *ls = s->lstm;
    lstm_eval_end(s);
    nc_sgd_opt_set_all(&s->params, NULL);
    nc_sgd_opt_end(s->opt);
    nc_param_list_end(&s->params);
    for (int l = 0; l < s->cfg.n_layer; l++) {
        Cell *lc = &ls->cells[l];
        nc_free_tensor(lc->c0); nc_free_tensor(lc->h0);
        nc_free_tensor(lc->c0_prev); nc_free_tensor(lc->h0_prev);
        nc_free_tensor(lc->c); nc_free_tensor(lc->h);
    }
    nc_free(ls->outputs);
    nc_free(ls->cells);
    nc_free(ls);
}

void lstm_reset(NNCPModel *s) /* nncp.c:1859-1870 */
{
    for (int l = 0; l < s->cfg.n_layer; l++) {
        nc_tensor_set_f32(s->lstm->cells[l].h0, 0);
        nc_tensor_set_f32(s->lstm->cells[l].c0, 0);
    }
}

/* sums n_in layer outputs into n_out groups (the lower groups take one more
   when n_in is not a multiple) and stacks the groups: nncp.c:1627-1648 */
static NCTensor *concat_add(NCTensor **tab, int n_in, int n_out)
{
    NCTensor **grp = nc_mallocz(sizeof(NCTensor *) * n_out), *out;
    int q = n_in / n_out, r = n_in % n_out, k = 0;
    for (int i = 0; i < n_out; i++) {
        int n = q + (i < r);
        grp[i] = tab[k++];
        for (int j = 1; j < n; j++)
            grp[i] = nc_add(grp[i], tab[k++]);
    }
    out = nc_vconcat(grp, n_out);
    nc_free(grp);
    return out;
}

NCTensor *lstm_eval(NNCPModel *s, int output_index, const NCTensor *input) /* nncp.c:1872-2058 */
{
    const NNCPConfig *c = &s->cfg;
    struct LstmState *ls = s->lstm;
    const int L = c->n_layer, T = c->seg_len, B = c->batch_size;
    int t0i, t1i; /* states evaluated: [t0i, t1i) */
    if (output_index < 0) { ls->seq_eval = 0; t0i = 0; t1i = T; }
    else { ls->seq_eval = 1; t0i = output_index; t1i = output_index + 1; }
    const int n = t1i - t0i;
    prof_start(PROF_EVAL); /* nncp.c:1881 */
    NCTensor **layer_out = nc_mallocz(sizeof(NCTensor *) * T * L);
    NCTensor **pre = nc_mallocz(sizeof(NCTensor *) * T);
    NCTensor **tmp = nc_mallocz(sizeof(NCTensor *) * (T > L ? T : L));
    NCTensor *t0, *t1;

    for (int l = 0; l < L; l++) {
        Cell *lc = &ls->cells[l];
        /* the part of the gate pre-activations that does not depend on the
           recurrence, for all states at once: ws[:, token] (+ w * lower layers) */
        t0 = nc_slice_alias(input, 1, t0i, t1i);
        t0 = nc_tensor_to_device(t0, s->dev);
        t0 = nc_reshape_1d(t0, (size_t)n * B);
        t1 = nc_get_col(nc_dup_tensor(lc->ws), t0);
        if (l != 0) {
            for (int t = t0i; t < t1i; t++) {
                if (!c->lstm_full_connect || l == 1) {
                    tmp[t - t0i] = nc_dup_tensor(layer_out[t * L + l - 1]);
                } else {
                    NCTensor **below = nc_mallocz(sizeof(NCTensor *) * l);
                    for (int i = 0; i < l; i++)
                        below[i] = nc_dup_tensor(layer_out[t * L + i]);
                    tmp[t - t0i] = nc_vconcat(below, l);
                    nc_free(below);
                }
            }
            t0 = nc_hconcat(tmp, n);
            t1 = nc_add(t1, nc_matmul(nc_dup_tensor(lc->w), t0));
        }
        nc_split(pre + t0i, t1, n, NULL, 1);

        if (t0i == 0) { /* a new segment starts from the carried state, without its graph */
            nc_tensor_copy(lc->h0_prev, lc->h0);
            nc_tensor_copy(lc->c0_prev, lc->c0);
            nc_free_tensor(lc->h);
            lc->h = nc_new_tensor_2d(s->dev, NC_TYPE_F32, c->lstm_n_cells, B);
            nc_tensor_copy(lc->h, lc->h0);
            nc_free_tensor(lc->c);
            lc->c = nc_new_tensor_2d(s->dev, NC_TYPE_F32, c->lstm_n_cells2, B);
            nc_tensor_copy(lc->c, lc->c0);
        }
        NCTensor *h = lc->h, *cm = lc->c;
        for (int t = t0i; t < t1i; t++) {
            NCTensor *tab[MAT_MAX], *fg, *ig, *og, *in;
            t0 = nc_matmul(nc_dup_tensor(lc->u), h);
            t0 = nc_add(t0, pre[t]);
            nc_split(tab, t0, lc->mat_count, NULL, 0);
            for (int j = 0; j < lc->mat_count; j++) {
                if (c->lstm_use_layer_norm)
                    tab[j] = nc_mul(nc_rms_norm(tab[j], 1e-5f), nc_dup_tensor(lc->g[j]));
                tab[j] = nc_add(tab[j], nc_dup_tensor(lc->b[j]));
            }
            fg = nc_sigmoid(tab[FORGET_GATE]);
            og = nc_sigmoid(tab[OUTPUT_GATE]);
            in = nc_tanh(tab[INPUT_NODE]);
            switch (c->lstm_type) { /* nncp.c:1989-2007 */
            case NNCP_LSTM_NORMAL:
                ig = nc_sigmoid(tab[INPUT_GATE]);
                cm = nc_add(nc_mul(cm, fg), nc_mul(in, ig));
                h = nc_mul(og, nc_tanh(nc_dup_tensor(cm)));
                break;
            case NNCP_LSTM_CLAMPED:
                ig = nc_sigmoid(tab[INPUT_GATE]);
                cm = nc_lstm_clamped(cm, in, fg, ig);
                h = nc_mul(og, nc_dup_tensor(cm));
                break;
            default: /* tied: the input gate is 1 - forget gate */
                cm = nc_lerp(in, cm, fg);
                h = nc_mul(og, nc_dup_tensor(cm));
                break;
            }
            if (lc->p)
                h = nc_matmul(nc_dup_tensor(lc->p), h);
            layer_out[t * L + l] = nc_dup_tensor(h);
            if (t == T - 1) { /* state handed to the next segment */
                nc_tensor_copy(lc->h0, h);
                nc_tensor_copy(lc->c0, cm);
            }
        }
        lc->h = h;
        lc->c = cm;
    }

    /* output layer on all evaluated states at once, nncp.c:2028-2047 */
    for (int t = t0i; t < t1i; t++)
        tmp[t - t0i] = concat_add(layer_out + t * L, L, c->lstm_n_embed_out);
    t0 = nc_hconcat(tmp, n);
    t0 = nc_matmul(nc_dup_tensor(ls->fc_w), t0);
    t0 = nc_add(t0, nc_dup_tensor(ls->fc_b));
    t0 = nc_reshape_3d(t0, c->n_symbols, B, n);
    nc_free_tensor(ls->logits);
    ls->logits = nc_dup_tensor(t0);
    NCTensor *output = nc_soft_max(t0);
    if (ls->outputs[t0i])
        die("lstm_eval: previous evaluation not consumed (call lstm_eval_gradient or lstm_eval_end)");
    ls->outputs[t0i] = nc_dup_tensor(output);
    nc_free(layer_out);
    nc_free(pre);
    nc_free(tmp);
    prof_end(PROF_EVAL); /* nncp.c:2056 */
    return output;
}

void lstm_eval_end(NNCPModel *s) /* nncp.c:2060-2068 */
{
    struct LstmState *ls = s->lstm;
    for (int i = 0; i < s->cfg.seg_len; i++) {
        nc_free_tensor(ls->outputs[i]);
        ls->outputs[i] = NULL;
    }
    nc_free_tensor(ls->logits);
    ls->logits = NULL;
}

float lstm_eval_gradient(NNCPModel *s, const NCTensor *expected_output) /* nncp.c:2070-2133 */
{
    const NNCPConfig *c = &s->cfg;
    struct LstmState *ls = s->lstm;
    NCTensor *output, *loss;
    float ret;
    prof_start(PROF_GRAD); /* nncp.c:2079 */
    if (ls->seq_eval) {
        NCNode *node;
        output = nc_concat(ls->outputs, c->seg_len, 2);
        for (int i = 0; i < c->seg_len; i++)
            ls->outputs[i] = NULL;
        node = nc_get_node(output);
        nc_concat_optimization(s->ctx, &node, 1);
    } else {
        output = ls->outputs[0];
        ls->outputs[0] = NULL;
    }
    loss = nc_indexed_log(output, nc_tensor_to_device(nc_dup_tensor(expected_output), s->dev));
    loss = nc_sum(loss);
    ret = nc_get_scalar_f32(loss);
    loss = nc_mul(loss, nc_new_f32(s->dev, -1.0f / (float)(c->seg_len * c->batch_size)));
    /* (the reference also merges the per-timestep input products with
       nc_combine_nodes, nncp.c:2099-2117: an optimisation of the backward pass) */
    nc_backward(loss, nc_new_f32(s->dev, 1.0f), nncp_backward_cb, 0);
    nc_free_tensor(loss);
    nc_free_tensor(ls->logits);
    ls->logits = NULL;
    prof_end(PROF_GRAD); /* nncp.c:2131 */
    return ret;
}

void lstm_update(NNCPModel *s) /* nncp.c:2136-2142 */
{
    prof_start(PROF_UPDATE); /* nncp.c:2139 */
    nc_sgd_opt_update(s->opt);
    prof_end(PROF_UPDATE); /* nncp.c:2141 */
    s->train_step++; /* counted by process_block in the reference (nncp.c:3056) */
}

/* for an evaluation that must leave no trace: the state goes back to what the
   evaluation started from */
static void lstm_eval_discard(NNCPModel *s)
{
    lstm_eval_end(s);
    for (int l = 0; l < s->cfg.n_layer; l++) {
        Cell *lc = &s->lstm->cells[l];
        nc_tensor_copy(lc->h0, lc->h0_prev);
        nc_tensor_copy(lc->c0, lc->c0_prev);
    }
}

static void lstm_set_lr(NNCPModel *s, float lr) { nc_sgd_opt_set_lr(s->opt, lr); } /* nncp.c:2251 */
static void lstm_set_retrain(NNCPModel *s, int enabled) { (void)s; (void)enabled; }
static NCTensor *lstm_last_logits(NNCPModel *s) { return s->lstm->logits; }

const NNCPModelClass nncp_lstm_class = { /* nncp.c:2312-2330 */
    lstm_eval, lstm_eval_end, lstm_eval_gradient, lstm_reset, lstm_update, lstm_set_lr, lstm_set_retrain,
    lstm_last_logits, lstm_eval_discard, NULL,
};
