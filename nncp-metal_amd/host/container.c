/*
 * File container around the block loop: the profiles of nncp_init_params
 * (nncp.c:2464-2636), the schedule syntax of parse_interp_param /
 * dump_interp_param (cp_utils.c:412-470), the big-endian file header
 * (nncp_write_file_header / nncp_read_file_header, nncp.c:2662-2760, with
 * trf_write_params nncp.c:1333-1365, lstm_write_params nncp.c:2198-2211 and
 * fput_sgd_opt cp_utils.c:214-229) and the file loops of encode_file /
 * decode_file (nncp.c:3307-3506, 3508-3677) without the dictionary
 * preprocessor.
 *
 * The byte after the header is the reference's "preprocessed" flag (bit 0,
 * always 0 here).  Its other bits, which the reference's reader ignores, hold
 * what this build adds to the stream format: bits 1-3 the NNCP_MODE_ /
 * NNCP_CODER_ flags, bit 4 cfg.fused.  With all of them 0 the container is
 * byte for byte the reference's.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "../../include/nncp_host.h"

#define FILE_MAGIC 0xb727ac58u /* nncp.c:2662 */
#define FILE_VERSION 1
#define INTERP_MAX_STEPS 8     /* cp_utils.h:60 */
#define ARITH_BUF_LEN 65536    /* nncp.c:3185 */

/* ---- schedules as text ----------------------------------------------------- */
int nncp_parse_interp(NNCPInterp *p, const char *r)
{
    char *e;
    memset(p, 0, sizeof(*p));
    p->val[0] = (float)strtod(r, &e);
    if (e == r)
        return -1;
    r = e;
    while (*r != '\0') {
        if (*r++ != ',')
            return -1;
        if (*r == 'p') {                       /* ",p<power>" ends the list */
            p->decay_power = (float)strtod(r + 1, &e);
            return (e == r + 1 || *e != '\0') ? -1 : 0;
        }
        if (p->n_steps >= INTERP_MAX_STEPS)
            return -1;
        p->pos[p->n_steps] = lrint(strtod(r, &e));
        if (e == r || *e != ',')
            return -1;
        r = e + 1;
        p->val[++p->n_steps] = (float)strtod(r, &e);
        if (e == r)
            return -1;
        r = e;
    }
    return 0;
}

int nncp_format_interp(char *buf, size_t size, const NNCPInterp *p)
{
    int n = snprintf(buf, size, "%g", p->val[0]);
    for (int i = 0; i < p->n_steps; i++)
        n += snprintf(n < (int)size ? buf + n : NULL, n < (int)size ? size - n : 0, ",%llu,%g",
                      (unsigned long long)p->pos[i], p->val[i + 1]);
    if (p->decay_power != 0)
        n += snprintf(n < (int)size ? buf + n : NULL, n < (int)size ? size - n : 0, ",p%g", p->decay_power);
    return n;
}

/* ---- profiles ---------------------------------------------------------------- */
int nncp_profile(NNCPConfig *c, NNCPFileParams *fp, const char *profile)
{
    memset(fp, 0, sizeof(*fp));
    fp->max_size = -1;
    if (!strcmp(profile, "default")) {
        nncp_config_default(c);
        fp->block_len.val[0] = 500000;
        fp->lr.n_steps = 1;
        fp->lr.val[0] = 3e-4f;
        fp->lr.val[1] = 1e-4f;
        fp->lr.pos[0] = (int64_t)(5e6 / 32);
    } else if (!strcmp(profile, "enwik8") || !strcmp(profile, "enwik9")) {
        const int is8 = !strcmp(profile, "enwik8");
        nncp_config_default(c);
        c->batch_size = 32; c->seg_len = 64; c->n_symbols = 256;
        nncp_parse_interp(&fp->block_len, is8 ? "100000,500000,100000,500000,500000" : "500000");
        nncp_parse_interp(&fp->lr, "1.6e-4,10000,1.0e-4,p0.5");
        c->retrain_len = is8 ? 15000000 : 7500000;
        c->retrain_period = 1;
        c->has_retrain_lr = 1;
        nncp_parse_interp(&c->retrain_lr, "1.6e-4,10000,1.0e-4,p0.5");
        fp->use_bf16 = 1;
        c->n_layer = 20; c->d_model = 1024; c->n_head = 8;
        c->d_key = c->d_value = c->d_model / c->n_head;
        c->d_inner = 3072;
        c->ff_act = NNCP_FF_GEGLU;
        c->d_pos = 320; c->mem_len = 256;
        for (int i = 0; i < c->n_layer; i++)
            c->attn_len[i] = c->mem_len + c->seg_len;
        c->init_range = 0.79f;
        c->tied_w_r = 0;
        c->ln_flags = NNCP_LN_PRE | NNCP_LN_FINAL | NNCP_LN_RMSNORM;
        c->dropout_prob = c->dropout_att_prob = 0.19f;
        c->sgd_opt.u.adam.gradient_clip = 0.05f;
    } else if (!strcmp(profile, "lstm") || !strcmp(profile, "lstm_fast")) {
        const int fast = !strcmp(profile, "lstm_fast");
        nncp_config_default_lstm(c);
        fp->block_len.val[0] = fast ? 100000000 : 500000;
        fp->lr.val[0] = fast ? 1e-2f : 4e-3f;
        if (fast) {
            c->batch_size = 256;
            c->lstm_n_cells = c->lstm_n_cells2 = 512;
        }
    } else {
        return -1;
    }
    c->sgd_opt.lr = fp->lr.val[0];
    return 0;
}

/* ---- header -------------------------------------------------------------------- */
typedef struct {
    uint8_t *w;
    const uint8_t *r;
    size_t pos, cap;
    int bad; /* ran past the end */
} Cur;

static void put8(Cur *c, unsigned v)
{
    if (c->pos < c->cap)
        c->w[c->pos] = (uint8_t)v;
    else
        c->bad = 1;
    c->pos++;
}
static void put16(Cur *c, unsigned v) { put8(c, v >> 8); put8(c, v); }
static void put32(Cur *c, uint32_t v) { put16(c, v >> 16); put16(c, v & 0xffff); }
static void putf(Cur *c, float f) { uint32_t u; memcpy(&u, &f, 4); put32(c, u); }

static unsigned get8(Cur *c)
{
    unsigned v = 0;
    if (c->pos < c->cap)
        v = c->r[c->pos];
    else
        c->bad = 1;
    c->pos++;
    return v;
}
static unsigned get16(Cur *c) { unsigned h = get8(c); return h << 8 | get8(c); }
static uint32_t get32(Cur *c) { uint32_t h = get16(c); return h << 16 | get16(c); }
static float getf(Cur *c) { uint32_t u = get32(c); float f; memcpy(&f, &u, 4); return f; }

static void put_interp(Cur *c, const NNCPInterp *p) /* nncp.c:1297-1306 */
{
    put8(c, p->n_steps);
    for (int i = 0; i <= p->n_steps; i++)
        putf(c, p->val[i]);
    for (int i = 0; i < p->n_steps; i++)
        put32(c, (uint32_t)p->pos[i]);
    putf(c, p->decay_power);
}

static int get_interp(Cur *c, NNCPInterp *p) /* nncp.c:1308-1331 */
{
    memset(p, 0, sizeof(*p));
    p->n_steps = get8(c);
    if (p->n_steps > INTERP_MAX_STEPS)
        return -1;
    for (int i = 0; i <= p->n_steps; i++)
        p->val[i] = getf(c);
    for (int i = 0; i < p->n_steps; i++)
        p->pos[i] = get32(c);
    p->decay_power = getf(c);
    return 0;
}

/* algo 0 and 1 as the reference writes them; this build's RMSProp (algo 16)
   takes the same four fields, and the reference's reader rejects it */
static void put_sgd_opt(Cur *c, const SGDOptParams *p)
{
    put8(c, p->algo);
    if (p->algo != SGD_OPT_BASIC) {
        putf(c, p->u.adam.beta1);
        putf(c, p->u.adam.beta2);
        putf(c, p->u.adam.eps);
        putf(c, p->u.adam.gradient_clip);
    }
}

static int get_sgd_opt(Cur *c, SGDOptParams *p)
{
    p->algo = get8(c);
    if (p->algo == SGD_OPT_BASIC)
        return 0;
    if (p->algo != SGD_OPT_ADAM && p->algo != SGD_OPT_RMSPROP)
        return -1;
    p->u.adam.beta1 = getf(c);
    p->u.adam.beta2 = getf(c);
    p->u.adam.eps = getf(c);
    p->u.adam.gradient_clip = getf(c);
    return 0;
}

static int finite_interp(const NNCPInterp *p)
{
    for (int i = 0; i <= p->n_steps; i++)
        if (!isfinite(p->val[i]))
            return 0;
    return isfinite(p->decay_power);
}

/* A header comes from a file: sizes that would divide by zero, index outside a table or make
   the model constructor give up (which ends the process) are refused here instead. */
static int config_is_sane(const NNCPConfig *c, const NNCPFileParams *fp)
{
    if (c->batch_size < 1 || c->seg_len < 1 || c->n_symbols < 2 || c->n_layer < 1 || c->n_layer > NNCP_N_LAYER_MAX)
        return 0;
    if (!finite_interp(&fp->lr) || !finite_interp(&fp->block_len) || fp->block_len.val[0] < 1.0f)
        return 0;
    if (c->retrain_period < 0 || (c->retrain_period != 0 && c->retrain_len < 1))
        return 0;
    if (c->has_retrain_lr && !finite_interp(&c->retrain_lr))
        return 0;
    if (c->sgd_opt.algo != SGD_OPT_BASIC &&
        !(isfinite(c->sgd_opt.u.adam.beta1) && isfinite(c->sgd_opt.u.adam.beta2) &&
          isfinite(c->sgd_opt.u.adam.eps) && isfinite(c->sgd_opt.u.adam.gradient_clip)))
        return 0;
    if (c->model_type == NNCP_MODEL_TRF) {
        if (c->n_head < 1 || c->d_key < 1 || c->d_value < 1 || c->d_inner < 1 ||
            (c->use_w_r && c->d_pos < 1))
            return 0;
        for (int i = 0; i < c->n_layer; i++)
            if (c->attn_len[i] < 1)
                return 0;
        if (c->ff_act > NNCP_FF_GATED_SILU ||
            (c->ln_flags & ~(NNCP_LN_POST | NNCP_LN_PRE | NNCP_LN_FINAL | NNCP_LN_COEF | NNCP_LN_RMSNORM)))
            return 0;
        if (!isfinite(c->init_range) || !isfinite(c->embed_mult) || !isfinite(c->dropout_prob) ||
            !isfinite(c->dropout_att_prob) || c->dropout_prob < 0 || c->dropout_prob >= 1 ||
            c->dropout_att_prob < 0 || c->dropout_att_prob >= 1)
            return 0;
    } else {
        if (c->lstm_n_cells < 1 || c->lstm_n_embed_out < 1 || c->lstm_n_embed_out > c->n_layer ||
            !isfinite(c->lstm_forget_bias))
            return 0;
    }
    return 1;
}

size_t nncp_header_write(uint8_t *buf, size_t cap, const NNCPConfig *c, const NNCPFileParams *fp)
{
    Cur k = { buf, NULL, 0, cap, 0 };
    put32(&k, FILE_MAGIC);
    put16(&k, FILE_VERSION);
    put8(&k, c->use_device != 0);
    put8(&k, fp->use_bf16 == 2 ? 2 : fp->use_bf16 != 0);
    put16(&k, c->batch_size);
    put16(&k, c->seg_len);
    put16(&k, c->n_symbols);
    put32(&k, c->seed);
    put_interp(&k, &fp->lr);
    put_interp(&k, &fp->block_len);
    put32(&k, (uint32_t)c->retrain_period);
    if (c->retrain_period != 0) {
        put32(&k, (uint32_t)c->retrain_len);
        put8(&k, c->has_retrain_lr != 0);
        if (c->has_retrain_lr)
            put_interp(&k, &c->retrain_lr);
    }
    put8(&k, c->model_type); /* model_id: trf 0 (nncp.c:1546), lstm 1 (nncp.c:2314) */
    if (c->model_type == NNCP_MODEL_TRF) {
        put8(&k, c->n_layer);
        put8(&k, c->n_head);
        put16(&k, c->d_key);
        put16(&k, c->d_value);
        put16(&k, c->d_inner);
        put16(&k, c->d_pos);
        put16(&k, c->mem_len);
        for (int i = 0; i < c->n_layer; i++)
            put16(&k, c->attn_len[i]);
        put8(&k, 0); /* tied_embed: not in this build */
        put8(&k, c->use_bias);
        put8(&k, c->use_w_r);
        put8(&k, c->tied_w_r);
        put8(&k, c->tied_b_r);
        put8(&k, c->query_bias);
        put8(&k, 0); /* rotary_pos_embed: not in this build */
        put8(&k, c->ln_flags);
        putf(&k, c->init_range);
        putf(&k, c->embed_mult);
        put8(&k, c->ff_act);
        put_sgd_opt(&k, &c->sgd_opt);
        if (c->retrain_period != 0) {
            putf(&k, c->dropout_prob);
            putf(&k, c->dropout_att_prob);
        }
        put8(&k, 0); /* use_sparse_grad */
    } else {
        put8(&k, c->lstm_type);
        put8(&k, c->n_layer);
        put8(&k, c->lstm_n_embed_out);
        put16(&k, c->lstm_n_cells);
        put16(&k, c->seg_len); /* n_states */
        put8(&k, (c->lstm_use_layer_norm != 0) | (c->lstm_full_connect != 0) << 1);
        put_sgd_opt(&k, &c->sgd_opt);
        putf(&k, 0.0f); /* dropout_prob: the reference's LSTM never applies it */
        putf(&k, c->lstm_forget_bias);
        put8(&k, 0); /* use_sparse_grad */
    }
    return k.bad ? 0 : k.pos;
}

int nncp_header_read(const uint8_t *buf, size_t len, NNCPConfig *c, NNCPFileParams *fp, size_t *used)
{
    Cur k = { NULL, buf, 0, len, 0 };
    memset(c, 0, sizeof(*c));
    memset(fp, 0, sizeof(*fp));
    fp->max_size = -1;
    c->nb_threads = 1;
    if (get32(&k) != FILE_MAGIC || get16(&k) != FILE_VERSION || k.bad)
        return -1;
    c->use_device = get8(&k);
    fp->use_bf16 = get8(&k);
    c->batch_size = get16(&k);
    c->seg_len = get16(&k);
    c->n_symbols = get16(&k);
    c->seed = get32(&k);
    if (get_interp(&k, &fp->lr) || get_interp(&k, &fp->block_len))
        return -1;
    c->retrain_period = (int)get32(&k);
    if (c->retrain_period != 0) {
        c->retrain_len = (int)get32(&k);
        c->has_retrain_lr = get8(&k);
        if (c->has_retrain_lr && get_interp(&k, &c->retrain_lr))
            return -1;
    }
    c->model_type = get8(&k);
    if (c->model_type == NNCP_MODEL_TRF) {
        c->n_layer = get8(&k);
        c->n_head = get8(&k);
        c->d_key = get16(&k);
        c->d_model = c->d_key * c->n_head;
        c->d_value = get16(&k);
        c->d_inner = get16(&k);
        c->d_pos = get16(&k);
        c->mem_len = get16(&k);
        if (c->n_layer > NNCP_N_LAYER_MAX)
            return -1;
        for (int i = 0; i < c->n_layer; i++)
            c->attn_len[i] = get16(&k);
        if (get8(&k) != 0) /* tied_embed */
            return -2;
        c->use_bias = get8(&k);
        c->use_w_r = get8(&k);
        c->tied_w_r = get8(&k);
        c->tied_b_r = get8(&k);
        c->query_bias = get8(&k);
        if (get8(&k) != 0) /* rotary_pos_embed */
            return -2;
        c->ln_flags = get8(&k);
        c->init_range = getf(&k);
        c->embed_mult = getf(&k);
        c->ff_act = get8(&k);
        if (get_sgd_opt(&k, &c->sgd_opt))
            return -1;
        if (c->retrain_period != 0) {
            c->dropout_prob = getf(&k);
            c->dropout_att_prob = getf(&k);
        }
        get8(&k); /* use_sparse_grad: a backward-pass hint, same results */
    } else if (c->model_type == NNCP_MODEL_LSTM) {
        int flags, n_states;
        c->lstm_type = get8(&k);
        c->n_layer = get8(&k);
        c->lstm_n_embed_out = get8(&k);
        c->lstm_n_cells = c->lstm_n_cells2 = get16(&k);
        n_states = get16(&k);
        flags = get8(&k);
        c->lstm_use_layer_norm = flags & 1;
        c->lstm_full_connect = (flags >> 1) & 1;
        if (get_sgd_opt(&k, &c->sgd_opt))
            return -1;
        getf(&k); /* dropout_prob, unused by the reference's LSTM */
        c->lstm_forget_bias = getf(&k);
        get8(&k);
        if (n_states != c->seg_len || c->lstm_type > NNCP_LSTM_TIED)
            return -2;
    } else {
        return -1;
    }
    if (k.bad || !config_is_sane(c, fp))
        return -1;
    c->sgd_opt.lr = fp->lr.val[0];
    if (used)
        *used = k.pos;
    return 0;
}

/* ---- file loops ------------------------------------------------------------------ */
int nncp_block_len(const NNCPConfig *c, const NNCPInterp *sched, int64_t file_pos, int64_t remaining)
{
    const int unit = c->seg_len * c->batch_size;              /* nncp.c:3452-3457 */
    int n = (int)lrintf(nncp_interp(sched, file_pos));
    n = (n / unit > 1 ? n / unit : 1) * unit;
    return n > remaining ? (int)remaining : n;
}

typedef struct {
    FILE *f;
    int failed;
} FileSink;

static void file_sink(void *opaque, const uint8_t *buf, size_t n)
{
    FileSink *k = opaque;
    if (!k->failed && fwrite(buf, 1, n, k->f) != n)
        k->failed = 1;
}

static void add_stats(NNCPStats *to, const NNCPStats *from)
{
    to->n_symbols += from->n_symbols; to->n_steps += from->n_steps; to->loss_bits += from->loss_bits;
    to->t_eval += from->t_eval; to->t_code += from->t_code; to->t_grad += from->t_grad; to->t_update += from->t_update;
}

static int fail(const char *what, const char *name)
{
    fprintf(stderr, "nncp_host: %s%s%s\n", what, name ? ": " : "", name ? name : "");
    return -1;
}

static NNCPModel *model_for_file(const NNCPConfig *c, const NNCPFileParams *fp)
{
    NNCPConfig cfg = *c;
    if (fp->use_bf16 == 2)
        cfg.param_bf16 = 1;
    NNCPModel *s = nncp_model_new(&cfg);
    if (fp->use_bf16)
        nc_set_matmul_bf16(nncp_model_context(s), 1);
    return s;
}

int nncp_encode_file(const char *in_name, const char *out_name, const NNCPConfig *c, const NNCPFileParams *fp,
                     NNCPStats *st, NNCPStats *retrain_st)
{
    const int symb_shift = c->n_symbols > 256;                 /* nncp.c:3386-3391 */
    uint8_t head[1024], *arith_buf;
    uint16_t *block = NULL;
    int block_cap = 0;
    int64_t file_len, pos = 0;
    NNCPPutBit pb;
    NNCPStats dummy = { 0 }, dummy2 = { 0 };
    FILE *f = fopen(in_name, "rb"), *fo;
    size_t n;
    if (!f)
        return fail("cannot open", in_name);
    if (!(fo = fopen(out_name, "wb"))) {
        fclose(f);
        return fail("cannot create", out_name);
    }
    if (!st) st = &dummy;
    if (!retrain_st) retrain_st = &dummy2;
    n = nncp_header_write(head, sizeof(head) - 5, c, fp);
    if (n == 0) {
        fclose(f); fclose(fo);
        return fail("header does not fit", out_name);
    }
    head[n++] = (uint8_t)((fp->mode & 7) << 1 | (c->fused != 0) << 4); /* bit 0: no preprocessing */
    fseeko(f, 0, SEEK_END);
    file_len = ftello(f) >> symb_shift;
    fseeko(f, 0, SEEK_SET);
    if (fp->max_size >= 0 && file_len > fp->max_size)
        file_len = fp->max_size;
    if (file_len > 0xffffffffLL) {
        fclose(f); fclose(fo);
        return fail("input longer than the 32-bit length field of the container", in_name);
    }
    head[n++] = (uint8_t)(file_len >> 24); head[n++] = (uint8_t)(file_len >> 16);
    head[n++] = (uint8_t)(file_len >> 8); head[n++] = (uint8_t)file_len;
    FileSink sink = { fo, fwrite(head, 1, n, fo) != n };

    arith_buf = malloc(ARITH_BUF_LEN);
    nncp_put_bit_init(&pb, arith_buf, ARITH_BUF_LEN);
    nncp_put_bit_set_sink(&pb, file_sink, &sink);
    NNCPModel *s = model_for_file(c, fp);
    int rc = 0;
    while (pos < file_len) {
        const int len = nncp_block_len(c, &fp->block_len, pos, file_len - pos);
        NNCPStats bs = { 0 };
        if (len > block_cap) {
            free(block);
            block = malloc(sizeof(block[0]) * (size_t)len);
            block_cap = len;
        }
        for (int i = 0; i < len; i++) {                         /* read_block, nncp.c:3153-3172 */
            int v = fgetc(f);
            if (symb_shift && v >= 0) {
                int lo = fgetc(f);
                v = lo < 0 ? -1 : v << 8 | lo;
            }
            if (v < 0) {
                rc = fail("read error", in_name);
                break;
            }
            if (v >= c->n_symbols) {
                rc = fail("symbol outside the alphabet", in_name);
                break;
            }
            block[i] = (uint16_t)v;
        }
        if (rc)
            break;
        nncp_process_block(s, &pb, NULL, block, len, 0, fp->mode, &fp->lr, &bs);
        add_stats(st, &bs);
        pos += len;
        if (pos >= file_len)
            break;
        memset(&bs, 0, sizeof(bs));
        nncp_retrain_block(s, block, len, &fp->lr, &bs);
        add_stats(retrain_st, &bs);
    }
    nncp_put_bit_flush(&pb);
    nc_prof_dump(); /* nncp.c:3505 */
    nncp_model_free(s);
    free(block);
    free(arith_buf);
    if (fclose(fo) != 0 || sink.failed)
        rc = fail("write error", out_name);
    fclose(f);
    return rc;
}

int nncp_decode_file(const char *in_name, const char *out_name, int use_device, int nb_threads,
                     NNCPStats *st, NNCPStats *retrain_st)
{
    NNCPConfig cfg;
    NNCPFileParams fp;
    NNCPStats dummy = { 0 }, dummy2 = { 0 };
    NNCPGetBit gb;
    uint8_t *data;
    uint16_t *block = NULL;
    int block_cap = 0, rc, flags;
    int64_t size, file_len, pos = 0;
    size_t used;
    FILE *f = fopen(in_name, "rb"), *fo;
    if (!f)
        return fail("cannot open", in_name);
    fseeko(f, 0, SEEK_END);
    size = ftello(f);
    fseeko(f, 0, SEEK_SET);
    data = malloc(size > 0 ? (size_t)size : 1);
    if (fread(data, 1, (size_t)size, f) != (size_t)size) {
        fclose(f); free(data);
        return fail("read error", in_name);
    }
    fclose(f);
    rc = nncp_header_read(data, (size_t)size, &cfg, &fp, &used);
    if (rc == 0 && used + 5 > (size_t)size)
        rc = -1;
    if (rc) {
        free(data);
        return fail(rc == -2 ? "the file uses a model option this build does not have "
                               "(tied_embed, rot_pos, GRU, n_states != seg_len)" : "invalid file header", in_name);
    }
    flags = data[used++];
    if (flags & 1) {
        free(data);
        return fail("the file was written with the dictionary preprocessor, which is not part of this build", in_name);
    }
    fp.mode = (flags >> 1) & 7;
    cfg.fused = (flags >> 4) & 1;
    cfg.use_device = use_device; /* as nncp.c:3557-3565: the decoder's own choice wins */
    cfg.nb_threads = nb_threads > 0 ? nb_threads : 1;
    file_len = (int64_t)data[used] << 24 | data[used + 1] << 16 | data[used + 2] << 8 | data[used + 3];
    used += 4;
    if (!(fo = fopen(out_name, "wb"))) {
        free(data);
        return fail("cannot create", out_name);
    }
    if (!st) st = &dummy;
    if (!retrain_st) retrain_st = &dummy2;
    nncp_get_bit_init(&gb, data + used, (size_t)size - used);
    NNCPModel *s = model_for_file(&cfg, &fp);
    const int symb_shift = cfg.n_symbols > 256;
    while (pos < file_len) {
        const int len = nncp_block_len(&cfg, &fp.block_len, pos, file_len - pos);
        NNCPStats bs = { 0 };
        if (len > block_cap) {
            free(block);
            block = malloc(sizeof(block[0]) * (size_t)len);
            block_cap = len;
        }
        nncp_process_block(s, NULL, &gb, block, len, 1, fp.mode, &fp.lr, &bs);
        add_stats(st, &bs);
        for (int i = 0; i < len; i++) {                         /* write_block, nncp.c:3174-3183 */
            if (symb_shift)
                fputc(block[i] >> 8, fo);
            fputc(block[i] & 0xff, fo);
        }
        fflush(fo);
        pos += len;
        if (pos >= file_len)
            break;
        memset(&bs, 0, sizeof(bs));
        nncp_retrain_block(s, block, len, &fp.lr, &bs);
        add_stats(retrain_st, &bs);
    }
    nc_prof_dump(); /* nncp.c:3676 */
    nncp_model_free(s);
    free(block);
    free(data);
    rc = 0;
    if (fclose(fo) != 0)
        rc = fail("write error", out_name);
    return rc;
}
