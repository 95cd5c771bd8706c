/*
 * Block loop of the compressor / decompressor: process_block of the reference
 * (nncp.c:2968-3147) restated over in-memory buffers.  A block of block_len
 * symbols is cut into B contiguous sub-streams (the first block_len % B one
 * symbol longer, nncp.c:2943-2965); each step codes one segment of T symbols
 * of every stream from the model's probabilities, then trains on it; a tail
 * shorter than T is coded without training.
 *
 * Modes (nncp_host.h): NNCP_MODE_SEQ_EVAL evaluates one timestep at a time on
 * both sides, exactly as `nncp c` / `nncp d`.  NNCP_MODE_SEGMENT evaluates the
 * whole segment at once when encoding (`nncp --encode_only`); the decoder then
 * replays that same whole-segment evaluation once per timestep with the
 * symbols known so far.  Column t of the evaluation depends only on inputs
 * 0..t (causal mask; masked terms contribute exact zeros), so the replay
 * reproduces the encoder's probabilities bit for bit.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include "../../include/nncp_host.h"

static void die_stream(const char *msg)
{
    fprintf(stderr, "nncp_host: %s\n", msg);
    abort();
}

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return ts.tv_sec + 1e-9 * ts.tv_nsec;
}

typedef struct {
    const uint16_t *rbuf;
    uint16_t *wbuf;
    int stride, rem;
} BlockView;

static int get_symb(const BlockView *v, int stream, int pos) /* nncp.c:2945-2954 */
{
    int e = stream < v->rem;
    if (pos < 0 || pos >= v->stride + e)
        return 0;
    return v->rbuf[v->stride * stream + (v->rem < stream ? v->rem : stream) + pos];
}

static void put_symb(BlockView *v, int stream, int pos, int c) /* nncp.c:2956-2965 */
{
    int e = stream < v->rem;
    if (pos < 0 || pos >= v->stride + e)
        abort();
    v->wbuf[v->stride * stream + (v->rem < stream ? v->rem : stream) + pos] = (uint16_t)c;
}

typedef struct {
    NNCPModel *s;
    const NNCPModelClass *cls;
    NNCPPutBit *pb;
    NNCPGetBit *gb;
    BlockView view;
    int is_decode, coder, n_symbols, B, step_decode;
    NNCPStats *st;
} Coder;

/* probabilities (or CDF rows) of one evaluation on the host: column index
   col = t*B + stream for a segment evaluation, stream for a timestep */
typedef struct {
    NCTensor *host;
    const float *prob;
    const uint16_t *cdf;
    const uint16_t *path; /* encoder, whole segment: per column the CDF entries its symbol's walk reads */
    size_t stride;
} HostDist;

/* `symbols` (consumed; may be NULL): the symbol of every column, one I32 each on the model's
   device, known to an encoder before it codes.  With them only the CDF entries that the coder
   will read cross to the host. */
static HostDist fetch_dist(Coder *c, NCTensor *output, NCTensor *symbols)
{
    HostDist d;
    memset(&d, 0, sizeof(d));
    if (c->coder == NNCP_CODER_CDF16) {
        NCTensor *logits = c->cls->last_logits(c->s);
        size_t dims[NC_N_DIMS_MAX], cols = 1;
        int nd = nc_tensor_get_dims(logits, dims);
        for (int i = 1; i < nd; i++) cols *= dims[i];
        nc_free_tensor(output);
        if (symbols) { /* already on the model's device */
            NCDevice *dev = nc_get_tensor_device(logits);
            d.host = nc_soft_max_cdf16_path_to_host(nc_dup_tensor(logits), symbols);
            nc_synchronize(dev); /* the one wait of the evaluation: these entries, and the loss if it was queued */
            d.path = nc_tensor_get_ptr(d.host, &d.stride);
            return d;
        }
        if (cols <= 64) { /* a timestep's rows: the kernel writes them to the host itself */
            NCDevice *dev = nc_get_tensor_device(logits);
            d.host = nc_soft_max_cdf16_to_host(nc_dup_tensor(logits));
            nc_synchronize(dev);
        } else {
            d.host = nc_tensor_to_cpu_device(nc_soft_max_cdf16(nc_dup_tensor(logits)));
        }
        d.cdf = nc_tensor_get_ptr(d.host, &d.stride);
    } else {
        d.host = nc_tensor_to_cpu_device(output);
        d.prob = nc_tensor_get_ptr(d.host, &d.stride);
    }
    return d;
}

/* codes (or decodes) the symbol of `stream` at block position pos */
static int code_symbol(Coder *c, const HostDist *d, size_t col, int stream, int pos)
{
    int sym;
    prof_start(PROF_WRITE_SYM); /* nncp.c:3007, 3039 */
    if (!c->is_decode) {
        sym = get_symb(&c->view, stream, pos);
        if (d->path) nncp_write_sym_cdf_path(c->pb, d->path + col * d->stride, c->n_symbols, sym);
        else if (d->cdf) nncp_write_sym_cdf(c->pb, d->cdf + col * d->stride, c->n_symbols, sym);
        else nncp_write_sym(c->pb, d->prob + col * d->stride, c->n_symbols, sym);
    } else {
        if (d->cdf) sym = nncp_read_sym_cdf(c->gb, d->cdf + col * d->stride, c->n_symbols);
        else sym = nncp_read_sym(c->gb, d->prob + col * d->stride, c->n_symbols);
        put_symb(&c->view, stream, pos, sym);
    }
    prof_end(PROF_WRITE_SYM); /* nncp.c:3018, 3041 */
    return sym;
}

static int symbol_is_coded(int t, int stream, int len2, int rem, int full)
{
    return full || t < len2 || (t == len2 && stream < rem); /* nncp.c:3099-3100 */
}

/* The encoder's whole-segment evaluation in two halves.  The first fills the input (and the
   training targets: the encoder knows its symbols before it codes them), evaluates the
   segment and brings the distributions to the host; the second feeds them to the
   arithmetic coder.  Between the two a caller may queue the training step, whose kernels
   then run while the host codes (nncp.c:3024-3050 does the same work in sequence: eval,
   code, train; the bytes and the weights do not depend on the order of the last two). */
static HostDist encode_segment_eval(Coder *c, int idx, int n_t, int len2, int full,
                                    NCTensor *input, NCTensor *expected)
{
    int B = c->B;
    NCTensor *symbols = NULL;
    if (c->coder == NNCP_CODER_CDF16) { /* (B, T) like input: column t*B + b, zero where nothing is coded */
        size_t dims[2];
        nc_tensor_get_dims(input, dims);
        symbols = nc_new_tensor_2d(nc_get_tensor_device(input), NC_TYPE_I32, dims[0], dims[1]);
    }
    for (int t = 0; t < n_t; t++)
        for (int b = 0; b < B; b++) {
            nc_set1_i32_2d(input, b, t, get_symb(&c->view, b, idx + t - 1));
            if (!symbol_is_coded(t, b, len2, c->view.rem, full))
                continue;
            if (expected) nc_set1_i32_2d(expected, b, t, get_symb(&c->view, b, idx + t));
            if (symbols) nc_set1_i32_2d(symbols, b, t, get_symb(&c->view, b, idx + t));
        }
    double t0 = now_s();
    if (symbols)
        symbols = nc_tensor_to_device(symbols, nncp_model_device(c->s));
    NCTensor *out = c->cls->eval(c->s, -1, input);
    /* a full segment that training follows: its expected symbols are these, so the loss is queued
       behind the evaluation now and arrives with the CDF entries */
    if (symbols && expected && full && c->cls->queue_loss)
        c->cls->queue_loss(c->s, nc_dup_tensor(symbols));
    HostDist d = fetch_dist(c, out, symbols);
    c->st->t_eval += now_s() - t0;
    return d;
}

static void encode_segment_emit(Coder *c, HostDist *d, int idx, int n_t, int len2, int full)
{
    int B = c->B;
    double t0 = now_s();
    for (int t = 0; t < n_t; t++)
        for (int b = 0; b < B; b++)
            if (symbol_is_coded(t, b, len2, c->view.rem, full))
                code_symbol(c, d, (size_t)t * B + b, b, idx + t);
    c->st->t_code += now_s() - t0;
    nc_free_tensor(d->host);
    d->host = NULL;
}

/* One segment starting at block position idx: n_t timesteps are coded (T for a
   full segment, fewer in the tail).  Fills `expected` when training follows. */
static void code_segment(Coder *c, int mode, int idx, int n_t, int len2, int full,
                         NCTensor *input, NCTensor *expected)
{
    NNCPModel *s = c->s;
    int B = c->B;
    double t0;
    if (mode == NNCP_MODE_SEGMENT && !c->is_decode) {
        /* nncp.c:3024-3046 */
        HostDist d = encode_segment_eval(c, idx, n_t, len2, full, input, expected);
        encode_segment_emit(c, &d, idx, n_t, len2, full);
        return;
    }
    if (mode == NNCP_MODE_SEGMENT && c->step_decode) {
        /* decoder, one token column per timestep against the K/V caches */
        trf_step_begin(s);
        trf_step_logits_only(s, c->coder == NNCP_CODER_CDF16); /* the CDFs come from the logits: no softmax launch */
        for (int t = 0; t < n_t; t++) {
            for (int b = 0; b < B; b++)
                nc_set1_i32_2d(input, b, t, get_symb(&c->view, b, idx + t - 1));
            t0 = now_s();
            NCTensor *out = trf_eval_step(s, t, input);
            HostDist d = fetch_dist(c, out, NULL);
            c->st->t_eval += now_s() - t0;
            t0 = now_s();
            for (int b = 0; b < B; b++)
                if (symbol_is_coded(t, b, len2, c->view.rem, full)) {
                    int sym = code_symbol(c, &d, (size_t)b, b, idx + t);
                    if (expected) nc_set1_i32_2d(expected, b, t, sym);
                }
            c->st->t_code += now_s() - t0;
            nc_free_tensor(d.host);
        }
        trf_step_end(s);
        if (expected) { /* the graph the encoder differentiated: one whole-segment evaluation */
            t0 = now_s();
            nc_free_tensor(c->cls->eval(s, -1, input));
            c->st->t_eval += now_s() - t0;
        }
        return;
    }
    for (int t = 0; t < n_t; t++) {
        /* nncp.c:2996-3022 (and 3087-3114 for the tail) */
        for (int b = 0; b < B; b++)
            nc_set1_i32_2d(input, b, t, get_symb(&c->view, b, idx + t - 1));
        t0 = now_s();
        NCTensor *out = c->cls->eval(s, mode == NNCP_MODE_SEGMENT ? -1 : t, input);
        HostDist d = fetch_dist(c, out, NULL);
        c->st->t_eval += now_s() - t0;
        t0 = now_s();
        for (int b = 0; b < B; b++)
            if (symbol_is_coded(t, b, len2, c->view.rem, full)) {
                size_t col = mode == NNCP_MODE_SEGMENT ? (size_t)t * B + b : (size_t)b;
                int sym = code_symbol(c, &d, col, b, idx + t);
                if (expected) nc_set1_i32_2d(expected, b, t, sym);
            }
        c->st->t_code += now_s() - t0;
        nc_free_tensor(d.host);
        /* replayed segment evaluations are discarded, except the last one of a
           trained segment, whose graph the gradient needs */
        if (mode == NNCP_MODE_SEGMENT && !(expected && t == n_t - 1))
            c->cls->eval_discard(s);
    }
    /* decoder in segment mode: the last replay was built once every input of
       the segment was known (the last symbol is a target only), so its graph
       is the one the encoder differentiated */
}

void nncp_process_block(NNCPModel *s, NNCPPutBit *pb, NNCPGetBit *gb, uint16_t *block_buf,
                        int block_len, int is_decode, int mode_flags, const NNCPInterp *lr,
                        NNCPStats *st)
{
    NNCPStats local;
    Coder c;
    int mode = mode_flags & 1;
    memset(&local, 0, sizeof(local));
    memset(&c, 0, sizeof(c));
    c.s = s; c.cls = nncp_model_class(s); c.pb = pb; c.gb = gb; c.is_decode = is_decode;
    c.coder = mode_flags & NNCP_CODER_CDF16;
    if (mode_flags & NNCP_MODE_STEP_DECODE) {
        if (mode != NNCP_MODE_SEGMENT)
            die_stream("NNCP_MODE_STEP_DECODE goes with NNCP_MODE_SEGMENT");
        if (nncp_model_config(s)->model_type != NNCP_MODEL_TRF)
            die_stream("NNCP_MODE_STEP_DECODE is a path of the Transformer model class");
        /* both sides: products whose columns do not depend on how many are computed together */
        nc_set_matmul_width_invariant(nncp_model_context(s), 1);
        c.step_decode = is_decode;
    }
    c.st = st ? st : &local;

    const NNCPConfig *cfg = nncp_model_config(s);
    int B = cfg->batch_size, T = cfg->seg_len;
    /* symbols index the embedding table and the probability columns on the device, where
       nothing checks them: an encoder refuses a block that holds one outside the alphabet
       (a decoder only ever produces symbols below n_symbols) */
    if (!is_decode)
        for (int i = 0; i < block_len; i++)
            if (block_buf[i] >= cfg->n_symbols)
                die_stream("a symbol of the block lies outside the model's alphabet");
    c.n_symbols = cfg->n_symbols;
    c.B = B;
    c.view.rbuf = block_buf; c.view.wbuf = block_buf;
    c.view.stride = block_len / B;
    c.view.rem = block_len % B;

    NCDevice *cpu = nncp_model_cpu_device(s);
    NCTensor *input = nc_new_tensor_2d(cpu, NC_TYPE_I32, B, T);
    NCTensor *expected = nc_new_tensor_2d(cpu, NC_TYPE_I32, B, T);
    c.cls->reset(s); /* nncp.c:2988 */

    int idx = 0;
    const int overlap = mode == NNCP_MODE_SEGMENT && !is_decode; /* code while the training kernels run */
    while (idx + T <= c.view.stride) { /* nncp.c:2993 */
        HostDist pending = { 0 };
        prof_start(PROF_TOTAL); /* nncp.c:2994 */
        if (overlap)
            pending = encode_segment_eval(&c, idx, T, T, 1, input, expected);
        else
            code_segment(&c, mode, idx, T, T, 1, input, expected);
        float rate = nncp_interp(lr, nncp_model_train_step(s)); /* nncp.c:3048-3050 */
        c.cls->set_lr(s, rate);
        double t0 = now_s();
        float loss = c.cls->eval_gradient(s, expected);
        c.st->t_grad += now_s() - t0;
        t0 = now_s();
        c.cls->update(s);
        c.st->t_update += now_s() - t0;
        if (overlap)
            encode_segment_emit(&c, &pending, idx, T, T, 1);
        c.st->loss_bits -= loss / log(2.0);
        c.st->n_steps++;
        c.st->n_symbols += (int64_t)T * B;
        idx += T;
        prof_end_ops(PROF_TOTAL, T * B); /* nncp.c:3056 */
    }
    int len2 = c.view.stride - idx, len1 = len2 + (c.view.rem != 0); /* nncp.c:3076-3077 */
    if (len1 > 0) {
        for (int t = 0; t < T; t++)
            for (int b = 0; b < B; b++)
                nc_set1_i32_2d(input, b, t, 0);
        code_segment(&c, mode, idx, len1, len2, 0, input, NULL);
        c.cls->eval_end(s);
        c.st->n_symbols += (int64_t)len2 * B + c.view.rem;
    }
    nc_free_tensor(expected);
    nc_free_tensor(input);
}

int nncp_fifo_symbol(const uint16_t *buf, int rpos, int size, int idx) /* nncp.c:2811-2819 */
{
    if (idx < 0)
        return 0;
    return buf[(rpos + idx) % size];
}

void nncp_retrain_block(NNCPModel *s, const uint16_t *block_buf, int block_len,
                        const NNCPInterp *lr, NNCPStats *st)
{
    const NNCPConfig *cfg = nncp_model_config(s);
    NNCPRetrainState *r = nncp_model_retrain_state(s);
    const NNCPModelClass *cls = nncp_model_class(s);
    const int B = cfg->batch_size, T = cfg->seg_len;
    if (cfg->retrain_period == 0)
        return;
    if (cfg->retrain_len <= 0)
        die_stream("retrain needs a buffer (cfg.retrain_len > 0)");
    if (!r->buf)
        r->buf = nc_mallocz(sizeof(r->buf[0]) * cfg->retrain_len);
    /* append the block, overwriting the oldest symbols (nncp.c:2837-2849) */
    for (int pos = 0; pos < block_len;) {
        int l = cfg->retrain_len - r->buf_pos;
        if (l > block_len - pos)
            l = block_len - pos;
        memcpy(r->buf + r->buf_pos, block_buf + pos, sizeof(r->buf[0]) * l);
        r->buf_pos += l;
        if (r->buf_pos == cfg->retrain_len)
            r->buf_pos = 0;
        pos += l;
    }
    r->buf_len = r->buf_len + block_len < cfg->retrain_len ? r->buf_len + block_len : cfg->retrain_len;
    r->pos += block_len;
    if (r->pos < cfg->retrain_period)
        return;
    r->pos = 0;
    const int stride = r->buf_len / B; /* nncp.c:2858 */
    if (stride == 0)
        return;

    NCDevice *cpu = nncp_model_cpu_device(s);
    NCTensor *input = nc_new_tensor_2d(cpu, NC_TYPE_I32, B, T);
    NCTensor *expected = nc_new_tensor_2d(cpu, NC_TYPE_I32, B, T);
    cls->set_retrain(s, 1);
    cls->reset(s);
    /* nncp.c:2882: whole segments while (seg_len + first) * B symbols are held */
    for (int first = 0; r->buf_len >= (T + first) * B; first += T) {
        for (int t = 0; t < T; t++)
            for (int b = 0; b < B; b++) {
                nc_set1_i32_2d(input, b, t, nncp_fifo_symbol(r->buf, r->buf_pos, r->buf_len, stride * b + first + t - 1));
                nc_set1_i32_2d(expected, b, t, nncp_fifo_symbol(r->buf, r->buf_pos, r->buf_len, stride * b + first + t));
            }
        nc_free_tensor(cls->eval(s, -1, input));
        const int64_t step = nncp_model_train_step(s);
        cls->set_lr(s, cfg->has_retrain_lr ? nncp_interp(&cfg->retrain_lr, r->train_step) : nncp_interp(lr, step));
        float loss = cls->eval_gradient(s, expected);
        cls->update(s); /* advances the model's step counter */
        if (cfg->has_retrain_lr) { /* nncp.c:2914-2918 */
            nncp_model_set_train_step(s, step);
            r->train_step++;
        }
        if (st) {
            st->loss_bits -= loss / log(2.0);
            st->n_steps++;
            st->n_symbols += (int64_t)T * B;
        }
    }
    nc_free_tensor(expected);
    nc_free_tensor(input);
    cls->set_retrain(s, 0);
}

size_t nncp_compress(NNCPModel *s, const uint16_t *syms, int n, uint8_t *out, size_t cap,
                     int mode, const NNCPInterp *lr, NNCPStats *st)
{
    NNCPPutBit pb;
    uint16_t *buf = nc_malloc(sizeof(uint16_t) * (n > 0 ? n : 1));
    memcpy(buf, syms, sizeof(uint16_t) * n);
    nncp_put_bit_init(&pb, out, cap);
    nncp_process_block(s, &pb, NULL, buf, n, 0, mode, lr, st);
    size_t len = nncp_put_bit_flush(&pb);
    nc_free(buf);
    if (pb.overflow) {
        fprintf(stderr, "nncp_compress: output buffer too small (%zu needed)\n", len);
        abort();
    }
    return len;
}

void nncp_decompress(NNCPModel *s, const uint8_t *in, size_t len, uint16_t *syms, int n,
                     int mode, const NNCPInterp *lr, NNCPStats *st)
{
    NNCPGetBit gb;
    nncp_get_bit_init(&gb, in, len);
    nncp_process_block(s, NULL, &gb, syms, n, 1, mode, lr, st);
}
