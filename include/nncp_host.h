/*
 * nncp_host.h - host side of the train+code step, above the libnc ABI.
 *
 * A C mirror of the part of nncp.c that drives libnc for the Transformer-XL
 * model: the NNCPModelClass entry points of the `trf` model (nncp.c:49-69,
 * 1544-1562) with the same names, argument meaning and ownership rules, the
 * block loop of process_block (nncp.c:2968-3147), the symbol coder of
 * cp_utils.c:299-349 and the binary range coder of arith.c.  It links against
 * any library exporting nc_api.h (+ nc_ext.h when cfg.fused is set), so the
 * same code runs on libnc_hip.so (product) and on the CPU checker (tests).
 */
#ifndef NNCP_HOST_H
#define NNCP_HOST_H

#include "nc_api.h"
#include "nc_ext.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- binary range coder, bit-compatible with arith.c ----------------------- */
#define NNCP_PROB_BITS 15 /* arith.h:27 */

typedef struct { /* arith.h:32-43, in-memory output */
    uint32_t range, low;
    uint8_t current_byte;
    uint32_t n_bytes;
    uint8_t *buf;
    size_t buf_size, idx;
    int overflow;
    /* optional: a full buffer is handed to sink and reused (the write_func of
       arith.c:43); without one, bytes past buf_size are dropped and overflow is set */
    void (*sink)(void *opaque, const uint8_t *buf, size_t n);
    void *sink_opaque;
    size_t n_flushed; /* bytes handed to sink so far */
} NNCPPutBit;

typedef struct { /* arith.h:50-61, in-memory input, zero padded past the end */
    const uint8_t *buf;
    size_t buf_len, idx;
    uint32_t low, range;
} NNCPGetBit;

void nncp_put_bit_init(NNCPPutBit *s, uint8_t *buf, size_t buf_size);  /* arith.c:43 */
void nncp_put_bit_set_sink(NNCPPutBit *s, void (*sink)(void *, const uint8_t *, size_t), void *opaque);
void nncp_put_bit(NNCPPutBit *s, int prob0, int bit);                  /* arith.c:122 */
size_t nncp_put_bit_flush(NNCPPutBit *s);        /* arith.c:164; returns bytes written (all of
                                                    them already handed to the sink, if one is set) */
void nncp_get_bit_init(NNCPGetBit *s, const uint8_t *buf, size_t len); /* arith.c:233 */
int nncp_get_bit(NNCPGetBit *s, int prob0);                            /* arith.c:259 */

/* ---- symbol coders ------------------------------------------------------------ */
/* float probabilities, balanced binary decomposition (cp_utils.c:299-349) */
void nncp_write_sym(NNCPPutBit *pb, const float *prob, int n_symb, int sym);
int nncp_read_sym(NNCPGetBit *gb, const float *prob, int n_symb);
/* same decomposition driven by a 16-bit integer CDF (cdf[0] = 0, implicit
   cdf[n_symb] = 65536): prob0 = ((cdf[mid]-cdf[lo]) << 15) / (cdf[hi]-cdf[lo])
   clamped to [1, 32767]; O(log n_symb) integer work per symbol */
void nncp_write_sym_cdf(NNCPPutBit *pb, const uint16_t *cdf, int n_symb, int sym);
int nncp_read_sym_cdf(NNCPGetBit *gb, const uint16_t *cdf, int n_symb);
/* nncp_write_sym_cdf given only the entries it reads for this symbol, in reading order (a column
   of nc_cdf_path, nc_ext.h): the same bits */
void nncp_write_sym_cdf_path(NNCPPutBit *pb, const uint16_t *path, int n_symb, int sym);

/* piece-wise linear schedule with optional power decay (cp_utils.c:380-410) */
typedef struct {
    int n_steps;
    float val[9];
    int64_t pos[8];
    float decay_power;
} NNCPInterp;
float nncp_interp(const NNCPInterp *p, int64_t pos);
/* The address of nc_context_init as the calls of this library resolve it.  A loader that
   holds the libnc it meant to pair with this library compares it with that library's own
   symbol: a libnc that sits in the process-wide namespace (RTLD_GLOBAL, LD_PRELOAD) is found
   first by the dynamic linker and would otherwise take the calls unnoticed.  (No
   counterpart in the reference, which links one libnc statically into one executable.) */
const void *nncp_bound_libnc(void);

/* ---- Transformer-XL model ------------------------------------------------------ */
#define NNCP_LN_POST (1 << 0)    /* nncp.c:74-78 */
#define NNCP_LN_PRE (1 << 1)
#define NNCP_LN_FINAL (1 << 2)
#define NNCP_LN_COEF (1 << 3)
#define NNCP_LN_RMSNORM (1 << 4)
#define NNCP_FF_RELU 0           /* nncp.c:82-87 */
#define NNCP_FF_GELU 1
#define NNCP_FF_GEGLU 2
#define NNCP_FF_GATED_SILU 3
#define NNCP_N_LAYER_MAX 32

typedef struct { /* TransformerModelParams + the NNCPModelParams fields it needs */
    int n_layer, d_model, n_head, d_key, d_value, d_inner, d_pos, mem_len;
    int attn_len[NNCP_N_LAYER_MAX];
    int use_bias, use_w_r, tied_w_r, tied_b_r, query_bias, ln_flags, ff_act;
    float init_range, embed_mult;
    SGDOptParams sgd_opt;
    int batch_size, seg_len, n_symbols;
    uint32_t seed;
    int use_device; /* nncp --cuda: compute on the accelerator device */
    int fused;      /* 1: trf_eval uses nc_linear / nc_relpos_attention /
                       nc_fused_layer_norm (full-segment evaluation only) */
    int nb_threads;
    /* retrain (NNCPModelParams, nncp.c:112-113, 153-156): all zero = off, as in
       the default profile */
    float dropout_prob, dropout_att_prob; /* used during retrain only */
    int retrain_period;  /* in symbols; a retrain pass runs between blocks once this many were coded */
    int retrain_len;     /* length of the retrain buffer, in symbols */
    int has_retrain_lr;
    NNCPInterp retrain_lr;
    /* model class (NNCPModelParams.model_class): 0 = Transformer-XL, the fields
       above; 1 = LSTM (LSTMParams, nncp.c:124-140), which uses n_layer,
       batch_size, seg_len, n_symbols, seed, sgd_opt, use_device, nb_threads
       from above and the fields below */
    int model_type;
    int lstm_n_cells, lstm_n_cells2, lstm_n_embed_out; /* n_cells2 >= n_cells: with projection */
    int lstm_type;                                     /* NNCP_LSTM_* */
    int lstm_full_connect, lstm_use_layer_norm;
    float lstm_forget_bias;
    /* parameters are NC_TYPE_BF16 tensors, 2 bytes per element (param_type of nncp.c:343-346
       and 1727-1730 under nncp --bf16); matrix products then round their other operand to bf16
       as well.  The optimiser keeps an fp32 master of every parameter; activations and the
       memories stay f32. */
    int param_bf16;
} NNCPConfig;

#define NNCP_MODEL_TRF 0
#define NNCP_MODEL_LSTM 1
#define NNCP_LSTM_NORMAL 0  /* nncp.c:117-122 */
#define NNCP_LSTM_CLAMPED 1
#define NNCP_LSTM_TIED 2

typedef struct { /* nncp.c:183-193 */
    uint16_t *buf;
    int buf_pos, buf_len; /* next write position; symbols held */
    int pos;              /* symbols coded since the last retrain pass */
    int64_t train_step;   /* steps of the retrain schedule (has_retrain_lr) */
} NNCPRetrainState;

typedef struct NNCPModel NNCPModel;

void nncp_config_default(NNCPConfig *cfg);           /* nncp.c:2471-2513 */
void nncp_config_default_lstm(NNCPConfig *cfg);      /* the "lstm" profile, nncp.c:2574-2603 */
NNCPModel *nncp_model_new(const NNCPConfig *cfg);    /* nncp_init + trf_init, nncp.c:2762, 304 */
void nncp_model_free(NNCPModel *s);                  /* nncp_end + trf_end, nncp.c:2802, 522 */
const NNCPConfig *nncp_model_config(NNCPModel *s);
NCContext *nncp_model_context(NNCPModel *s);
NCDevice *nncp_model_device(NNCPModel *s);
NCDevice *nncp_model_cpu_device(NNCPModel *s);
/* address of the parameter tensor registered under `name` ("w_q_0", "embed",
   ...: the names of trf_init), or NULL */
NCTensor **nncp_model_param(NNCPModel *s, const char *name);
int nncp_model_param_count(NNCPModel *s);
const char *nncp_model_param_name(NNCPModel *s, int index);
int64_t nncp_model_train_step(NNCPModel *s);
/* What a training step carries over to the next besides the parameters, for checkpoints and
   for tests that put two models into the same state: the optimiser's moment `which` of the
   named parameter (nc_sgd_opt_get_state / nc_sgd_opt_set_state of nc_ext.h; get returns an
   owned host tensor or NULL, set copies v in) and the memory of layer l, the (d_model, B,
   mem_len) tensor mem_h[l] of nncp.c:1205-1221 (borrowed until the model's next update, which
   may replace it: on the GPU a memory longer than a segment is a window that moves through a
   larger store; Transformer models only, NULL for an LSTM or without memory). */
NCTensor *nncp_model_opt_state(NNCPModel *s, const char *name, int which);
void nncp_model_set_opt_state(NNCPModel *s, const char *name, int which, const NCTensor *v);
NCTensor *nncp_model_memory(NNCPModel *s, int l);
/* every registered parameter to / from a parameter file (nc_save_coefs / nc_load_coefs,
   libnc.h:530, 536; the file named by --load_coefs, nncp.c:3761).  Loading needs a model of
   the same configuration: names, shapes and types must match. */
void nncp_model_save_coefs(NNCPModel *s, const char *filename);
void nncp_model_load_coefs(NNCPModel *s, const char *filename);

/* the `trf` model class (nncp.c:1544-1562); input/expected are (B, T) i32
   host tensors, borrowed; trf_eval returns an owned (V, B, T|1) tensor */
NCTensor *trf_eval(NNCPModel *s, int output_index, const NCTensor *input); /* nncp.c:581 */
void trf_eval_end(NNCPModel *s);                                           /* nncp.c:1032 */
float trf_eval_gradient(NNCPModel *s, const NCTensor *expected_output);    /* nncp.c:1099 */
void trf_reset(NNCPModel *s);                                              /* nncp.c:1195 */
void trf_update(NNCPModel *s);                                             /* nncp.c:1224 */
void trf_set_lr(NNCPModel *s, float lr);                                   /* nncp.c:1243 */
/* dropout on (only if cfg.dropout_prob != 0) / off; while it is on, trf_eval
   takes the op-by-op path even when cfg.fused is set */
void trf_set_retrain(NNCPModel *s, int enabled);                           /* nncp.c:1237 */
NNCPRetrainState *nncp_model_retrain_state(NNCPModel *s);
void nncp_model_set_train_step(NNCPModel *s, int64_t step);
/* logits of the last trf_eval (V, B, T|1), borrowed; used by the CDF path */
NCTensor *trf_last_logits(NNCPModel *s);
/* the `lstm` model class (nncp.c:1565-2330: lstm_eval, lstm_eval_gradient, ...),
   same calling conventions; n_states = seg_len (no overlap), no dropout */
NCTensor *lstm_eval(NNCPModel *s, int output_index, const NCTensor *input); /* nncp.c:1872 */
void lstm_eval_end(NNCPModel *s);                                           /* nncp.c:2060 */
float lstm_eval_gradient(NNCPModel *s, const NCTensor *expected_output);    /* nncp.c:2070 */
void lstm_reset(NNCPModel *s);                                              /* nncp.c:1859 */
void lstm_update(NNCPModel *s);                                             /* nncp.c:2136 */

/* NNCPModelClass (nncp.c:49-69): what the block loop calls; trf_* or lstm_* */
typedef struct {
    NCTensor *(*eval)(NNCPModel *s, int output_index, const NCTensor *input);
    void (*eval_end)(NNCPModel *s);
    float (*eval_gradient)(NNCPModel *s, const NCTensor *expected_output);
    void (*reset)(NNCPModel *s);
    void (*update)(NNCPModel *s);
    void (*set_lr)(NNCPModel *s, float lr);
    void (*set_retrain)(NNCPModel *s, int enabled);
    NCTensor *(*last_logits)(NNCPModel *s); /* logits of the last eval, borrowed */
    /* eval_end for an evaluation that is to leave no trace (the replaying decoder of
       NNCP_MODE_SEGMENT): also takes back the recurrent state it handed on */
    void (*eval_discard)(NNCPModel *s);
    /* optional (NULL: not offered).  After a whole-segment eval, with the expected symbols
       already on the model's device ((B, T) i32, consumed): queues the loss of that evaluation
       and its transfer to the host, without waiting.  The eval_gradient that follows - after
       the caller has synchronised the device for its own purposes - takes the loss from there
       instead of uploading `expected_output`, computing it and waiting for it. */
    void (*queue_loss)(NNCPModel *s, NCTensor *expected_on_device);
} NNCPModelClass;
const NNCPModelClass *nncp_model_class(NNCPModel *s);
/* logits of the last evaluation of either class (V, B, T|1), borrowed */
NCTensor *nncp_model_last_logits(NNCPModel *s);

/* Per-timestep evaluation with K/V caches through the fused entry points (the
   decoder's view of a segment, nncp.c:801-863; cfg.fused = 1 and the shapes of
   the single-kernel attention).  trf_step_begin once per segment, then
   trf_eval_step(t, input) for t = 0, 1, ...: evaluates the one token column t of
   input (B, T) against the memory and the columns evaluated so far and returns
   the owned probabilities (V, B, 1); no graph is kept.  With
   nc_set_matmul_width_invariant() on for both sides, its logits equal column t
   of the whole-segment trf_eval bit for bit. */
void trf_step_begin(NNCPModel *s);
NCTensor *trf_eval_step(NNCPModel *s, int t, const NCTensor *input);
void trf_step_end(NNCPModel *s);
/* until the next trf_step_begin / trf_step_end: trf_eval_step returns the logits (V, B, 1)
   instead of the probabilities - for a caller that builds integer CDFs from them and has no
   use for the softmax launch */
void trf_step_logits_only(NNCPModel *s, int on);

/* ---- block loop (process_block, nncp.c:2968-3147) ------------------------------ */
#define NNCP_MODE_SEQ_EVAL 0   /* one trf_eval per timestep: decodable, as nncp c/d */
#define NNCP_MODE_SEGMENT 1    /* one trf_eval per segment (nncp --encode_only); the
                                  decoder replays the same segment evaluation T times */
#define NNCP_MODE_STEP_DECODE 4 /* with NNCP_MODE_SEGMENT: the decoder evaluates one token
                                  column per timestep against K/V caches (trf_eval_step)
                                  instead of replaying the segment; both sides then run
                                  their forward products width-invariant, so the flag is
                                  part of the stream's format */
#define NNCP_CODER_FLOAT 0     /* write_sym on float probabilities */
#define NNCP_CODER_CDF16 2     /* nc_soft_max_cdf16 + integer symbol coder */

typedef struct {
    int64_t n_symbols, n_steps;
    double loss_bits;   /* -sum log2 p[target] over the trained symbols */
    double t_eval, t_code, t_grad, t_update; /* seconds, host wall clock */
} NNCPStats;

/* Codes block_len symbols (values < n_symbols) as one block: B contiguous
   sub-streams, training after every full segment, the tail without training.
   is_decode = 0: reads block_buf, writes through pb.  is_decode = 1: reads
   through gb, fills block_buf.  lr: learning-rate schedule. */
void nncp_process_block(NNCPModel *s, NNCPPutBit *pb, NNCPGetBit *gb, uint16_t *block_buf,
                        int block_len, int is_decode, int mode, const NNCPInterp *lr,
                        NNCPStats *st);

/* retrain_block (nncp.c:2821-2941): appends the block just coded (encoder) or
   decoded (decoder) to the retrain buffer; once cfg.retrain_period symbols have
   gone by since the last pass, resets the memory and trains over the whole
   buffer again, B streams of buffer_len / B symbols, one segment per step, with
   dropout on and the rate of cfg.retrain_lr (its own step counter) or of `lr`
   (the model's counter, which then advances).  Both sides must call it after
   every block.  No-op when cfg.retrain_period is 0.  st (or NULL) receives the
   steps and the loss of the pass. */
void nncp_retrain_block(NNCPModel *s, const uint16_t *block_buf, int block_len,
                        const NNCPInterp *lr, NNCPStats *st);
/* symbol idx of a FIFO that holds `size` symbols whose oldest one sits at rpos
   (nncp.c:2811-2819); 0 before the start */
int nncp_fifo_symbol(const uint16_t *buf, int rpos, int size, int idx);

/* convenience: whole buffer as one block, in memory; returns the number of
   bytes written (compress) */
size_t nncp_compress(NNCPModel *s, const uint16_t *syms, int n, uint8_t *out, size_t cap,
                     int mode, const NNCPInterp *lr, NNCPStats *st);
void nncp_decompress(NNCPModel *s, const uint8_t *in, size_t len, uint16_t *syms, int n,
                     int mode, const NNCPInterp *lr, NNCPStats *st);

/* ---- file container (encode_file / decode_file, nncp.c:3307-3677) ---------------- */
/* NNCPModelParams' file-level fields that NNCPConfig does not hold (nncp.c:142-156) */
typedef struct {
    NNCPInterp lr, block_len; /* per training step; per file position */
    int use_bf16;             /* nncp --bf16.  1: matrix products round their operands to bf16,
                                 parameters stay f32; 2: parameters are stored as bf16 as well
                                 (NNCPConfig.param_bf16).  The header byte holds the value. */
    int64_t max_size;         /* encoder: truncate the input to this many symbols; -1: no limit */
    int mode;                 /* NNCP_MODE_* | NNCP_CODER_*; 0 is the reference's stream */
} NNCPFileParams;

/* nncp_init_params (nncp.c:2464-2636): "default", "enwik8", "enwik9", "lstm",
   "lstm_fast"; -1 for an unknown name */
int nncp_profile(NNCPConfig *cfg, NNCPFileParams *fp, const char *profile);
/* "v0,pos0,v1,...[,p<power>]" (parse_interp_param / dump_interp_param,
   cp_utils.c:412-470); parse returns -1 on a syntax error, format the length */
int nncp_parse_interp(NNCPInterp *p, const char *str);
int nncp_format_interp(char *buf, size_t size, const NNCPInterp *p);
/* the big-endian header of nncp.c:2662-2760 with the model's own fields
   (nncp.c:1333-1365, 2198-2211).  write returns the length, 0 if cap is too
   small.  read returns 0, -1 for an invalid header, -2 for a valid one that
   asks for an option this build does not have (tied_embed, rot_pos, GRU,
   n_states != seg_len); cfg.fused, cfg.nb_threads and fp.mode are not part of
   it (the file loops keep them in the byte that follows). */
size_t nncp_header_write(uint8_t *buf, size_t cap, const NNCPConfig *cfg, const NNCPFileParams *fp);
int nncp_header_read(const uint8_t *buf, size_t len, NNCPConfig *cfg, NNCPFileParams *fp, size_t *used);
/* length of the block that starts at file_pos (nncp.c:3452-3457): the schedule's
   value rounded down to whole steps of seg_len * batch_size, at least one, at
   most what remains */
int nncp_block_len(const NNCPConfig *cfg, const NNCPInterp *sched, int64_t file_pos, int64_t remaining);
/* Whole files: header, flag byte, 32-bit symbol count, then every block through
   one range coder with the retrain pass between blocks.  Symbols are bytes, or
   big-endian 16-bit values when cfg.n_symbols > 256.  No dictionary
   preprocessor: decode refuses a file written with one.  The decoder takes the
   model from the file and the device from its caller, as nncp d does.
   Return 0, or -1 after a message on stderr.  st / retrain_st (or NULL)
   accumulate the statistics of coding and of the retrain passes. */
int nncp_encode_file(const char *in_name, const char *out_name, const NNCPConfig *cfg,
                     const NNCPFileParams *fp, NNCPStats *st, NNCPStats *retrain_st);
int nncp_decode_file(const char *in_name, const char *out_name, int use_device, int nb_threads,
                     NNCPStats *st, NNCPStats *retrain_st);

#ifdef __cplusplus
}
#endif
#endif /* NNCP_HOST_H */
