/*
 * model_internal.h - what the model classes and the block loop share: the
 * model object (NNCPModelState of nncp.c:170-200 with the fields of both model
 * classes) and the class table (NNCPModelClass, nncp.c:49-69).
 */
#ifndef NNCP_MODEL_INTERNAL_H
#define NNCP_MODEL_INTERNAL_H

#include "../../include/nncp_host.h"

typedef struct {
    NCTensor *w_q, *w_kv, *b_q, *w_o;
    NCTensor *ff1, *ff2, *ff_bias1, *ff_bias2;
    NCTensor *w_r, *b_r;
    NCTensor *ln_g1, *ln_b1, *ln_g2, *ln_b2, *alpha;
    /* per-timestep evaluation only */
    NCTensor *mem_key, *mem_value, *tmp_w_r, *tmp_b_r, *attn_mask;
    NCNode **key_nodes, **kq_nodes, **value_nodes, **va_nodes;
} Layer;

struct LstmState;

struct NNCPModel {
    NNCPConfig cfg;
    const NNCPModelClass *cls;
    struct LstmState *lstm; /* model_type 1 */
    NCContext *ctx;
    NCDevice *dev, *cpu;
    NCRNDState *rnd;
    NCTypeEnum param_type; /* F32 or BF16 (nncp.c:255, 343-346) */
    NCParamList params;
    Layer *layers;
    NCTensor *ln_g, *ln_b, *embed, *embed_out, *out_bias;
    NCTensor **mem_h, **train_h, **outputs;
    /* on the GPU with mem_len > seg_len: mem_h[l] is a window of mem_len steps in mem_store[l]
       (mem_cap steps), which an update moves by one segment instead of shifting the rows */
    NCTensor **mem_store;
    int *mem_pos, mem_cap;
    NCTensor **step_kv, **step_kvm; /* per-timestep decoding: K/V of the segment so far, K/V of the memory */
    NCTensor *step_embed_mult; /* the embedding scale as a device scalar, kept for the timesteps of a segment */
    int step_logits_only;      /* trf_eval_step returns the logits: the caller builds integer CDFs from them */
    NCTensor *logits;
    NCTensor *pending_loss, *pending_loss_host; /* queue_loss: the summed log-likelihood with its graph, and its copy on the way to the host */
    NCSGDOptState *opt;
    int seq_eval;
    float embed_mult;
    int64_t train_step;
    /* retrain (nncp.c:183-193, 257-259): dropout is on only inside retrain_block */
    int dropout_enabled;
    int fused_now; /* cfg.fused, except while dropout is on (masks sit between the fused steps) */
    NNCPRetrainState retrain;
};


/* lstm_model.c */
extern const NNCPModelClass nncp_lstm_class;
void lstm_init(NNCPModel *s);
void lstm_end(NNCPModel *s);
/* trf_model.c */
extern const NNCPModelClass nncp_trf_class;
void nncp_backward_cb(void *opaque, NCTensor *yg, NCTensor *get_col_index);

#endif
