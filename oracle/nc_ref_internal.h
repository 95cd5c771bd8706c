/*
 * Internal structures of libnc_ref, the scalar CPU restatement of the libnc
 * API.  TEST INFRASTRUCTURE ONLY: it is the checker the GPU library is
 * compared against and the timed CPU baseline; nothing in the product links,
 * loads or calls it.
 */
#ifndef NC_REF_INTERNAL_H
#define NC_REF_INTERNAL_H

#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <assert.h>
#include "../include/nc_api.h"
#include "../include/nc_ext.h"

#define NC_MAX_ARGS 4

struct NCContext {
    int nb_threads;
    NCDevice *cpu;
    int64_t node_seq;
};

struct NCDevice {
    NCContext *ctx;
};

struct NCTensorBuffer {
    int ref;
    void *data;
    size_t size;
};

struct NCTensor {
    int ref;
    NCDevice *dev;
    NCTensorBuffer *buf;
    size_t off; /* element offset into buf */
    NCTypeEnum type;
    int n_dims;
    size_t dims[NC_N_DIMS_MAX];
    size_t strides[NC_N_DIMS_MAX]; /* in elements */
    NCNode *node;
};

typedef enum {
    OP_PARAM, OP_ADD, OP_MUL, OP_CONVERT, OP_MASKED_FILL, OP_SIGMOID, OP_TANH,
    OP_RELU, OP_GELU, OP_GATED_SWISH, OP_LSTM_CLAMPED, OP_LERP, OP_RESHAPE,
    OP_REPEAT, OP_REDUCE_SUM, OP_SUM, OP_SLICE, OP_CONCAT, OP_SPLIT_PART,
    OP_PAD, OP_PERMUTE, OP_MATMUL, OP_GET_COL, OP_SOFT_MAX, OP_INDEXED_LOG,
    OP_LAYER_NORM, OP_REL_SHIFT, OP_CONCAT_NODE, OP_FUSED_LN, OP_RELPOS_ATTN,
    OP_LINEAR,
} NCOpEnum;

struct NCNode {
    int ref;
    NCOpEnum op;
    int64_t seq;
    int n_args;
    NCNode **parents;    /* n_args entries, NULL = no gradient wanted */
    NCTensor *saved[6];  /* tensors kept for the backward pass */
    /* shapes of the arguments (for un-broadcasting gradients) */
    int arg_ndims[NC_MAX_ARGS];
    size_t arg_dims[NC_MAX_ARGS][NC_N_DIMS_MAX];
    int out_ndims;
    size_t out_dims[NC_N_DIMS_MAX];
    /* op attributes */
    int ia[8];
    float fa[4];
    size_t *sizes; /* concat / concat_node piece sizes */
    void *opaque;  /* OP_PARAM */
    /* backward-walk state */
    NCTensor *grad;
    int pending;
    int mark;
};

/* nc_ref_core.c */
void nc_fatal(const char *fmt, ...) __attribute__((noreturn, format(printf, 1, 2)));
size_t nc_type_size(NCTypeEnum t);
size_t nc_numel(const NCTensor *x);
int nc_is_contig(const NCTensor *x);
NCTensor *nc_contig(NCTensor *x); /* consumes, returns contiguous */
NCTensor *nc_alloc_like(const NCTensor *x);
NCTensor *nc_alloc(NCDevice *d, NCTypeEnum type, int n_dims, const size_t *dims, int zero);
NCTensor *nc_view(const NCTensor *x); /* new header sharing the buffer, no node */
float *nc_f32(const NCTensor *x);     /* data pointer (offset applied) */
void nc_copy_strided(NCTensor *dst, const NCTensor *src);

/* bf16 <-> f32: nearest even on the way down (NaN stays a quiet NaN), exact on the way up */
static inline uint16_t nc_bf16_bits(float f)
{
    union { float f; uint32_t u; } v = { f };
    if ((v.u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((v.u >> 16) | 0x40);
    v.u += 0x7fff + ((v.u >> 16) & 1);
    return (uint16_t)(v.u >> 16);
}

static inline float nc_bf16_widen(uint16_t b)
{
    union { uint32_t u; float f; } v = { (uint32_t)b << 16 };
    return v.f;
}

/* nc_ref_ops.c */
NCNode *nc_new_node(NCContext *m, NCOpEnum op, int n_args, NCTensor **args);
void nc_attach(NCTensor *y, NCNode *n);
int nc_needs_grad(NCTensor **args, int n);

/* nc_ref_ext.c */
void nc_relpos_attention_bw(NCNode *nd, NCTensor *g, NCTensor **ga);

/* nc_ref_gemm.c : C(m x n) = alpha * op(A) * op(B) + beta * C, column-major */
void ref_sgemm(int ta, int tb, int m, int n, int k, float alpha,
               const float *a, int lda, const float *b, int ldb,
               float beta, float *c, int ldc);

#endif
