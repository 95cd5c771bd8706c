/*
 * nc_api.h - the libnc-compatible C ABI exported by this repository.
 *
 * Two libraries export exactly these symbols:
 *   - libnc_hip.so  (nncp-metal_amd/csrc): the MI355X/gfx950 product, every
 *                    compute op runs as a HIP kernel;
 *   - libnc_ref.so  (oracle/): the scalar CPU checker used by the tests only.
 *
 * Each declaration replaces the declaration of the same name in the
 * reference's libnc.h (cited as "libnc.h:<line>"), which is the interface
 * nncp.c and cp_utils.c link against.  Types are layout-compatible with the
 * reference header: when that header has already been included (LIBNC_H
 * defined) the type block below is skipped and only the prototypes are
 * re-declared, which makes the C compiler check the two against each other.
 *
 * Conventions (inferred from how nncp.c drives the API):
 *   - tensors are column-major: dims[0] is the contiguous axis;
 *   - every op taking "NCTensor *" consumes one reference of each argument and
 *     returns a new owned tensor; "const NCTensor *" arguments are borrowed;
 *   - there are no error codes: misuse aborts with a message on stderr.
 */
#ifndef NC_API_H
#define NC_API_H

#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <sys/types.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Profiling hooks of the boundary (libnc.h:14-67).  The reference's prof_start / prof_end are
   inline in its header and count cycles into prof_cycles[] only when built with -DPROFILE;
   here they are always live: they forward to the library, which adds the elapsed nanoseconds
   to prof_cycles[idx], counts the sample and - when the environment variable NC_PROFILE is set
   - opens / closes a roctx range of the section's name ("EVAL", "GRAD", ...), so the sections of
   nncp.c:606/1027, 1108/1191, 1227/1234, 2881/2917 show up in a rocprofv3 marker trace.
   nc_prof_dump (libnc.h:67) prints the table to stderr when NC_PROFILE is set. */
void nc_prof_begin(int idx);
void nc_prof_finish(int idx, int n_ops);

#ifndef LIBNC_H /* ---- types (skipped when the reference header is present) */

typedef enum { /* libnc.h:16-25 */
    PROF_EVAL,
    PROF_GRAD,
    PROF_SGD,
    PROF_UPDATE,
    PROF_WRITE_SYM,
    PROF_PROBE,
    PROF_TOTAL,
    PROF_COUNT,
} ProfEnum;

extern int64_t prof_cycles[PROF_COUNT];  /* libnc.h:29-31; nanoseconds here */
extern int64_t prof_samples[PROF_COUNT];
extern int64_t prof_ops[PROF_COUNT];

static inline void prof_start(int idx) { nc_prof_begin(idx); }                      /* libnc.h:33 */
static inline void prof_end(int idx) { nc_prof_finish(idx, 0); }                    /* libnc.h:38 */
static inline void prof_end_ops(int idx, int n_ops) { nc_prof_finish(idx, n_ops); } /* libnc.h:44 */

#ifndef CUTILS_H
typedef int BOOL;
#endif

#ifndef LIST_H
struct list_head {
    struct list_head *prev;
    struct list_head *next;
};
#endif

typedef struct NCContext NCContext;           /* libnc.h:71 */
typedef struct NCDevice NCDevice;             /* libnc.h:72 */
typedef struct NCTensor NCTensor;             /* libnc.h:73 */
typedef struct NCTensorBuffer NCTensorBuffer; /* libnc.h:74 */
typedef struct NCNode NCNode;                 /* libnc.h:75 */
typedef struct NCRNDState NCRNDState;         /* libnc.h:77 */
typedef struct NCSGDOptState NCSGDOptState;   /* libnc.h:78 */

/* libnc.h:80-98; only F32, BF16, I8, I32, U16 carry data here */
typedef enum {
    NC_TYPE_F32, NC_TYPE_BF16, NC_TYPE_F16, NC_TYPE_I8, NC_TYPE_I16,
    NC_TYPE_I32, NC_TYPE_U8, NC_TYPE_U16, NC_TYPE_U32, NC_TYPE_E4M3,
    NC_TYPE_E5M2, NC_TYPE_BF8, NC_TYPE_BF4, NC_TYPE_BF3, NC_TYPE_BF8L,
    NC_TYPE_BF8C, NC_TYPE_COUNT,
} NCTypeEnum;

#define NC_N_DIMS_MAX 8 /* libnc.h:104 */

typedef struct NCTensorData { /* libnc.h:106-115 */
    NCTypeEnum item_type;
    size_t item_size;
    void *data;
    size_t stride;
    size_t n_strides;
    int n_dims;
    const size_t *dims;
    const size_t *strides;
} NCTensorData;

typedef enum { /* libnc.h:325-331 */
    NC_PAD_ZERO,
    NC_PAD_DUP,
    NC_TRIM_NORMAL = NC_PAD_ZERO,
    NC_TRIM_SUM,
} NCPadEnum;

typedef void NCParamUpdateFunc(void *opaque, NCTensor *grad,
                               NCTensor *get_col_index); /* libnc.h:453 */

#define NC_BW_KEEP_GRAD_GRAPH (1 << 0) /* libnc.h:474 */
#define NC_BW_SPARSE_GRAD     (1 << 1) /* libnc.h:476 */
#define NC_BW_KEEP_ARGS       (1 << 2) /* libnc.h:478 */

struct NCConvertToF8Context;

typedef struct { /* libnc.h:501-510 */
    struct list_head link;
    NCTensor **pval;
    char *name;
    NCTensor *saved_grad;
    struct SGDOptVarState *sgd_opt;
    float lr_mult;
    struct NCConvertToF8Context *fcs;
} NCParam;

typedef struct { /* libnc.h:512-516 */
    NCContext *ctx;
    struct list_head param_list;
    BOOL add_graph;
} NCParamList;

typedef enum { /* libnc.h:540-544 */
    SGD_OPT_BASIC,
    SGD_OPT_ADAM,
    SGD_OPT_TEST,
} SGDOptAlgoEnum;

typedef struct { /* libnc.h:546-559 */
    SGDOptAlgoEnum algo;
    union {
        struct {
            float beta1;
            float beta2;
            float eps;
            float gradient_clip;
            float weight_decay;
            float loss_scale;
        } adam;
    } u;
    float lr;
} SGDOptParams;

#endif /* !LIBNC_H */

/* Extension value for SGDOptParams.algo (not in the reference enum):
   plain RMSProp, v = b2*v + (1-b2)*g*g ; w -= lr*g/(sqrt(v)+eps), no bias
   correction, no clipping.  Uses u.adam.beta2 and u.adam.eps. */
#define SGD_OPT_RMSPROP 16

/* ---- memory, context, devices ------------------------------------------ */
void *nc_malloc(size_t size);                         /* libnc.h:117 */
void *nc_mallocz(size_t size);                        /* libnc.h:118 */
void nc_free(void *ptr);                              /* libnc.h:119 */
NCContext *nc_context_init(int nb_threads);           /* libnc.h:124 */
void nc_context_end(NCContext *m);                    /* libnc.h:125 */
NCDevice *nc_new_cpu_device(NCContext *m);            /* libnc.h:127 */
/* In libnc_hip.so this returns the HIP device (so nncp's --cuda flag selects
   the MI355X); in libnc_ref.so it returns the CPU device. */
NCDevice *nc_new_cuda_device(NCContext *m, int device_index); /* libnc.h:128 */
NCDevice *nc_new_device(NCContext *m, const char *device_name); /* libnc.h:129 */
void nc_synchronize(NCDevice *d);                     /* libnc.h:130 */
void nc_prof_dump(void);                              /* libnc.h:67 */

/* ---- tensor creation / bookkeeping -------------------------------------- */
NCTensor *nc_new_tensor(NCDevice *d, NCTypeEnum type, int n_dims,
                        const size_t *dims);                           /* libnc.h:153 */
NCTensor *nc_new_tensor_nz(NCDevice *d, NCTypeEnum type, int n_dims,
                           const size_t *dims);                        /* libnc.h:163 */
NCTensor *nc_new_tensor_from_tensor_nz(const NCTensor *x);             /* libnc.h:165 */
NCTensor *nc_new_scalar(NCDevice *d, NCTypeEnum type);                 /* libnc.h:156 */
NCTensor *nc_new_tensor_1d(NCDevice *d, NCTypeEnum type, size_t len);  /* libnc.h:157 */
NCTensor *nc_new_tensor_2d(NCDevice *d, NCTypeEnum type, size_t n0,
                           size_t n1);                                 /* libnc.h:158 */
NCTensor *nc_new_tensor_3d(NCDevice *d, NCTypeEnum type, size_t n0,
                           size_t n1, size_t n2);                      /* libnc.h:159 */
NCTensor *nc_new_tensor_4d(NCDevice *d, NCTypeEnum type, size_t n0,
                           size_t n1, size_t n2, size_t n3);           /* libnc.h:161 */
NCTensor *nc_new_f32(NCDevice *d, float val);                          /* libnc.h:278 */
NCTensor *__attribute__((format(printf, 2, 3)))
nc_tensor_set_name(NCTensor *x, const char *fmt, ...);                 /* libnc.h:172 */
NCTensor *nc_dup_tensor(const NCTensor *x);                            /* libnc.h:173 */
void nc_free_tensor(NCTensor *x);                                      /* libnc.h:174 */
uint32_t nc_tensor_get_hash(const NCTensor *x);                        /* libnc.h:177 */
NCNode *nc_get_node(NCTensor *x);                                      /* libnc.h:180 */
NCTypeEnum nc_tensor_get_item_type(const NCTensor *x);                 /* libnc.h:181 */
void *nc_tensor_get_ptr(const NCTensor *x, size_t *pstride);           /* libnc.h:185 */
int nc_tensor_get_dims(const NCTensor *x, size_t *dims);               /* libnc.h:189 */
void nc_tensor_set_zero(NCTensor *y);                                  /* libnc.h:192 */
void nc_tensor_set_f32(NCTensor *y, float val);                        /* libnc.h:194 */
NCRNDState *nc_rnd_init(NCDevice *d, uint32_t seed);                   /* libnc.h:195 */
void nc_rnd_end(NCRNDState *s);                                        /* libnc.h:196 */
void nc_tensor_set_rnd_unif(NCTensor *y, float avg, float range,
                            NCRNDState *rnd_state);                    /* libnc.h:197 */
void nc_tensor_set_dropout(NCTensor *y, float prob,
                           NCRNDState *rnd_state);                     /* libnc.h:201 */
void nc_set1_i32_2d(NCTensor *y, size_t i0, size_t i1, int32_t val);   /* libnc.h:206 */
float nc_get_scalar_f32(const NCTensor *x);                            /* libnc.h:214 */
void nc_tensor_copy(NCTensor *dst, NCTensor *src);                     /* libnc.h:218 */
void nc_tensor_copy_slice(NCTensor *dst, NCTensor *src, int axis,
                          size_t dst_start, size_t dst_end,
                          size_t src_start);                           /* libnc.h:219 */
NCTensor *nc_tensor_to_device(NCTensor *x, NCDevice *d);               /* libnc.h:226 */
NCTensor *nc_tensor_to_cpu_device(NCTensor *x);                        /* libnc.h:227 */
NCDevice *nc_get_tensor_device(const NCTensor *x);                     /* libnc.h:228 */

/* ---- element-wise ops ---------------------------------------------------- */
/* Two item types carry values: NC_TYPE_F32 and NC_TYPE_BF16 (2 bytes per element: the storage
   type of parameters under nncp's bf16 switch, nncp.c:343-346).  F32 -> BF16 rounds to
   nearest even, BF16 -> F32 is exact; the gradient passes through a conversion unchanged, as
   F32.  Arithmetic is F32 throughout: an op that is handed a BF16 tensor works on its
   widened values and returns F32 (in libnc_hip.so a bf16-operand product reads the 2-byte
   storage directly).  The optimiser keeps an fp32 master of a BF16 parameter (nc_ext.h). */
NCTensor *nc_convert(NCTensor *x, NCTypeEnum new_type);                /* libnc.h:231 */
NCTensor *nc_add(NCTensor *x1, NCTensor *x2);                          /* libnc.h:232 */
NCTensor *nc_mul(NCTensor *x1, NCTensor *x2);                          /* libnc.h:235 */
NCTensor *nc_masked_fill(NCTensor *x, NCTensor *mask, float c,
                         BOOL mask_inv);                               /* libnc.h:244 */
NCTensor *nc_sigmoid(NCTensor *x);                                     /* libnc.h:245 */
NCTensor *nc_tanh(NCTensor *x);                                        /* libnc.h:246 */
NCTensor *nc_relu(NCTensor *x);                                        /* libnc.h:247 */
NCTensor *nc_gated_swish(NCTensor *g, NCTensor *x, float beta);        /* libnc.h:251 */
NCTensor *nc_gelu(NCTensor *x);                                        /* libnc.h:252 */
NCTensor *nc_lstm_clamped(NCTensor *cp, NCTensor *in, NCTensor *fg,
                          NCTensor *ig);                               /* libnc.h:262 */
NCTensor *nc_lerp(NCTensor *a, NCTensor *b, NCTensor *t);              /* libnc.h:273 */

/* ---- shape ops ----------------------------------------------------------- */
NCTensor *nc_reshape_1d(NCTensor *x, size_t n0);                       /* libnc.h:282 */
NCTensor *nc_reshape_2d(NCTensor *x, size_t n0, size_t n1);            /* libnc.h:283 */
NCTensor *nc_reshape_3d(NCTensor *x, size_t n0, size_t n1, size_t n2); /* libnc.h:284 */
NCTensor *nc_reshape_4d(NCTensor *x, size_t n0, size_t n1, size_t n2,
                        size_t n3);                                    /* libnc.h:285 */
NCTensor *nc_repeat_1d(NCTensor *x, size_t n0);                        /* libnc.h:291 */
NCTensor *nc_repeat_2d(NCTensor *x, size_t n0, size_t n1);             /* libnc.h:292 */
NCTensor *nc_reduce_sum(NCTensor *y0, NCTensor *x, int n_dims);        /* libnc.h:295 */
NCTensor *nc_sum(NCTensor *x);                                         /* libnc.h:299 */
NCTensor *nc_slice_alias(const NCTensor *x1, int axis, size_t start,
                         size_t end);                                  /* libnc.h:307 */
NCTensor *nc_slice(NCTensor *x, int axis, size_t start, size_t end);   /* libnc.h:308 */
NCTensor *nc_concat(NCTensor **inputs, int n_inputs, int axis);        /* libnc.h:311 */
NCTensor *nc_vconcat(NCTensor **inputs, int n_inputs);                 /* libnc.h:315 */
NCTensor *nc_hconcat(NCTensor **inputs, int n_inputs);                 /* libnc.h:317 */
void nc_split(NCTensor **tab_y, NCTensor *x, int n_outputs,
              const size_t *tab_size, int axis);                       /* libnc.h:319 */
NCTensor *nc_pad(NCTensor *x, ssize_t left_len, NCPadEnum left_op,
                 ssize_t right_len, NCPadEnum right_op);               /* libnc.h:334 */
NCTensor *nc_permute(NCTensor *x, int n_dims, const int *axis);        /* libnc.h:358 */
NCTensor *nc_permute_4d(NCTensor *x, int a0, int a1, int a2, int a3);  /* libnc.h:360 */

/* ---- linear algebra, normalisation, attention helpers -------------------- */
NCTensor *nc_matmul_add(NCTensor *w, NCTensor *x, NCTensor *c, BOOL w_trans,
                        BOOL x_trans, float alpha);                    /* libnc.h:370 */
NCTensor *nc_matmul(NCTensor *w, NCTensor *x);                         /* libnc.h:373 */
NCTensor *nc_get_col(NCTensor *w, NCTensor *x);                        /* libnc.h:375 */
NCTensor *nc_soft_max(NCTensor *x);                                    /* libnc.h:382 */
/* max(soft_max[i] * mult, 1) converted to int32 (floor), 0 <= mult <= 2^32; the integer
   CDF for the coder is nc_soft_max_cdf16 (nc_ext.h), which adds the exact total */
NCTensor *nc_soft_max_int(NCTensor *x, float mult);                    /* libnc.h:383-384 */
NCTensor *nc_indexed_log(NCTensor *x, NCTensor *eout);                 /* libnc.h:388 */
NCTensor *nc_layer_norm(NCTensor *x, float eps);                       /* libnc.h:389 */
NCTensor *nc_rms_norm(NCTensor *x, float eps);                         /* libnc.h:390 */
NCTensor *nc_fused_layer_norm(NCTensor *x, NCTensor *w, NCTensor *b,
                              float eps, BOOL avg_flag);               /* libnc.h:394 */
NCTensor *nc_rel_shift(NCTensor *x, ssize_t pos, ssize_t mult);        /* libnc.h:397 */
NCTensor *nc_cmul(NCTensor *x1, NCTensor *x2, BOOL is_conj,
                  BOOL is_planar);                                     /* libnc.h:402 */

/* ---- automatic differentiation ------------------------------------------ */
NCTensor *nc_set_param(NCTensor *x, void *opaque);                     /* libnc.h:457 */
NCNode *nc_dup_node(const NCNode *n);                                  /* libnc.h:462 */
void nc_free_node(NCNode *n);                                          /* libnc.h:463 */
void nc_combine_nodes(NCContext *m, NCNode **tab_op1, int count, int axis,
                      int elem_size, const size_t *tab_elem_size);     /* libnc.h:464 */
NCNode *nc_concat_node(NCContext *m, NCNode **inputs, int count, int axis,
                       const size_t *tab_size);                        /* libnc.h:466 */
void nc_concat_optimization(NCContext *m, NCNode **concat_nodes,
                            int count);                                /* libnc.h:468 */
void nc_node_set_parent(NCNode *n, int arg_index, const NCNode *n1);   /* libnc.h:469 */
void nc_node_set_arg(NCNode *n, int arg_index, const NCTensor *x);     /* libnc.h:470 */
void nc_backward(const NCTensor *x, NCTensor *grad,
                 NCParamUpdateFunc *param_update_func, int flags);     /* libnc.h:480 */

/* ---- parameters and optimiser -------------------------------------------- */
void nc_param_list_init(NCContext *m, NCParamList *pl);                /* libnc.h:518 */
__attribute__((format(printf, 3, 4))) NCParam *
nc_new_param(NCParamList *pl, NCTensor **pval, const char *fmt, ...);  /* libnc.h:521 */
void nc_param_list_end(NCParamList *pl);                               /* libnc.h:522 */
size_t nc_get_param_count(NCParamList *pl);                            /* libnc.h:525 */
NCParam *nc_find_param(NCParamList *pl, const char *name);             /* libnc.h:524 */
/* parameter files (libnc's own layout is not published: the layout is this library's,
   stated in csrc/nc_params_io.cpp; a file written by one build of this library is read by
   another, on either device) */
void nc_save_param_header(FILE *f, const char *config);                /* libnc.h:528 */
void nc_save_param(FILE *f, const NCTensor *v1, const char *name);     /* libnc.h:529 */
void nc_save_coefs(NCParamList *pl, const char *filename);             /* libnc.h:530 */
char *nc_load_param_header(FILE *f);                                   /* libnc.h:533 */
NCTensor *nc_load_param(NCContext *m, FILE *f, char *name,
                        size_t name_size);                             /* libnc.h:535 */
void nc_load_coefs(NCParamList *pl, const char *filename);             /* libnc.h:536 */
void nc_update_param(NCParamList *pl, const char *name,
                     const NCTensor *v);                               /* libnc.h:580 */
NCSGDOptState *nc_sgd_opt_init(NCContext *m, const SGDOptParams *p);   /* libnc.h:561 */
void nc_sgd_opt_end(NCSGDOptState *s);                                 /* libnc.h:562 */
void sgd_opt_update_var(void *opaque, NCTensor *yg,
                        NCTensor *get_col_index);                      /* libnc.h:563 */
void nc_sgd_opt_set_all(NCParamList *param_list, NCSGDOptState *s);    /* libnc.h:566 */
void nc_sgd_opt_update(NCSGDOptState *s);                              /* libnc.h:570 */
void nc_sgd_opt_set_lr(NCSGDOptState *s, float lr);                    /* libnc.h:572 */

/* host float sum used by the symbol coder; fixed left-to-right order */
float vec_sum_f32(const float *tab, size_t n);                         /* libnc.h:600 */

#ifdef __cplusplus
}
#endif
#endif /* NC_API_H */
