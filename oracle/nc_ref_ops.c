/*
 * libnc_ref ops and reverse-mode autodiff (CPU checker; test infrastructure
 * only).  Every op works on contiguous column-major f32 data with a fixed,
 * sequential reduction order.  The op list is the one trf_eval /
 * trf_eval_gradient issue (nncp.c:581-1193); semantics follow the comments of
 * libnc.h (cited per function).  Pinned by tests/test_oracle_*.py against
 * numpy restatements, closed forms and finite differences.
 */
#include <stdio.h>
#include "nc_ref_internal.h"

/* every op takes its operands through nc_operand (below): contiguous, bf16 widened */
NCTensor *nc_operand(NCTensor *x);
#define nc_contig(x) nc_operand(x)

/* ------------------------------------------------------------------------ */
/* graph nodes                                                              */

NCNode *nc_dup_node(const NCNode *n) /* libnc.h:462 */
{
    if (n)
        ((NCNode *)n)->ref++;
    return (NCNode *)n;
}

void nc_free_node(NCNode *n) /* libnc.h:463, NULL accepted (nncp.c:1047) */
{
    if (!n || --n->ref > 0)
        return;
    for (int i = 0; i < n->n_args; i++)
        nc_free_node(n->parents[i]);
    for (int i = 0; i < 6; i++)
        nc_free_tensor(n->saved[i]);
    nc_free_tensor(n->grad);
    free(n->parents);
    free(n->sizes);
    free(n);
}

int nc_needs_grad(NCTensor **args, int n)
{
    for (int i = 0; i < n; i++)
        if (args[i] && args[i]->node)
            return 1;
    return 0;
}

static NCContext *ctx_of(NCTensor **args, int n)
{
    for (int i = 0; i < n; i++)
        if (args[i])
            return args[i]->dev->ctx;
    return NULL;
}

/* a node is always created; it costs little and keeps the code uniform */
NCNode *nc_new_node(NCContext *m, NCOpEnum op, int n_args, NCTensor **args)
{
    NCNode *n = nc_mallocz(sizeof(*n));
    n->ref = 1;
    n->op = op;
    n->seq = m ? m->node_seq++ : 0;
    n->n_args = n_args;
    n->parents = nc_mallocz(sizeof(NCNode *) * (n_args ? n_args : 1));
    for (int i = 0; i < n_args; i++) {
        if (!args || !args[i])
            continue;
        n->parents[i] = nc_dup_node(args[i]->node);
        if (i < NC_MAX_ARGS) {
            n->arg_ndims[i] = args[i]->n_dims;
            memcpy(n->arg_dims[i], args[i]->dims, sizeof(size_t) * args[i]->n_dims);
        }
    }
    return n;
}

void nc_attach(NCTensor *y, NCNode *n)
{
    nc_free_node(y->node);
    y->node = n;
    n->out_ndims = y->n_dims;
    memcpy(n->out_dims, y->dims, sizeof(size_t) * y->n_dims);
}

/* drop the node again when no argument carries a graph */
static NCTensor *finish(NCTensor *y, NCNode *n, NCTensor **args, int n_args)
{
    if (nc_needs_grad(args, n_args)) {
        nc_attach(y, n);
    } else {
        nc_free_node(n);
    }
    return y;
}

NCTensor *nc_set_param(NCTensor *x, void *opaque) /* libnc.h:457 */
{
    NCNode *n = nc_new_node(x->dev->ctx, OP_PARAM, 0, NULL);
    n->opaque = opaque;
    nc_attach(x, n);
    return x;
}

/* libnc.h:470: force tensor x to be the saved argument arg_index of node n
   (nncp.c:827, 860) */
void nc_node_set_arg(NCNode *n, int arg_index, const NCTensor *x)
{
    nc_free_tensor(n->saved[arg_index]);
    n->saved[arg_index] = nc_view(x);
}

/* libnc.h:469: the gradient of argument arg_index of n is delivered to n1
   (nncp.c:1137, 1152) */
void nc_node_set_parent(NCNode *n, int arg_index, const NCNode *n1)
{
    nc_free_node(n->parents[arg_index]);
    n->parents[arg_index] = nc_dup_node(n1);
}

/* libnc.h:466: synthetic node; the gradient it receives is split along
   'axis' into pieces of tab_size[] and handed to inputs[] (nncp.c:1128-1131) */
NCNode *nc_concat_node(NCContext *m, NCNode **inputs, int count, int axis,
                       const size_t *tab_size)
{
    NCNode *n = nc_new_node(m, OP_CONCAT_NODE, count, NULL);
    for (int i = 0; i < count; i++)
        n->parents[i] = nc_dup_node(inputs[i]);
    n->ia[0] = axis;
    n->sizes = nc_malloc(sizeof(size_t) * count);
    memcpy(n->sizes, tab_size, sizeof(size_t) * count);
    return n;
}

/* libnc.h:468: a permission to merge sibling backward passes; no semantics */
void nc_concat_optimization(NCContext *m, NCNode **nodes, int count)
{
    (void)m; (void)nodes; (void)count;
}

void nc_combine_nodes(NCContext *m, NCNode **tab, int count, int axis,
                      int elem_size, const size_t *tab_elem_size)
{
    /* LSTM-only optimisation hint (nncp.c:2111-2114); no semantics */
    (void)m; (void)tab; (void)count; (void)axis; (void)elem_size; (void)tab_elem_size;
}

/* ------------------------------------------------------------------------ */
/* small helpers                                                            */

static NCTensor *new_out(const NCTensor *like, int n_dims, const size_t *dims)
{
    return nc_alloc(like->dev, NC_TYPE_F32, n_dims, dims, 0);
}

static void need_f32(const NCTensor *x, const char *op)
{
    if (x->type != NC_TYPE_F32)
        nc_fatal("%s: f32 tensor expected (type %d)", op, x->type);
}

/* broadcast plan: out dims and per-operand strides (0 on broadcast axes) */
typedef struct {
    int nd;
    size_t dims[NC_N_DIMS_MAX], sa[NC_N_DIMS_MAX], sb[NC_N_DIMS_MAX], n;
} BCast;

static void bcast_plan(BCast *bc, int na, const size_t *da, int nb, const size_t *db,
                       const char *op)
{
    size_t stra = 1, strb = 1;
    bc->nd = na > nb ? na : nb;
    bc->n = 1;
    for (int i = 0; i < bc->nd; i++) {
        size_t a = i < na ? da[i] : 1, b = i < nb ? db[i] : 1;
        if (a != b && a != 1 && b != 1)
            nc_fatal("%s: incompatible shapes on axis %d (%zu vs %zu)", op, i, a, b);
        bc->dims[i] = a > b ? a : b;
        bc->sa[i] = (a == 1) ? 0 : stra;
        bc->sb[i] = (b == 1) ? 0 : strb;
        stra *= a;
        strb *= b;
        bc->n *= bc->dims[i];
    }
}

/* true when operand b (nb dims) equals the leading axes of the result, so
   that its element index is simply io % numel(b) */
static int bcast_prefix(const BCast *bc, int nb, const size_t *db)
{
    for (int i = 0; i < nb; i++)
        if (db[i] != bc->dims[i]) {
            /* trailing size-1 axes of b are fine */
            for (int j = i; j < nb; j++)
                if (db[j] != 1)
                    return 0;
            break;
        }
    return 1;
}

#define BCAST_LOOP(bc, ia, ib, io, BODY)                                     \
    do {                                                                     \
        size_t idx_[NC_N_DIMS_MAX] = { 0 }, ia = 0, ib = 0;                  \
        for (size_t io = 0; io < (bc)->n; io++) {                            \
            BODY;                                                            \
            for (int a_ = 0; a_ < (bc)->nd; a_++) {                          \
                idx_[a_]++; ia += (bc)->sa[a_]; ib += (bc)->sb[a_];          \
                if (idx_[a_] < (bc)->dims[a_]) break;                        \
                ia -= (bc)->sa[a_] * (bc)->dims[a_];                         \
                ib -= (bc)->sb[a_] * (bc)->dims[a_];                         \
                idx_[a_] = 0;                                                \
            }                                                                \
        }                                                                    \
    } while (0)

/* sum g (shape gd) down to shape td (td[i] == gd[i] or 1 / missing) */
static NCTensor *unbroadcast(NCTensor *g, int tn, const size_t *td)
{
    BCast bc;
    NCTensor *y;
    size_t nt = 1;
    for (int i = 0; i < tn; i++)
        nt *= td[i];
    if (nt == nc_numel(g)) {
        /* same element count: only the header changes */
        y = nc_view(g);
        y->n_dims = tn;
        size_t s = 1;
        for (int i = 0; i < tn; i++) { y->dims[i] = td[i]; y->strides[i] = s; s *= td[i]; }
        nc_free_tensor(g);
        return y;
    }
    bcast_plan(&bc, g->n_dims, g->dims, tn, td, "unbroadcast");
    y = nc_alloc(g->dev, NC_TYPE_F32, tn, td, 1);
    {
        const float *gp = nc_f32(g);
        float *yp = nc_f32(y);
        BCAST_LOOP(&bc, ia, ib, io, yp[ib] += gp[ia]);
    }
    nc_free_tensor(g);
    return y;
}

/* ------------------------------------------------------------------------ */
/* element-wise                                                             */

static NCTensor *binary_op(NCTensor *a, NCTensor *b, NCOpEnum op)
{
    BCast bc;
    NCTensor *args[2], *y;
    NCNode *n;
    a = nc_contig(a); b = nc_contig(b);
    need_f32(a, "binary"); need_f32(b, "binary");
    bcast_plan(&bc, a->n_dims, a->dims, b->n_dims, b->dims, op == OP_ADD ? "add" : "mul");
    y = new_out(a, bc.nd, bc.dims);
    {
        const float *ap = nc_f32(a), *bp = nc_f32(b);
        float *yp = nc_f32(y);
        size_t nb = nc_numel(b);
        if (nc_numel(a) == bc.n && bcast_prefix(&bc, b->n_dims, b->dims)) {
            /* b is a leading-axes prefix of a (same shape, vector or scalar) */
            if (op == OP_ADD) for (size_t i = 0; i < bc.n; i++) yp[i] = ap[i] + bp[i % nb];
            else for (size_t i = 0; i < bc.n; i++) yp[i] = ap[i] * bp[i % nb];
        } else if (op == OP_ADD) {
            BCAST_LOOP(&bc, ia, ib, io, yp[io] = ap[ia] + bp[ib]);
        } else {
            BCAST_LOOP(&bc, ia, ib, io, yp[io] = ap[ia] * bp[ib]);
        }
    }
    args[0] = a; args[1] = b;
    n = nc_new_node(ctx_of(args, 2), op, 2, args);
    if (op == OP_MUL && nc_needs_grad(args, 2)) {
        n->saved[0] = nc_view(a);
        n->saved[1] = nc_view(b);
    }
    y = finish(y, n, args, 2);
    nc_free_tensor(a); nc_free_tensor(b);
    return y;
}

NCTensor *nc_add(NCTensor *x1, NCTensor *x2) { return binary_op(x1, x2, OP_ADD); } /* libnc.h:232 */
NCTensor *nc_mul(NCTensor *x1, NCTensor *x2) { return binary_op(x1, x2, OP_MUL); } /* libnc.h:235 */

/* libnc.h:231.  Two item types carry values here: F32 and BF16 (2 bytes, the storage type of
   parameters under nncp's bf16 switch, nncp.c:343-346).  Arithmetic is always F32: every op
   widens a BF16 operand first (nc_operand, exact) and gives an F32 result; F32 -> BF16 rounds
   to nearest even.  The gradient passes through a conversion unchanged, as F32. */
static NCTensor *convert_to(NCTensor *x, NCTypeEnum new_type)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t cnt;
    x = (nc_contig)(x);
    y = nc_alloc(x->dev, new_type, x->n_dims, x->dims, 0);
    cnt = nc_numel(x);
    if (new_type == NC_TYPE_F32) {
        const uint16_t *src = (const uint16_t *)x->buf->data + x->off;
        for (size_t i = 0; i < cnt; i++)
            nc_f32(y)[i] = nc_bf16_widen(src[i]);
    } else {
        uint16_t *dst = (uint16_t *)y->buf->data + y->off;
        for (size_t i = 0; i < cnt; i++)
            dst[i] = nc_bf16_bits(nc_f32(x)[i]);
    }
    args[0] = x;
    n = nc_new_node(x->dev->ctx, OP_CONVERT, 1, args);
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

NCTensor *nc_convert(NCTensor *x, NCTypeEnum new_type)
{
    if (x->type == new_type)
        return x;
    if ((x->type == NC_TYPE_BF16 && new_type == NC_TYPE_F32) ||
        (x->type == NC_TYPE_F32 && new_type == NC_TYPE_BF16))
        return convert_to(x, new_type);
    nc_fatal("convert: %d -> %d is not supported (f32 and bf16 only)", x->type, new_type);
}

/* what every op does to an operand: contiguous, and F32 if it was BF16 (consumes x) */
NCTensor *nc_operand(NCTensor *x)
{
    if (x->type == NC_TYPE_BF16)
        return convert_to(x, NC_TYPE_F32);
    return (nc_contig)(x);
}

/* libnc.h:242-244: y = mask ? c : x, mask broadcast over the trailing axes */
NCTensor *nc_masked_fill(NCTensor *x, NCTensor *mask, float c, BOOL mask_inv)
{
    BCast bc;
    NCTensor *y, *args[1];
    NCNode *n;
    x = nc_contig(x); mask = nc_contig(mask);
    need_f32(x, "masked_fill");
    if (mask->type != NC_TYPE_I8)
        nc_fatal("masked_fill: i8 mask expected");
    bcast_plan(&bc, x->n_dims, x->dims, mask->n_dims, mask->dims, "masked_fill");
    y = nc_alloc_like(x);
    {
        const float *xp = nc_f32(x);
        const int8_t *mp = (const int8_t *)mask->buf->data + mask->off;
        float *yp = nc_f32(y);
        if (bcast_prefix(&bc, mask->n_dims, mask->dims)) {
            size_t nm = nc_numel(mask);
            for (size_t i = 0; i < bc.n; i++)
                yp[i] = ((mp[i % nm] != 0) != (mask_inv != 0)) ? c : xp[i];
        } else {
            BCAST_LOOP(&bc, ia, ib, io, yp[io] = ((mp[ib] != 0) != (mask_inv != 0)) ? c : xp[ia]);
        }
    }
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_MASKED_FILL, 1, args);
    n->saved[0] = nc_view(mask);
    n->ia[0] = mask_inv != 0;
    y = finish(y, n, args, 1);
    nc_free_tensor(x); nc_free_tensor(mask);
    return y;
}

static inline float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

#define GELU_C0 0.7978845608f
#define GELU_C1 0.044715f

/* tanh-form GELU (build-defined choice; every restatement in the reference
   tree uses it: src/metal/compute/matrix_ops.metal:90-101,
   src/neural/compatibility/cuda_math_compat.c:349-368) */
static inline float gelu_f(float x)
{
    return 0.5f * x * (1.0f + tanhf(GELU_C0 * (x + GELU_C1 * x * x * x)));
}

static inline float gelu_grad_f(float x)
{
    float t = tanhf(GELU_C0 * (x + GELU_C1 * x * x * x));
    return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * GELU_C0 * (1.0f + 3.0f * GELU_C1 * x * x);
}

static NCTensor *unary_op(NCTensor *x, NCOpEnum op)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t cnt;
    x = nc_contig(x);
    need_f32(x, "unary");
    y = nc_alloc_like(x);
    cnt = nc_numel(x);
    const float *xp = nc_f32(x);
    float *yp = nc_f32(y);
    #pragma omp parallel for if (cnt > 65536)
    for (size_t i = 0; i < cnt; i++) {
        float v = xp[i];
        switch (op) {
        case OP_SIGMOID: v = sigmoidf_(v); break;
        case OP_TANH: v = tanhf(v); break;
        case OP_RELU: v = v > 0 ? v : 0; break;
        case OP_GELU: v = gelu_f(v); break;
        default: break;
        }
        yp[i] = v;
    }
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), op, 1, args);
    if (x->node)
        n->saved[0] = nc_view(x);
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

NCTensor *nc_sigmoid(NCTensor *x) { return unary_op(x, OP_SIGMOID); } /* libnc.h:245 */
NCTensor *nc_tanh(NCTensor *x) { return unary_op(x, OP_TANH); }       /* libnc.h:246 */
NCTensor *nc_relu(NCTensor *x) { return unary_op(x, OP_RELU); }       /* libnc.h:247 */
NCTensor *nc_gelu(NCTensor *x) { return unary_op(x, OP_GELU); }       /* libnc.h:252 */

static void same_shape(const NCTensor *a, const NCTensor *b, const char *op)
{
    if (nc_numel(a) != nc_numel(b))
        nc_fatal("%s: operands must have the same shape", op);
}

/* libnc.h:249-251: g * x * sigmoid(beta * x) */
NCTensor *nc_gated_swish(NCTensor *g, NCTensor *x, float beta)
{
    NCTensor *y, *args[2];
    NCNode *n;
    g = nc_contig(g); x = nc_contig(x);
    same_shape(g, x, "gated_swish");
    y = nc_alloc_like(x);
    size_t cnt = nc_numel(x);
    for (size_t i = 0; i < cnt; i++)
        nc_f32(y)[i] = nc_f32(g)[i] * nc_f32(x)[i] * sigmoidf_(beta * nc_f32(x)[i]);
    args[0] = g; args[1] = x;
    n = nc_new_node(ctx_of(args, 2), OP_GATED_SWISH, 2, args);
    n->saved[0] = nc_view(g); n->saved[1] = nc_view(x);
    n->fa[0] = beta;
    y = finish(y, n, args, 2);
    nc_free_tensor(g); nc_free_tensor(x);
    return y;
}

/* libnc.h:261-263: cp * fg + min(1 - fg, ig) * in */
NCTensor *nc_lstm_clamped(NCTensor *cp, NCTensor *in, NCTensor *fg, NCTensor *ig)
{
    NCTensor *y, *args[4];
    NCNode *n;
    cp = nc_contig(cp); in = nc_contig(in); fg = nc_contig(fg); ig = nc_contig(ig);
    same_shape(cp, in, "lstm_clamped"); same_shape(cp, fg, "lstm_clamped"); same_shape(cp, ig, "lstm_clamped");
    y = nc_alloc_like(cp);
    size_t cnt = nc_numel(cp);
    for (size_t i = 0; i < cnt; i++)
        nc_f32(y)[i] = nc_f32(cp)[i] * nc_f32(fg)[i] +
                       fminf(1.0f - nc_f32(fg)[i], nc_f32(ig)[i]) * nc_f32(in)[i];
    args[0] = cp; args[1] = in; args[2] = fg; args[3] = ig;
    n = nc_new_node(ctx_of(args, 4), OP_LSTM_CLAMPED, 4, args);
    for (int i = 0; i < 4; i++)
        n->saved[i] = nc_view(args[i]);
    y = finish(y, n, args, 4);
    for (int i = 0; i < 4; i++)
        nc_free_tensor(args[i]);
    return y;
}

/* libnc.h:272-273: a * (1 - t) + b * t */
NCTensor *nc_lerp(NCTensor *a, NCTensor *b, NCTensor *t)
{
    NCTensor *y, *args[3];
    NCNode *n;
    a = nc_contig(a); b = nc_contig(b); t = nc_contig(t);
    same_shape(a, b, "lerp"); same_shape(a, t, "lerp");
    y = nc_alloc_like(a);
    size_t cnt = nc_numel(a);
    for (size_t i = 0; i < cnt; i++)
        nc_f32(y)[i] = nc_f32(a)[i] * (1.0f - nc_f32(t)[i]) + nc_f32(b)[i] * nc_f32(t)[i];
    args[0] = a; args[1] = b; args[2] = t;
    n = nc_new_node(ctx_of(args, 3), OP_LERP, 3, args);
    for (int i = 0; i < 3; i++)
        n->saved[i] = nc_view(args[i]);
    y = finish(y, n, args, 3);
    for (int i = 0; i < 3; i++)
        nc_free_tensor(args[i]);
    return y;
}

/* ------------------------------------------------------------------------ */
/* shape ops                                                                */

static NCTensor *reshape_nd(NCTensor *x, int nd, const size_t *dims)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t cnt = 1, s = 1;
    x = nc_contig(x);
    for (int i = 0; i < nd; i++)
        cnt *= dims[i];
    if (cnt != nc_numel(x))
        nc_fatal("reshape: element count mismatch (%zu vs %zu)", cnt, nc_numel(x));
    y = nc_view(x);
    y->n_dims = nd;
    for (int i = 0; i < nd; i++) { y->dims[i] = dims[i]; y->strides[i] = s; s *= dims[i]; }
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_RESHAPE, 1, args);
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

/* libnc.h:282-286 */
NCTensor *nc_reshape_1d(NCTensor *x, size_t n0) { size_t d[1] = { n0 }; return reshape_nd(x, 1, d); }
NCTensor *nc_reshape_2d(NCTensor *x, size_t n0, size_t n1) { size_t d[2] = { n0, n1 }; return reshape_nd(x, 2, d); }
NCTensor *nc_reshape_3d(NCTensor *x, size_t n0, size_t n1, size_t n2) { size_t d[3] = { n0, n1, n2 }; return reshape_nd(x, 3, d); }
NCTensor *nc_reshape_4d(NCTensor *x, size_t n0, size_t n1, size_t n2, size_t n3) { size_t d[4] = { n0, n1, n2, n3 }; return reshape_nd(x, 4, d); }

/* libnc.h:289-292: duplicate the tensor by appending new trailing axes */
static NCTensor *repeat_nd(NCTensor *x, int nr, const size_t *rd)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t dims[NC_N_DIMS_MAX], cnt, rep = 1;
    x = nc_contig(x);
    need_f32(x, "repeat");
    memcpy(dims, x->dims, sizeof(size_t) * x->n_dims);
    for (int i = 0; i < nr; i++) { dims[x->n_dims + i] = rd[i]; rep *= rd[i]; }
    y = new_out(x, x->n_dims + nr, dims);
    cnt = nc_numel(x);
    for (size_t r = 0; r < rep; r++)
        memcpy(nc_f32(y) + r * cnt, nc_f32(x), cnt * sizeof(float));
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_REPEAT, 1, args);
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

NCTensor *nc_repeat_1d(NCTensor *x, size_t n0) { size_t d[1] = { n0 }; return repeat_nd(x, 1, d); }
NCTensor *nc_repeat_2d(NCTensor *x, size_t n0, size_t n1) { size_t d[2] = { n0, n1 }; return repeat_nd(x, 2, d); }

/* libnc.h:293-295: y0 + sum of x over the axes >= n_dims; y0 may be NULL */
NCTensor *nc_reduce_sum(NCTensor *y0, NCTensor *x, int n_dims)
{
    NCTensor *y, *args[2];
    NCNode *n;
    size_t inner = 1, outer;
    x = nc_contig(x);
    need_f32(x, "reduce_sum");
    for (int i = 0; i < n_dims; i++)
        inner *= x->dims[i];
    outer = nc_numel(x) / inner;
    y = nc_alloc(x->dev, NC_TYPE_F32, n_dims, x->dims, 1);
    if (y0) {
        y0 = nc_contig(y0);
        memcpy(nc_f32(y), nc_f32(y0), inner * sizeof(float));
    }
    for (size_t o = 0; o < outer; o++)
        for (size_t i = 0; i < inner; i++)
            nc_f32(y)[i] += nc_f32(x)[o * inner + i];
    args[0] = y0; args[1] = x;
    n = nc_new_node(ctx_of(args, 2), OP_REDUCE_SUM, 2, args);
    y = finish(y, n, args, 2);
    nc_free_tensor(y0); nc_free_tensor(x);
    return y;
}

/* libnc.h:298-299: sum of all the elements -> 0-dim tensor */
NCTensor *nc_sum(NCTensor *x)
{
    NCTensor *y, *args[1];
    NCNode *n;
    double s = 0;
    x = nc_contig(x);
    need_f32(x, "sum");
    size_t cnt = nc_numel(x);
    for (size_t i = 0; i < cnt; i++)
        s += nc_f32(x)[i];
    y = nc_new_f32(x->dev, (float)s);
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_SUM, 1, args);
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

/* libnc.h:306-307: alias (shares storage, carries no graph).  Writing through
   it with nc_tensor_copy mutates the parent (nncp.c:650-657, 697-702). */
NCTensor *nc_slice_alias(const NCTensor *x, int axis, size_t start, size_t end)
{
    NCTensor *y;
    if (axis >= x->n_dims || end > x->dims[axis] || start > end)
        nc_fatal("slice_alias: range [%zu,%zu) outside axis %d of size %zu", start, end, axis,
                 axis < x->n_dims ? x->dims[axis] : 0);
    y = nc_view(x);
    y->off += start * x->strides[axis];
    y->dims[axis] = end - start;
    return y;
}

/* libnc.h:308: copying slice that stays in the graph */
NCTensor *nc_slice(NCTensor *x, int axis, size_t start, size_t end)
{
    NCTensor *v, *y, *args[1];
    NCNode *n;
    v = nc_slice_alias(x, axis, start, end);
    y = nc_alloc(x->dev, x->type, v->n_dims, v->dims, 0);
    nc_copy_strided(y, v);
    nc_free_tensor(v);
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_SLICE, 1, args);
    n->ia[0] = axis; n->ia[1] = (int)start;
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

/* libnc.h:310-317 */
NCTensor *nc_concat(NCTensor **inputs, int n_inputs, int axis)
{
    NCTensor *y;
    NCNode *n;
    size_t dims[NC_N_DIMS_MAX], total = 0, pos = 0;
    int nd = inputs[0]->n_dims;
    if (axis >= nd)
        nc_fatal("concat: axis %d out of range", axis);
    memcpy(dims, inputs[0]->dims, sizeof(size_t) * nd);
    for (int i = 0; i < n_inputs; i++) {
        if (inputs[i]->n_dims != nd)
            nc_fatal("concat: rank mismatch");
        for (int a = 0; a < nd; a++)
            if (a != axis && inputs[i]->dims[a] != dims[a])
                nc_fatal("concat: shape mismatch on axis %d", a);
        total += inputs[i]->dims[axis];
    }
    dims[axis] = total;
    y = nc_alloc(inputs[0]->dev, inputs[0]->type, nd, dims, 0);
    n = nc_new_node(ctx_of(inputs, n_inputs), OP_CONCAT, n_inputs, NULL);
    n->sizes = nc_malloc(sizeof(size_t) * n_inputs);
    n->ia[0] = axis;
    for (int i = 0; i < n_inputs; i++) {
        NCTensor *v = nc_slice_alias(y, axis, pos, pos + inputs[i]->dims[axis]);
        nc_copy_strided(v, inputs[i]);
        nc_free_tensor(v);
        n->sizes[i] = inputs[i]->dims[axis];
        n->parents[i] = nc_dup_node(inputs[i]->node);
        pos += inputs[i]->dims[axis];
    }
    y = finish(y, n, inputs, n_inputs);
    for (int i = 0; i < n_inputs; i++)
        nc_free_tensor(inputs[i]);
    return y;
}

NCTensor *nc_vconcat(NCTensor **inputs, int n) { return nc_concat(inputs, n, 0); }
NCTensor *nc_hconcat(NCTensor **inputs, int n) { return nc_concat(inputs, n, 1); }

/* libnc.h:318-320: split along 'axis', equally when tab_size is NULL */
void nc_split(NCTensor **tab_y, NCTensor *x, int n_outputs, const size_t *tab_size, int axis)
{
    size_t pos = 0;
    for (int i = 0; i < n_outputs; i++) {
        size_t sz = tab_size ? tab_size[i] : x->dims[axis] / n_outputs;
        tab_y[i] = nc_slice(nc_dup_tensor(x), axis, pos, pos + sz);
        pos += sz;
    }
    nc_free_tensor(x);
}

/* libnc.h:325-335: pad (len > 0) or trim (len < 0) axis 0.  PAD_DUP repeats
   the edge element, TRIM_SUM adds the trimmed elements to the new edge (the
   adjoint of PAD_DUP).  nncp.c:777 left-pads R from d_pos to K rows. */
static void pad_map(size_t n_in, ssize_t left, int lop, ssize_t right, int rop,
                    const float *x, float *y, int adjoint)
{
    /* forward: y[(n_in+left+right)] from x[n_in]; adjoint: x += from y */
    ssize_t n_out = (ssize_t)n_in + left + right;
    if (!adjoint)
        memset(y, 0, sizeof(float) * n_out);
    for (ssize_t i = 0; i < n_out; i++) {
        ssize_t s = i - left; /* source index for the plain copy */
        if (s < 0) {
            if (lop != NC_PAD_DUP) continue;
            s = 0;
        } else if (s >= (ssize_t)n_in) {
            if (rop != NC_PAD_DUP) continue;
            s = n_in - 1;
        }
        if (!adjoint) y[i] += x[s];
        else ((float *)x)[s] += y[i];
    }
    /* TRIM_SUM: trimmed input elements are added to the nearest kept edge */
    if (left < 0 && lop == NC_TRIM_SUM)
        for (ssize_t s = 0; s < -left; s++) {
            if (!adjoint) y[0] += x[s];
            else ((float *)x)[s] += y[0];
        }
    if (right < 0 && rop == NC_TRIM_SUM)
        for (ssize_t s = (ssize_t)n_in + right; s < (ssize_t)n_in; s++) {
            if (!adjoint) y[n_out - 1] += x[s];
            else ((float *)x)[s] += y[n_out - 1];
        }
}

NCTensor *nc_pad(NCTensor *x, ssize_t left_len, NCPadEnum left_op,
                 ssize_t right_len, NCPadEnum right_op)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t dims[NC_N_DIMS_MAX], cols;
    x = nc_contig(x);
    need_f32(x, "pad");
    memcpy(dims, x->dims, sizeof(size_t) * x->n_dims);
    if ((ssize_t)dims[0] + left_len + right_len <= 0)
        nc_fatal("pad: empty result");
    dims[0] = dims[0] + left_len + right_len;
    y = new_out(x, x->n_dims, dims);
    cols = nc_numel(x) / x->dims[0];
    for (size_t c = 0; c < cols; c++)
        pad_map(x->dims[0], left_len, left_op, right_len, right_op,
                nc_f32(x) + c * x->dims[0], nc_f32(y) + c * dims[0], 0);
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_PAD, 1, args);
    n->ia[0] = (int)left_len; n->ia[1] = left_op; n->ia[2] = (int)right_len; n->ia[3] = right_op;
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

/* libnc.h:353-360: permute and make contiguous; result axis i is x axis
   axis[i] */
static NCTensor *permute_raw(const NCTensor *x, int nd, const int *axis)
{
    NCTensor *v = nc_view(x), *y;
    if (nd != x->n_dims)
        nc_fatal("permute: rank mismatch");
    for (int i = 0; i < nd; i++) {
        v->dims[i] = x->dims[axis[i]];
        v->strides[i] = x->strides[axis[i]];
    }
    y = nc_alloc(x->dev, x->type, nd, v->dims, 0);
    nc_copy_strided(y, v);
    nc_free_tensor(v);
    return y;
}

NCTensor *nc_permute(NCTensor *x, int n_dims, const int *axis)
{
    NCTensor *y, *args[1];
    NCNode *n;
    x = nc_contig(x);
    y = permute_raw(x, n_dims, axis);
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_PERMUTE, 1, args);
    for (int i = 0; i < n_dims; i++)
        n->ia[i] = axis[i];
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

NCTensor *nc_permute_4d(NCTensor *x, int a0, int a1, int a2, int a3)
{
    int axis[4] = { a0, a1, a2, a3 };
    return nc_permute(x, 4, axis);
}

/* libnc.h:396-397: column i (axis 1) is shifted by s = pos + i*mult elements
   along axis 0, zero filled: y[j,i] = x[j - s, i].  With pos = -(T-1),
   mult = 1 (nncp.c:784) row K-1 of column i ends up holding distance 0, which
   is the only reading consistent with the mask of nncp.c:355-363. */
static void rel_shift_raw(const float *x, float *y, size_t n0, size_t n1, size_t outer,
                          ssize_t pos, ssize_t mult, int adjoint)
{
    for (size_t o = 0; o < outer; o++)
        for (size_t i = 0; i < n1; i++) {
            ssize_t s = pos + (ssize_t)i * mult;
            const float *xc = x + (o * n1 + i) * n0;
            float *yc = y + (o * n1 + i) * n0;
            for (ssize_t j = 0; j < (ssize_t)n0; j++) {
                ssize_t src = adjoint ? j + s : j - s;
                yc[j] = (src >= 0 && src < (ssize_t)n0) ? xc[src] : 0.0f;
            }
        }
}

NCTensor *nc_rel_shift(NCTensor *x, ssize_t pos, ssize_t mult)
{
    NCTensor *y, *args[1];
    NCNode *n;
    x = nc_contig(x);
    need_f32(x, "rel_shift");
    if (x->n_dims < 2)
        nc_fatal("rel_shift: at least 2 axes expected");
    y = nc_alloc_like(x);
    rel_shift_raw(nc_f32(x), nc_f32(y), x->dims[0], x->dims[1],
                  nc_numel(x) / (x->dims[0] * x->dims[1]), pos, mult, 0);
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_REL_SHIFT, 1, args);
    n->ia[0] = (int)pos; n->ia[1] = (int)mult;
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

NCTensor *nc_cmul(NCTensor *x1, NCTensor *x2, BOOL is_conj, BOOL is_planar)
{
    (void)x1; (void)x2; (void)is_conj; (void)is_planar;
    nc_fatal("cmul (rotary position embedding, nncp.c:764-770) is not supported");
}

/* ------------------------------------------------------------------------ */
/* matmul                                                                   */

static int g_matmul_bf16;

int nc_set_matmul_bf16(NCContext *m, int enable)
{
    int old = g_matmul_bf16;
    (void)m;
    g_matmul_bf16 = enable;
    return old;
}

static float bf16_round(float f)
{
    union { float f; uint32_t u; } v = { f };
    v.u += 0x7fff + ((v.u >> 16) & 1);
    v.u &= 0xffff0000u;
    return v.f;
}

static NCTensor *maybe_bf16(NCTensor *x)
{
    if (!g_matmul_bf16)
        return nc_dup_tensor(x);
    NCTensor *y = nc_alloc_like(x);
    size_t n = nc_numel(x);
    for (size_t i = 0; i < n; i++)
        nc_f32(y)[i] = bf16_round(nc_f32(x)[i]);
    return y;
}

/* batched gemm on contiguous tensors; batch = product of axes >= 2 */
static void gemm_batched(int ta, int tb, size_t m, size_t n, size_t k, float alpha,
                         NCTensor *a, NCTensor *b, float beta, NCTensor *c, size_t batch,
                         int a_bcast)
{
    NCTensor *ar = maybe_bf16(a), *br = maybe_bf16(b);
    size_t sa = a_bcast ? 0 : m * k, sb = k * n, sc = m * n;
    for (size_t bi = 0; bi < batch; bi++)
        ref_sgemm(ta, tb, (int)m, (int)n, (int)k, alpha,
                  nc_f32(ar) + bi * sa, (int)(ta ? k : m),
                  nc_f32(br) + bi * sb, (int)(tb ? n : k),
                  beta, nc_f32(c) + bi * sc, (int)m);
    nc_free_tensor(ar); nc_free_tensor(br);
}

/* libnc.h:365-373: alpha * op(a) * op(b) + c on the first two axes, batched
   over identical trailing axes.  A 2-D 'a' against an n-D untransposed 'b' is
   applied to every column of b. */
NCTensor *nc_matmul_add(NCTensor *a, NCTensor *b, NCTensor *c, BOOL ta, BOOL tb, float alpha)
{
    NCTensor *y, *args[3];
    NCNode *nd;
    size_t m, k, kb, n, batch = 1, dims[NC_N_DIMS_MAX];
    int flat = 0, out_nd;
    a = nc_contig(a); b = nc_contig(b);
    need_f32(a, "matmul"); need_f32(b, "matmul");
    if (a->n_dims < 2 || b->n_dims < 2)
        nc_fatal("matmul: operands need at least 2 axes");
    m = ta ? a->dims[1] : a->dims[0];
    k = ta ? a->dims[0] : a->dims[1];
    if (a->n_dims == 2 && b->n_dims > 2 && !tb) {
        flat = 1;
        kb = b->dims[0];
        n = nc_numel(b) / kb;
    } else {
        if (a->n_dims != b->n_dims)
            nc_fatal("matmul: rank mismatch (%d vs %d)", a->n_dims, b->n_dims);
        for (int i = 2; i < a->n_dims; i++) {
            if (a->dims[i] != b->dims[i])
                nc_fatal("matmul: batch axis %d mismatch", i);
            batch *= a->dims[i];
        }
        kb = tb ? b->dims[1] : b->dims[0];
        n = tb ? b->dims[0] : b->dims[1];
    }
    if (k != kb)
        nc_fatal("matmul: inner dimension mismatch (%zu vs %zu)", k, kb);
    out_nd = b->n_dims;
    memcpy(dims, b->dims, sizeof(size_t) * b->n_dims);
    dims[0] = m;
    if (!flat)
        dims[1] = n;
    y = nc_alloc(a->dev, NC_TYPE_F32, out_nd, dims, 0);
    if (c) {
        c = nc_contig(c);
        if (nc_numel(c) != nc_numel(y))
            nc_fatal("matmul_add: addend shape mismatch");
        memcpy(nc_f32(y), nc_f32(c), nc_numel(y) * sizeof(float));
    }
    gemm_batched(ta, tb, m, n, k, alpha, a, b, c ? 1.0f : 0.0f, y, batch, 0);
    args[0] = a; args[1] = b; args[2] = c;
    nd = nc_new_node(ctx_of(args, 3), OP_MATMUL, 3, args);
    nd->saved[0] = nc_view(a);
    nd->saved[1] = nc_view(b);
    nd->ia[0] = ta != 0; nd->ia[1] = tb != 0; nd->ia[2] = flat;
    nd->fa[0] = alpha;
    y = finish(y, nd, args, 3);
    nc_free_tensor(a); nc_free_tensor(b); nc_free_tensor(c);
    return y;
}

NCTensor *nc_matmul(NCTensor *w, NCTensor *x) { return nc_matmul_add(w, x, NULL, 0, 0, 1.0f); }

static void matmul_bw(NCNode *nd, NCTensor *g, NCTensor **ga)
{
    NCTensor *a = nd->saved[0], *b = nd->saved[1];
    int ta = nd->ia[0], tb = nd->ia[1], flat = nd->ia[2];
    float alpha = nd->fa[0];
    size_t m = ta ? a->dims[1] : a->dims[0], k = ta ? a->dims[0] : a->dims[1];
    size_t n, batch = 1;
    if (flat) {
        n = nc_numel(b) / k;
    } else {
        n = tb ? b->dims[0] : b->dims[1];
        for (int i = 2; i < a->n_dims; i++)
            batch *= a->dims[i];
    }
    if (nd->parents[0]) {
        NCTensor *da = nc_alloc_like(a);
        if (!ta) /* dA(m,k) = dY(m,n) * op(B)^T */
            gemm_batched(0, !tb, m, k, n, alpha, g, b, 0.0f, da, batch, 0);
        else     /* dA(k,m) = op(B)(k,n) * dY^T(n,m) */
            gemm_batched(tb, 1, k, m, n, alpha, b, g, 0.0f, da, batch, 0);
        ga[0] = da;
    }
    if (nd->parents[1]) {
        NCTensor *db = nc_alloc_like(b);
        if (!tb) /* dB(k,n) = op(A)^T(k,m) * dY(m,n) */
            gemm_batched(!ta, 0, k, n, m, alpha, a, g, 0.0f, db, batch, 0);
        else     /* dB(n,k) = dY^T(n,m) * op(A)(m,k) */
            gemm_batched(1, ta, n, k, m, alpha, g, a, 0.0f, db, batch, 0);
        ga[1] = db;
    }
    if (nd->parents[2])
        ga[2] = nc_dup_tensor(g);
}

/* y = act(w x + bias): the fused form of nncp.c:930-943 (see nc_ext.h) */
NCTensor *nc_linear(NCTensor *w, NCTensor *x, NCTensor *bias, int act)
{
    NCTensor *y = nc_matmul(w, x);
    if (bias)
        y = nc_add(y, bias);
    if (act == NC_ACT_GELU)
        y = nc_gelu(y);
    else if (act == NC_ACT_RELU)
        y = nc_relu(y);
    return y;
}

/* y = act(w x + bias) + res: a linear layer with its residual connection
   (nncp.c:896, 979; see nc_ext.h) */
NCTensor *nc_linear_add(NCTensor *w, NCTensor *x, NCTensor *bias, int act, NCTensor *res)
{
    return nc_add(nc_linear(w, x, bias, act), res);
}

/* ------------------------------------------------------------------------ */
/* embedding, softmax, loss, norms                                          */

/* libnc.h:374-375: columns of w (D,V) selected by the i32 indices x (n) */
NCTensor *nc_get_col(NCTensor *w, NCTensor *x)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t dims[2];
    w = nc_contig(w); x = nc_contig(x);
    need_f32(w, "get_col");
    if (x->type != NC_TYPE_I32 || w->n_dims != 2)
        nc_fatal("get_col: (D,V) f32 matrix and i32 indices expected");
    dims[0] = w->dims[0]; dims[1] = nc_numel(x);
    y = new_out(w, 2, dims);
    const int32_t *ip = (const int32_t *)x->buf->data + x->off;
    for (size_t c = 0; c < dims[1]; c++) {
        if (ip[c] < 0 || (size_t)ip[c] >= w->dims[1])
            nc_fatal("get_col: index %d out of range", ip[c]);
        memcpy(nc_f32(y) + c * dims[0], nc_f32(w) + (size_t)ip[c] * dims[0], dims[0] * sizeof(float));
    }
    args[0] = w;
    n = nc_new_node(ctx_of(args, 1), OP_GET_COL, 1, args);
    n->saved[0] = nc_view(x);
    y = finish(y, n, args, 1);
    nc_free_tensor(w); nc_free_tensor(x);
    return y;
}

/* libnc.h:382: softmax over axis 0 (max-subtract, exp, sequential sum,
   divide: the order of src/neural/compatibility/cuda_math_compat.c:287-332) */
NCTensor *nc_soft_max(NCTensor *x)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t n0, cols;
    x = nc_contig(x);
    need_f32(x, "soft_max");
    n0 = x->dims[0];
    cols = nc_numel(x) / n0;
    y = nc_alloc_like(x);
    #pragma omp parallel for if (cols * n0 > 65536)
    for (size_t c = 0; c < cols; c++) {
        const float *xp = nc_f32(x) + c * n0;
        float *yp = nc_f32(y) + c * n0, mx = xp[0], s = 0;
        for (size_t i = 1; i < n0; i++)
            mx = xp[i] > mx ? xp[i] : mx;
        for (size_t i = 0; i < n0; i++) {
            yp[i] = expf(xp[i] - mx);
            s += yp[i];
        }
        float inv = 1.0f / s;
        for (size_t i = 0; i < n0; i++)
            yp[i] *= inv;
    }
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_SOFT_MAX, 1, args);
    if (x->node)
        n->saved[0] = nc_view(y);
    y = finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

/* libnc.h:385-388: y[n] = log x[eout[n], n].  When x comes straight out of
   nc_soft_max the gradient is sent to the logits as g*(onehot - p), the fused
   form the header announces; otherwise the plain g/x is scattered. */
NCTensor *nc_indexed_log(NCTensor *x, NCTensor *eout)
{
    NCTensor *y, *args[1];
    NCNode *n;
    size_t v, cols;
    x = nc_contig(x); eout = nc_contig(eout);
    need_f32(x, "indexed_log");
    if (eout->type != NC_TYPE_I32)
        nc_fatal("indexed_log: i32 indices expected");
    v = x->dims[0];
    cols = nc_numel(x) / v;
    if (nc_numel(eout) != cols)
        nc_fatal("indexed_log: %zu indices for %zu columns", nc_numel(eout), cols);
    y = nc_alloc(x->dev, NC_TYPE_F32, x->n_dims - 1, x->dims + 1, 0);
    const int32_t *ip = (const int32_t *)eout->buf->data + eout->off;
    for (size_t c = 0; c < cols; c++) {
        if (ip[c] < 0 || (size_t)ip[c] >= v)
            nc_fatal("indexed_log: index %d out of range", ip[c]);
        nc_f32(y)[c] = logf(nc_f32(x)[c * v + ip[c]]);
    }
    args[0] = x;
    n = nc_new_node(ctx_of(args, 1), OP_INDEXED_LOG, 1, args);
    if (x->node) {
        n->saved[0] = nc_view(x);
        n->saved[1] = nc_view(eout);
        if (x->node->op == OP_SOFT_MAX && x->node->parents[0]) {
            /* bypass the softmax node */
            nc_free_node(n->parents[0]);
            n->parents[0] = nc_dup_node(x->node->parents[0]);
            n->ia[0] = 1;
        }
    }
    y = finish(y, n, args, 1);
    nc_free_tensor(x); nc_free_tensor(eout);
    return y;
}

/* libnc.h:389-395.  (x-mean)/sqrt(var+eps) with the biased variance, or
   x/sqrt(mean(x^2)+eps) for rms; optional affine.  eps placement and biased
   variance follow the restatements in the reference tree
   (src/neural/acceleration/MetalComputeAccelerator.mm:233-252,
   src/neural/ops/nncp_lstm_metal_shaders.metal:117-131). */
static NCTensor *norm_op(NCTensor *x, NCTensor *w, NCTensor *b, float eps, int avg)
{
    NCTensor *y, *xhat, *rstd, *args[3];
    NCNode *n;
    size_t d, cols;
    x = nc_contig(x);
    need_f32(x, "layer_norm");
    d = x->dims[0];
    cols = nc_numel(x) / d;
    if (w) { w = nc_contig(w); b = nc_contig(b); }
    y = nc_alloc_like(x);
    xhat = w ? nc_alloc_like(x) : nc_dup_tensor(y);
    rstd = nc_alloc(x->dev, NC_TYPE_F32, 1, &cols, 0);
    #pragma omp parallel for if (cols * d > 65536)
    for (size_t c = 0; c < cols; c++) {
        const float *xp = nc_f32(x) + c * d;
        float mean = 0, var = 0, r;
        if (avg) {
            for (size_t i = 0; i < d; i++) mean += xp[i];
            mean /= (float)d;
        }
        for (size_t i = 0; i < d; i++) var += (xp[i] - mean) * (xp[i] - mean);
        var /= (float)d;
        r = 1.0f / sqrtf(var + eps);
        nc_f32(rstd)[c] = r;
        for (size_t i = 0; i < d; i++) {
            float h = (xp[i] - mean) * r;
            nc_f32(xhat)[c * d + i] = h;
            if (w)
                nc_f32(y)[c * d + i] = h * nc_f32(w)[i] + nc_f32(b)[i];
        }
    }
    args[0] = x; args[1] = w; args[2] = b;
    n = nc_new_node(ctx_of(args, 3), w ? OP_FUSED_LN : OP_LAYER_NORM, 3, args);
    if (nc_needs_grad(args, 3)) {
        n->saved[0] = nc_view(xhat);
        n->saved[1] = nc_view(rstd);
        if (w)
            n->saved[2] = nc_view(w);
    }
    n->ia[0] = avg;
    y = finish(y, n, args, 3);
    nc_free_tensor(xhat); nc_free_tensor(rstd);
    nc_free_tensor(x); nc_free_tensor(w); nc_free_tensor(b);
    return y;
}

NCTensor *nc_layer_norm(NCTensor *x, float eps) { return norm_op(x, NULL, NULL, eps, 1); }
NCTensor *nc_rms_norm(NCTensor *x, float eps) { return norm_op(x, NULL, NULL, eps, 0); }

NCTensor *nc_fused_layer_norm(NCTensor *x, NCTensor *w, NCTensor *b, float eps, BOOL avg_flag)
{
    if ((w == NULL) != (b == NULL))
        nc_fatal("fused_layer_norm: w and b must both be given or both be NULL");
    return norm_op(x, w, b, eps, avg_flag != 0);
}

static void norm_bw(NCNode *nd, NCTensor *g, NCTensor **ga)
{
    NCTensor *xhat = nd->saved[0], *rstd = nd->saved[1], *w = nd->saved[2];
    size_t d = xhat->dims[0], cols = nc_numel(xhat) / d;
    int avg = nd->ia[0];
    NCTensor *dx = nc_alloc_like(xhat);
    #pragma omp parallel for if (cols * d > 65536)
    for (size_t c = 0; c < cols; c++) {
        const float *gp = nc_f32(g) + c * d, *hp = nc_f32(xhat) + c * d;
        float s1 = 0, s2 = 0, r = nc_f32(rstd)[c];
        for (size_t i = 0; i < d; i++) {
            float gh = w ? gp[i] * nc_f32(w)[i] : gp[i];
            s1 += gh;
            s2 += gh * hp[i];
        }
        s1 = avg ? s1 / (float)d : 0.0f;
        s2 /= (float)d;
        for (size_t i = 0; i < d; i++) {
            float gh = w ? gp[i] * nc_f32(w)[i] : gp[i];
            nc_f32(dx)[c * d + i] = r * (gh - s1 - hp[i] * s2);
        }
    }
    if (nd->parents[0]) ga[0] = dx; else nc_free_tensor(dx);
    if (w) {
        NCTensor *dw = nc_alloc(g->dev, NC_TYPE_F32, 1, &d, 1);
        NCTensor *db = nc_alloc(g->dev, NC_TYPE_F32, 1, &d, 1);
        for (size_t c = 0; c < cols; c++)
            for (size_t i = 0; i < d; i++) {
                nc_f32(dw)[i] += nc_f32(g)[c * d + i] * nc_f32(xhat)[c * d + i];
                nc_f32(db)[i] += nc_f32(g)[c * d + i];
            }
        if (nd->parents[1]) ga[1] = dw; else nc_free_tensor(dw);
        if (nd->parents[2]) ga[2] = db; else nc_free_tensor(db);
    }
}

/* ------------------------------------------------------------------------ */
/* backward                                                                 */

static NCTensor *reshape_to(NCTensor *g, int nd, const size_t *dims)
{
    NCTensor *y;
    size_t s = 1;
    g = nc_contig(g);
    y = nc_view(g);
    y->n_dims = nd;
    for (int i = 0; i < nd; i++) { y->dims[i] = dims[i]; y->strides[i] = s; s *= dims[i]; }
    nc_free_tensor(g);
    return y;
}

/* computes the gradients ga[i] of the arguments whose parent is set */
static void node_backward(NCNode *nd, NCTensor *g, NCTensor **ga)
{
    size_t cnt = nc_numel(g);
    switch (nd->op) {
    case OP_ADD:
        if (nd->parents[0]) ga[0] = unbroadcast(nc_dup_tensor(g), nd->arg_ndims[0], nd->arg_dims[0]);
        if (nd->parents[1]) ga[1] = unbroadcast(nc_dup_tensor(g), nd->arg_ndims[1], nd->arg_dims[1]);
        break;
    case OP_MUL: {
        BCast bc;
        bcast_plan(&bc, nd->arg_ndims[0], nd->arg_dims[0], nd->arg_ndims[1], nd->arg_dims[1], "mul_bw");
        for (int w = 0; w < 2; w++) {
            if (!nd->parents[w]) continue;
            NCTensor *t = nc_alloc_like(g);
            const float *gp = nc_f32(g), *op = nc_f32(nd->saved[1 - w]);
            float *tp = nc_f32(t);
            size_t n0_ = nc_numel(nd->saved[0]), n1_ = nc_numel(nd->saved[1]);
            if (n0_ == bc.n && bcast_prefix(&bc, nd->arg_ndims[1], nd->arg_dims[1])) {
                if (w == 0) for (size_t i = 0; i < bc.n; i++) tp[i] = gp[i] * op[i % n1_];
                else        for (size_t i = 0; i < bc.n; i++) tp[i] = gp[i] * op[i];
            } else if (w == 0) BCAST_LOOP(&bc, ia, ib, io, tp[io] = gp[io] * op[ib]);
            else        BCAST_LOOP(&bc, ia, ib, io, tp[io] = gp[io] * op[ia]);
            ga[w] = unbroadcast(t, nd->arg_ndims[w], nd->arg_dims[w]);
        }
        break;
    }
    case OP_MASKED_FILL: {
        BCast bc;
        NCTensor *mask = nd->saved[0], *t = nc_alloc_like(g);
        const int8_t *mp = (const int8_t *)mask->buf->data + mask->off;
        bcast_plan(&bc, g->n_dims, g->dims, mask->n_dims, mask->dims, "masked_fill_bw");
        BCAST_LOOP(&bc, ia, ib, io,
                   nc_f32(t)[io] = ((mp[ib] != 0) != (nd->ia[0] != 0)) ? 0.0f : nc_f32(g)[io]);
        ga[0] = t;
        break;
    }
    case OP_SIGMOID: case OP_TANH: case OP_RELU: case OP_GELU: {
        NCTensor *t = nc_alloc_like(g);
        const float *xp = nc_f32(nd->saved[0]);
        #pragma omp parallel for if (cnt > 65536)
        for (size_t i = 0; i < cnt; i++) {
            float x = xp[i], d;
            switch (nd->op) {
            case OP_SIGMOID: { float s = sigmoidf_(x); d = s * (1 - s); break; }
            case OP_TANH: { float th = tanhf(x); d = 1 - th * th; break; }
            case OP_RELU: d = x > 0 ? 1.0f : 0.0f; break;
            default: d = gelu_grad_f(x); break;
            }
            nc_f32(t)[i] = nc_f32(g)[i] * d;
        }
        ga[0] = t;
        break;
    }
    case OP_GATED_SWISH: {
        const float *gp = nc_f32(nd->saved[0]), *xp = nc_f32(nd->saved[1]);
        float beta = nd->fa[0];
        NCTensor *dg = nc_alloc_like(g), *dx = nc_alloc_like(g);
        for (size_t i = 0; i < cnt; i++) {
            float s = sigmoidf_(beta * xp[i]);
            nc_f32(dg)[i] = nc_f32(g)[i] * xp[i] * s;
            nc_f32(dx)[i] = nc_f32(g)[i] * gp[i] * (s + beta * xp[i] * s * (1 - s));
        }
        if (nd->parents[0]) ga[0] = dg; else nc_free_tensor(dg);
        if (nd->parents[1]) ga[1] = dx; else nc_free_tensor(dx);
        break;
    }
    case OP_LSTM_CLAMPED: {
        const float *cp = nc_f32(nd->saved[0]), *in = nc_f32(nd->saved[1]);
        const float *fg = nc_f32(nd->saved[2]), *ig = nc_f32(nd->saved[3]);
        NCTensor *t[4];
        for (int a = 0; a < 4; a++) t[a] = nc_alloc_like(g);
        for (size_t i = 0; i < cnt; i++) {
            float gi = nc_f32(g)[i];
            int clamped = (1.0f - fg[i]) < ig[i];
            nc_f32(t[0])[i] = gi * fg[i];
            nc_f32(t[1])[i] = gi * fminf(1.0f - fg[i], ig[i]);
            nc_f32(t[2])[i] = gi * cp[i] - (clamped ? gi * in[i] : 0.0f);
            nc_f32(t[3])[i] = clamped ? 0.0f : gi * in[i];
        }
        for (int a = 0; a < 4; a++)
            if (nd->parents[a]) ga[a] = t[a]; else nc_free_tensor(t[a]);
        break;
    }
    case OP_LERP: {
        const float *a = nc_f32(nd->saved[0]), *b = nc_f32(nd->saved[1]), *t = nc_f32(nd->saved[2]);
        NCTensor *r[3];
        for (int q = 0; q < 3; q++) r[q] = nc_alloc_like(g);
        for (size_t i = 0; i < cnt; i++) {
            float gi = nc_f32(g)[i];
            nc_f32(r[0])[i] = gi * (1.0f - t[i]);
            nc_f32(r[1])[i] = gi * t[i];
            nc_f32(r[2])[i] = gi * (b[i] - a[i]);
        }
        for (int q = 0; q < 3; q++)
            if (nd->parents[q]) ga[q] = r[q]; else nc_free_tensor(r[q]);
        break;
    }
    case OP_CONVERT:
        ga[0] = nc_dup_tensor(g);
        break;
    case OP_RESHAPE:
        ga[0] = reshape_to(nc_dup_tensor(g), nd->arg_ndims[0], nd->arg_dims[0]);
        break;
    case OP_REPEAT:
        ga[0] = nc_reduce_sum(NULL, nc_dup_tensor(g), nd->arg_ndims[0]);
        break;
    case OP_REDUCE_SUM:
        if (nd->parents[0]) ga[0] = nc_dup_tensor(g);
        if (nd->parents[1])
            ga[1] = repeat_nd(nc_dup_tensor(g), nd->arg_ndims[1] - g->n_dims,
                              nd->arg_dims[1] + g->n_dims);
        break;
    case OP_SUM: {
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, nd->arg_ndims[0], nd->arg_dims[0], 0);
        size_t c2 = nc_numel(t);
        for (size_t i = 0; i < c2; i++)
            nc_f32(t)[i] = nc_f32(g)[0];
        ga[0] = t;
        break;
    }
    case OP_SLICE: {
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, nd->arg_ndims[0], nd->arg_dims[0], 1);
        NCTensor *v = nc_slice_alias(t, nd->ia[0], nd->ia[1], nd->ia[1] + g->dims[nd->ia[0]]);
        nc_copy_strided(v, g);
        nc_free_tensor(v);
        ga[0] = t;
        break;
    }
    case OP_CONCAT: case OP_CONCAT_NODE: {
        size_t pos = 0;
        for (int i = 0; i < nd->n_args; i++) {
            if (nd->parents[i]) {
                NCTensor *v = nc_slice_alias(g, nd->ia[0], pos, pos + nd->sizes[i]);
                ga[i] = nc_alloc(g->dev, NC_TYPE_F32, v->n_dims, v->dims, 0);
                nc_copy_strided(ga[i], v);
                nc_free_tensor(v);
            }
            pos += nd->sizes[i];
        }
        break;
    }
    case OP_PAD: {
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, nd->arg_ndims[0], nd->arg_dims[0], 1);
        size_t n_in = nd->arg_dims[0][0], cols = nc_numel(t) / n_in;
        for (size_t c = 0; c < cols; c++)
            pad_map(n_in, nd->ia[0], nd->ia[1], nd->ia[2], nd->ia[3],
                    nc_f32(t) + c * n_in, nc_f32(g) + c * g->dims[0], 1);
        ga[0] = t;
        break;
    }
    case OP_PERMUTE: {
        int inv[NC_N_DIMS_MAX];
        for (int i = 0; i < g->n_dims; i++)
            inv[nd->ia[i]] = i;
        ga[0] = permute_raw(g, g->n_dims, inv);
        break;
    }
    case OP_REL_SHIFT: {
        NCTensor *t = nc_alloc_like(g);
        rel_shift_raw(nc_f32(g), nc_f32(t), g->dims[0], g->dims[1],
                      cnt / (g->dims[0] * g->dims[1]), nd->ia[0], nd->ia[1], 1);
        ga[0] = t;
        break;
    }
    case OP_MATMUL:
        matmul_bw(nd, g, ga);
        break;
    case OP_GET_COL: {
        NCTensor *idx = nd->saved[0];
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, nd->arg_ndims[0], nd->arg_dims[0], 1);
        const int32_t *ip = (const int32_t *)idx->buf->data + idx->off;
        size_t d = g->dims[0], cols = cnt / d;
        for (size_t c = 0; c < cols; c++)
            for (size_t i = 0; i < d; i++)
                nc_f32(t)[(size_t)ip[c] * d + i] += nc_f32(g)[c * d + i];
        ga[0] = t;
        break;
    }
    case OP_SOFT_MAX: {
        NCTensor *y = nd->saved[0], *t = nc_alloc_like(g);
        size_t n0 = y->dims[0], cols = cnt / n0;
        for (size_t c = 0; c < cols; c++) {
            const float *yp = nc_f32(y) + c * n0, *gp = nc_f32(g) + c * n0;
            float s = 0;
            for (size_t i = 0; i < n0; i++) s += gp[i] * yp[i];
            for (size_t i = 0; i < n0; i++) nc_f32(t)[c * n0 + i] = yp[i] * (gp[i] - s);
        }
        ga[0] = t;
        break;
    }
    case OP_INDEXED_LOG: {
        NCTensor *p = nd->saved[0], *idx = nd->saved[1];
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, p->n_dims, p->dims, 1);
        const int32_t *ip = (const int32_t *)idx->buf->data + idx->off;
        size_t v = p->dims[0], cols = nc_numel(p) / v;
        for (size_t c = 0; c < cols; c++) {
            float gc = nc_f32(g)[c];
            if (nd->ia[0]) {
                for (size_t i = 0; i < v; i++)
                    nc_f32(t)[c * v + i] = -gc * nc_f32(p)[c * v + i];
                nc_f32(t)[c * v + ip[c]] += gc;
            } else {
                nc_f32(t)[c * v + ip[c]] = gc / nc_f32(p)[c * v + ip[c]];
            }
        }
        ga[0] = t;
        break;
    }
    case OP_LAYER_NORM: case OP_FUSED_LN:
        norm_bw(nd, g, ga);
        break;
    case OP_RELPOS_ATTN:
        nc_relpos_attention_bw(nd, g, ga);
        break;
    default:
        nc_fatal("backward: op %d not handled", nd->op);
    }
}

static void count_edges(NCNode *n, int epoch)
{
    /* iterative DFS */
    NCNode **stack = nc_malloc(sizeof(NCNode *) * 64);
    int sp = 0, cap = 64;
    n->mark = epoch;
    n->pending = 0;
    stack[sp++] = n;
    while (sp > 0) {
        NCNode *c = stack[--sp];
        for (int i = 0; i < c->n_args; i++) {
            NCNode *p = c->parents[i];
            if (!p)
                continue;
            if (p->mark != epoch) {
                p->mark = epoch;
                p->pending = 0;
                if (sp == cap) { cap *= 2; stack = realloc(stack, sizeof(NCNode *) * cap); }
                stack[sp++] = p;
            }
            p->pending++;
        }
    }
    free(stack);
}

static void accumulate(NCNode *p, NCTensor *g)
{
    if (!p->grad) {
        p->grad = nc_contig(g);
        return;
    }
    g = nc_contig(g);
    size_t cnt = nc_numel(g);
    if (cnt != nc_numel(p->grad))
        nc_fatal("backward: gradient shape mismatch at op %d (%zu vs %zu)", p->op, cnt, nc_numel(p->grad));
    if (p->grad->ref > 1 || p->grad->buf->ref > 1) {
        /* shared storage: copy before accumulating in place */
        NCTensor *t = nc_alloc_like(p->grad);
        memcpy(nc_f32(t), nc_f32(p->grad), cnt * sizeof(float));
        nc_free_tensor(p->grad);
        p->grad = t;
    }
    for (size_t i = 0; i < cnt; i++)
        nc_f32(p->grad)[i] += nc_f32(g)[i];
    nc_free_tensor(g);
}

/* libnc.h:480-481: x borrowed, grad consumed; one callback per parameter
   leaf with the summed gradient (tied tensors used in several layers arrive
   once, already summed, because the leaf node is shared). */
void nc_backward(const NCTensor *x, NCTensor *grad, NCParamUpdateFunc *cb, int flags)
{
    static int epoch;
    NCNode **ready;
    int sp = 0, cap = 256;
    (void)flags;
    if (!x->node) {
        nc_free_tensor(grad);
        return;
    }
    epoch++;
    count_edges(x->node, epoch);
    ready = nc_malloc(sizeof(NCNode *) * cap);
    x->node->grad = grad;
    ready[sp++] = x->node;
    while (sp > 0) {
        NCNode *nd = ready[--sp];
        NCTensor *g = nd->grad;
        nd->grad = NULL;
        if (nd->op == OP_PARAM) {
            if (cb)
                cb(nd->opaque, g, NULL);
            else
                nc_free_tensor(g);
            continue;
        }
        NCTensor **ga = nc_mallocz(sizeof(NCTensor *) * (nd->n_args ? nd->n_args : 1));
        if (g)
            node_backward(nd, g, ga);
        for (int i = 0; i < nd->n_args; i++) {
            NCNode *p = nd->parents[i];
            if (!p) {
                nc_free_tensor(ga[i]);
                continue;
            }
            if (ga[i])
                accumulate(p, ga[i]);
            if (--p->pending == 0) {
                if (sp == cap) { cap *= 2; ready = realloc(ready, sizeof(NCNode *) * cap); }
                ready[sp++] = p;
            }
        }
        nc_free_tensor(g);
        free(ga);
    }
    free(ready);
}
