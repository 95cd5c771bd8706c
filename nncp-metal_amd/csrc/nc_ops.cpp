// libnc_hip ops: shape logic, graph recording and the per-op backward, all
// dispatching to the gfx950 kernels (k_*.hip).  The op list is the one
// trf_eval / trf_eval_gradient issue (nncp.c:581-1193) plus the fused entry
// points of nc_ext.h.  Device tensors only: a host tensor reaching a compute op
// aborts (see need_dev).
#include <math.h>
#include "nc_hip_internal.h"
#include <algorithm>

#define LAUNCHED(x) (nc_ctx(x)->launches++)
// every op takes its operands through nc_operand: contiguous, bf16 tensors as their f32 copies
#define nc_contig(x) nc_operand(x)

static NCTensor *new_f32(const NCTensor *like, int nd, const size_t *dims)
{
    return nc_alloc(like->dev, NC_TYPE_F32, nd, dims, false);
}

static void need_f32(const NCTensor *x, const char *op)
{
    need_dev(x, op);
    if (x->type != NC_TYPE_F32) nc_fatal("%s: f32 tensor expected (type %d)", op, (int)x->type);
}

static void same_numel(const NCTensor *a, const NCTensor *b, const char *op)
{
    if (nc_numel(a) != nc_numel(b)) nc_fatal("%s: operands must have the same shape", op);
}

// ---- broadcasting -----------------------------------------------------------
struct BPlan {
    int nd;
    size_t dims[NC_N_DIMS_MAX], n;
    NdDesc desc;
};

static void bplan(BPlan *bp, int na, const size_t *da, int nb, const size_t *db, const char *op)
{
    size_t sa = 1, sb = 1;
    bp->nd = na > nb ? na : nb;
    bp->n = 1;
    bp->desc.nd = bp->nd;
    for (int i = 0; i < bp->nd; i++) {
        size_t a = i < na ? da[i] : 1, b = i < nb ? db[i] : 1;
        if (a != b && a != 1 && b != 1)
            nc_fatal("%s: incompatible shapes on axis %d (%zu vs %zu)", op, i, a, b);
        bp->dims[i] = a > b ? a : b;
        bp->desc.dims[i] = (int64_t)bp->dims[i];
        bp->desc.sa[i] = a == 1 ? 0 : (int64_t)sa;
        bp->desc.sb[i] = b == 1 ? 0 : (int64_t)sb;
        sa *= a; sb *= b;
        bp->n *= bp->dims[i];
    }
    if (bp->nd == 0) { bp->desc.nd = 1; bp->desc.dims[0] = 1; bp->desc.sa[0] = bp->desc.sb[0] = 0; }
}

// b's dims equal the leading dims of the result (trailing 1s allowed)
static bool is_prefix(const BPlan *bp, int nb, const size_t *db)
{
    for (int i = 0; i < nb; i++)
        if (db[i] != bp->dims[i]) {
            for (int j = i; j < nb; j++)
                if (db[j] != 1) return false;
            break;
        }
    return true;
}

// a op b with broadcasting; operands borrowed and contiguous
static NCTensor *dev_binary(int op, const NCTensor *a, const NCTensor *b)
{
    BPlan bp;
    bplan(&bp, a->n_dims, a->dims, b->n_dims, b->dims, op == KB_ADD ? "add" : "mul");
    NCTensor *y = new_f32(a, bp.nd, bp.dims);
    if (bp.n == 0) return y;
    if (nc_numel(a) == bp.n && is_prefix(&bp, b->n_dims, b->dims))
        k_binary_prefix(nc_stream(a), op, nc_f32(a), nc_f32(b), nc_f32(y), (int64_t)bp.n, (int64_t)nc_numel(b));
    else if (nc_numel(b) == bp.n && is_prefix(&bp, a->n_dims, a->dims))
        k_binary_prefix(nc_stream(a), op, nc_f32(b), nc_f32(a), nc_f32(y), (int64_t)bp.n, (int64_t)nc_numel(a));
    else
        k_binary_nd(nc_stream(a), op, nc_f32(a), nc_f32(b), nc_f32(y), &bp.desc, (int64_t)bp.n);
    LAUNCHED(a);
    return y;
}

// sums g (consumed) down to `target` (each target dim equals g's or is 1/missing)
static void defer_sum(NCContext *m, const float *src, NCTensor *dst, int rows, int64_t stride, int n,
                      const NCNode *param);
bool nc_can_defer_shared_sum(const NCContext *m, const NCNode *parent);
static NCTensor *defer_shared_sum(NCContext *m, const float *src, NCTensor *like, int rows, int64_t stride,
                                  const NCNode *param);

// defer_param: the parameter node the result is the gradient of, when its
// final sum over partial rows may wait for the end of nc_backward
static NCTensor *dev_unbroadcast(NCTensor *g, const Shape &target, const NCNode *defer_param = nullptr)
{
    size_t nt = 1;
    for (int i = 0; i < target.nd; i++) nt *= target.d[i];
    if (nt == nc_numel(g)) return nc_reshape_view(g, target.nd, target.d);
    NCContext *m = nc_ctx(g);
    g = nc_contig(g);
    NCTensor *y = nc_alloc(g->dev, NC_TYPE_F32, target.nd, target.d, false);
    // trailing reduction: target dims are a prefix of g's
    bool prefix = true;
    for (int i = 0; i < target.nd && prefix; i++)
        if (target.d[i] != g->dims[i]) {
            for (int j = i; j < target.nd; j++)
                if (target.d[j] != 1) prefix = false;
            break;
        }
    size_t cap;
    if (nt == 1) {
        float *tmp = nc_tmp_f32(m, 1024, &cap);
        k_reduce_all(m->stream, nc_f32(g), nc_f32(y), tmp, (int64_t)nc_numel(g));
        nc_tmp_free(m, tmp, cap);
    } else if (prefix) {
        int64_t inner = (int64_t)nt, outer = (int64_t)(nc_numel(g) / nt);
        float *tmp = nc_tmp_f32(m, (size_t)k_reduce_trailing_nsplit(inner, outer) * inner, &cap);
        if (defer_param && nc_can_defer_sum(m, defer_param) && inner < (1 << 30)) {
            int ns = k_reduce_trailing_partials(m->stream, nc_f32(g), tmp, inner, outer);
            defer_sum(m, tmp, y, ns, inner, (int)inner, defer_param);
            DeferredTmp dt = { tmp, cap };
            m->deferred_tmp.push_back(dt);
        } else {
            k_reduce_trailing(m->stream, nc_f32(g), nullptr, nc_f32(y), tmp, inner, outer);
            nc_tmp_free(m, tmp, cap);
            m->launches++; // second stage
        }
    } else {
        // general case: one thread per kept element loops over the reduced axes
        NdDesc keep, red;
        keep.nd = red.nd = 0;
        int64_t stride = 1, nred = 1;
        for (int i = 0; i < g->n_dims; i++) {
            size_t td = i < target.nd ? target.d[i] : 1;
            if (td == g->dims[i]) {
                keep.dims[keep.nd] = (int64_t)g->dims[i]; keep.sa[keep.nd] = stride; keep.sb[keep.nd] = 0; keep.nd++;
            } else {
                red.dims[red.nd] = (int64_t)g->dims[i]; red.sa[red.nd] = stride; red.sb[red.nd] = 0; red.nd++;
                nred *= (int64_t)g->dims[i];
            }
            stride *= (int64_t)g->dims[i];
        }
        if (keep.nd == 0) { keep.nd = 1; keep.dims[0] = 1; keep.sa[0] = keep.sb[0] = 0; }
        if (red.nd == 0) { red.nd = 1; red.dims[0] = 1; red.sa[0] = red.sb[0] = 0; }
        k_unbroadcast_nd(m->stream, nc_f32(g), nc_f32(y), &keep, &red, (int64_t)nt, nred);
    }
    m->launches++;
    nc_free_tensor(g);
    return y;
}

static NCTensor *binary_op(NCTensor *a, NCTensor *b, int kop, int op)
{
    a = nc_contig(a); b = nc_contig(b);
    need_f32(a, "binary op"); need_f32(b, "binary op");
    NCTensor *y = dev_binary(kop, a, b);
    NCTensor *args[2] = { a, b };
    NCNode *n = nc_new_node(nc_ctx(a), op, 2, args);
    if (op == OP_MUL && (a->node || b->node)) {
        n->saved[0] = nc_view(a);
        n->saved[1] = nc_view(b);
    }
    y = nc_finish(y, n, args, 2);
    nc_free_tensor(a); nc_free_tensor(b);
    return y;
}

extern "C" NCTensor *nc_add(NCTensor *x1, NCTensor *x2) { return binary_op(x1, x2, KB_ADD, OP_ADD); } // libnc.h:232
extern "C" NCTensor *nc_mul(NCTensor *x1, NCTensor *x2) { return binary_op(x1, x2, KB_MUL, OP_MUL); } // libnc.h:235

// libnc.h:231.  BF16 -> F32 is what every op does to a bf16 operand anyway (nc_operand: the
// buffer's f32 copy, same node); F32 -> BF16 is one rounding pass into a new 2-byte tensor
// that keeps the node too (the gradient of a conversion is the identity, in f32).
extern "C" NCTensor *nc_convert(NCTensor *x, NCTypeEnum new_type)
{
    if (x->type == new_type) return x;
    if (x->type == NC_TYPE_BF16 && new_type == NC_TYPE_F32) return nc_operand(x);
    if (x->type == NC_TYPE_F32 && new_type == NC_TYPE_BF16) {
        x = nc_contig(x);
        need_dev(x, "nc_convert");
        if (((uintptr_t)nc_data(x) & 15) != 0) { // a view at an odd offset: the cast reads 16-byte units
            NCTensor *c = nc_alloc_like(x);
            nc_copy_any(c, x);
            c->node = nc_dup_node(x->node);
            nc_free_tensor(x);
            x = c;
        }
        NCTensor *y = nc_alloc(x->dev, NC_TYPE_BF16, x->n_dims, x->dims, false);
        if (nc_numel(x)) {
            if (nchip_cast_bf16(nc_stream(x), nc_f32(x), (uint16_t *)nc_data(y), (int64_t)nc_numel(x)))
                nc_fatal("nc_convert: bf16 cast failed");
            LAUNCHED(x);
        }
        y->node = nc_dup_node(x->node);
        nc_free_tensor(x);
        return y;
    }
    nc_fatal("nc_convert %d -> %d: f32 and bf16 are the item types that carry values here", (int)x->type, (int)new_type);
}

extern "C" NCTensor *nc_masked_fill(NCTensor *x, NCTensor *mask, float c, BOOL mask_inv)
{
    x = nc_contig(x); mask = nc_contig(mask);
    need_f32(x, "nc_masked_fill"); need_dev(mask, "nc_masked_fill");
    if (mask->type != NC_TYPE_I8) nc_fatal("nc_masked_fill: i8 mask expected");
    BPlan bp;
    bplan(&bp, x->n_dims, x->dims, mask->n_dims, mask->dims, "masked_fill");
    if (bp.n != nc_numel(x) || !is_prefix(&bp, mask->n_dims, mask->dims))
        nc_fatal("nc_masked_fill: the mask must match the leading axes of x");
    NCTensor *y = nc_alloc_like(x);
    k_masked_fill(nc_stream(x), nc_f32(x), (const int8_t *)nc_data(mask), nc_f32(y),
                  (int64_t)bp.n, (int64_t)nc_numel(mask), c, mask_inv != 0);
    LAUNCHED(x);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_MASKED_FILL, 1, args);
    n->saved[0] = nc_view(mask);
    n->ia[0] = mask_inv != 0;
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x); nc_free_tensor(mask);
    return y;
}

static NCTensor *unary_op(NCTensor *x, int kop)
{
    x = nc_contig(x);
    need_f32(x, "activation");
    NCTensor *y = nc_alloc_like(x);
    k_unary_fwd(nc_stream(x), kop, nc_f32(x), nc_f32(y), (int64_t)nc_numel(x));
    LAUNCHED(x);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_UNARY, 1, args);
    n->ia[0] = kop;
    if (x->node) n->saved[0] = nc_view(x);
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_sigmoid(NCTensor *x) { return unary_op(x, KU_SIGMOID); } // libnc.h:245
extern "C" NCTensor *nc_tanh(NCTensor *x) { return unary_op(x, KU_TANH); }       // libnc.h:246
extern "C" NCTensor *nc_relu(NCTensor *x) { return unary_op(x, KU_RELU); }       // libnc.h:247
extern "C" NCTensor *nc_gelu(NCTensor *x) { return unary_op(x, KU_GELU); }       // libnc.h:252 (tanh form)

extern "C" NCTensor *nc_gated_swish(NCTensor *g, NCTensor *x, float beta) // libnc.h:249-251
{
    g = nc_contig(g); x = nc_contig(x);
    need_f32(g, "nc_gated_swish"); need_f32(x, "nc_gated_swish");
    same_numel(g, x, "nc_gated_swish");
    NCTensor *y = nc_alloc_like(x);
    k_gated_swish_fwd(nc_stream(x), nc_f32(g), nc_f32(x), nc_f32(y), (int64_t)nc_numel(x), beta);
    LAUNCHED(x);
    NCTensor *args[2] = { g, x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_GATED_SWISH, 2, args);
    n->saved[0] = nc_view(g); n->saved[1] = nc_view(x);
    n->fa[0] = beta;
    y = nc_finish(y, n, args, 2);
    nc_free_tensor(g); nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_lstm_clamped(NCTensor *cp, NCTensor *in, NCTensor *fg, NCTensor *ig) // libnc.h:261-263
{
    NCTensor *args[4] = { nc_contig(cp), nc_contig(in), nc_contig(fg), nc_contig(ig) };
    for (int i = 0; i < 4; i++) { need_f32(args[i], "nc_lstm_clamped"); same_numel(args[0], args[i], "nc_lstm_clamped"); }
    NCTensor *y = nc_alloc_like(args[0]);
    k_lstm_clamped_fwd(nc_stream(y), nc_f32(args[0]), nc_f32(args[1]), nc_f32(args[2]), nc_f32(args[3]),
                       nc_f32(y), (int64_t)nc_numel(y));
    LAUNCHED(y);
    NCNode *n = nc_new_node(nc_ctx(y), OP_LSTM_CLAMPED, 4, args);
    for (int i = 0; i < 4; i++) n->saved[i] = nc_view(args[i]);
    y = nc_finish(y, n, args, 4);
    for (int i = 0; i < 4; i++) nc_free_tensor(args[i]);
    return y;
}

extern "C" NCTensor *nc_lerp(NCTensor *a, NCTensor *b, NCTensor *t) // libnc.h:272-273
{
    NCTensor *args[3] = { nc_contig(a), nc_contig(b), nc_contig(t) };
    for (int i = 0; i < 3; i++) { need_f32(args[i], "nc_lerp"); same_numel(args[0], args[i], "nc_lerp"); }
    NCTensor *y = nc_alloc_like(args[0]);
    k_lerp_fwd(nc_stream(y), nc_f32(args[0]), nc_f32(args[1]), nc_f32(args[2]), nc_f32(y), (int64_t)nc_numel(y));
    LAUNCHED(y);
    NCNode *n = nc_new_node(nc_ctx(y), OP_LERP, 3, args);
    for (int i = 0; i < 3; i++) n->saved[i] = nc_view(args[i]);
    y = nc_finish(y, n, args, 3);
    for (int i = 0; i < 3; i++) nc_free_tensor(args[i]);
    return y;
}

// ---- shape ops --------------------------------------------------------------
static NCTensor *reshape_nd(NCTensor *x, int nd, const size_t *dims)
{
    x = nc_contig(x);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_RESHAPE, 1, args);
    NCTensor *y = nc_reshape_view(nc_dup_tensor(x), nd, dims);
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_reshape_1d(NCTensor *x, size_t n0) { size_t d[1] = { n0 }; return reshape_nd(x, 1, d); }
extern "C" NCTensor *nc_reshape_2d(NCTensor *x, size_t n0, size_t n1) { size_t d[2] = { n0, n1 }; return reshape_nd(x, 2, d); }
extern "C" NCTensor *nc_reshape_3d(NCTensor *x, size_t n0, size_t n1, size_t n2) { size_t d[3] = { n0, n1, n2 }; return reshape_nd(x, 3, d); }
extern "C" NCTensor *nc_reshape_4d(NCTensor *x, size_t n0, size_t n1, size_t n2, size_t n3) { size_t d[4] = { n0, n1, n2, n3 }; return reshape_nd(x, 4, d); }

// libnc.h:289-292: duplicate along new trailing axes (stride-0 source copy)
static NCTensor *repeat_raw(const NCTensor *x, int nr, const size_t *rd)
{
    size_t dims[NC_N_DIMS_MAX];
    if (x->n_dims + nr > NC_N_DIMS_MAX) nc_fatal("repeat: too many axes");
    memcpy(dims, x->dims, sizeof(size_t) * x->n_dims);
    for (int i = 0; i < nr; i++) dims[x->n_dims + i] = rd[i];
    NCTensor *y = nc_alloc(x->dev, x->type, x->n_dims + nr, dims, false);
    NCTensor *v = nc_view(x);
    v->n_dims = x->n_dims + nr;
    for (int i = 0; i < nr; i++) { v->dims[x->n_dims + i] = rd[i]; v->strides[x->n_dims + i] = 0; }
    nc_copy_any(y, v);
    nc_free_tensor(v);
    return y;
}

static NCTensor *repeat_nd(NCTensor *x, int nr, const size_t *rd)
{
    x = nc_contig(x);
    need_dev(x, "nc_repeat");
    NCTensor *y = repeat_raw(x, nr, rd);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_REPEAT, 1, args);
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_repeat_1d(NCTensor *x, size_t n0) { size_t d[1] = { n0 }; return repeat_nd(x, 1, d); }
extern "C" NCTensor *nc_repeat_2d(NCTensor *x, size_t n0, size_t n1) { size_t d[2] = { n0, n1 }; return repeat_nd(x, 2, d); }

// libnc.h:293-295: y0 + sum over the axes >= n_dims
extern "C" NCTensor *nc_reduce_sum(NCTensor *y0, NCTensor *x, int n_dims)
{
    x = nc_contig(x);
    need_f32(x, "nc_reduce_sum");
    if (y0) { y0 = nc_contig(y0); need_f32(y0, "nc_reduce_sum"); }
    NCContext *m = nc_ctx(x);
    int64_t inner = 1;
    for (int i = 0; i < n_dims; i++) inner *= (int64_t)x->dims[i];
    int64_t outer = (int64_t)nc_numel(x) / inner;
    if (y0 && (int64_t)nc_numel(y0) != inner) nc_fatal("nc_reduce_sum: y0 shape mismatch");
    NCTensor *y = new_f32(x, n_dims, x->dims);
    size_t cap;
    float *tmp = nc_tmp_f32(m, (size_t)k_reduce_trailing_nsplit(inner, outer) * inner, &cap);
    k_reduce_trailing(m->stream, nc_f32(x), y0 ? nc_f32(y0) : nullptr, nc_f32(y), tmp, inner, outer);
    nc_tmp_free(m, tmp, cap);
    m->launches += 2;
    NCTensor *args[2] = { y0, x };
    NCNode *n = nc_new_node(m, OP_REDUCE_SUM, 2, args);
    y = nc_finish(y, n, args, 2);
    nc_free_tensor(y0); nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_sum(NCTensor *x) // libnc.h:298-299
{
    x = nc_contig(x);
    need_f32(x, "nc_sum");
    NCContext *m = nc_ctx(x);
    NCTensor *y = nc_alloc(x->dev, NC_TYPE_F32, 0, nullptr, false);
    size_t cap;
    float *tmp = nc_tmp_f32(m, 1024, &cap);
    k_reduce_all(m->stream, nc_f32(x), nc_f32(y), tmp, (int64_t)nc_numel(x));
    nc_tmp_free(m, tmp, cap);
    m->launches += 2;
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(m, OP_SUM, 1, args);
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

// libnc.h:306-307: alias sharing storage, no graph; writing through it with
// nc_tensor_copy mutates the parent (nncp.c:650-657, 697-702)
extern "C" NCTensor *nc_slice_alias(const NCTensor *x, int axis, size_t start, size_t end)
{
    if (axis < 0 || axis >= x->n_dims || end > x->dims[axis] || start > end)
        nc_fatal("nc_slice_alias: range [%zu,%zu) outside axis %d", start, end, axis);
    NCTensor *y = nc_view(x);
    y->off += start * x->strides[axis];
    y->dims[axis] = end - start;
    return y;
}

extern "C" NCTensor *nc_slice(NCTensor *x, int axis, size_t start, size_t end) // libnc.h:308
{
    NCTensor *v = nc_slice_alias(x, axis, start, end);
    NCTensor *y = nc_alloc(x->dev, x->type, v->n_dims, v->dims, false);
    nc_copy_any(y, v);
    nc_free_tensor(v);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_SLICE, 1, args);
    n->ia[0] = axis; n->ia[1] = (int)start;
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_concat(NCTensor **inputs, int n_inputs, int axis) // libnc.h:310-311
{
    int nd = inputs[0]->n_dims;
    size_t dims[NC_N_DIMS_MAX], total = 0, pos = 0;
    if (axis < 0 || axis >= nd) nc_fatal("nc_concat: axis %d out of range", axis);
    memcpy(dims, inputs[0]->dims, sizeof(size_t) * nd);
    for (int i = 0; i < n_inputs; i++) {
        if (inputs[i]->n_dims != nd) nc_fatal("nc_concat: rank mismatch");
        for (int a = 0; a < nd; a++)
            if (a != axis && inputs[i]->dims[a] != dims[a]) nc_fatal("nc_concat: shape mismatch on axis %d", a);
        total += inputs[i]->dims[axis];
    }
    dims[axis] = total;
    NCTensor *y = nc_alloc(inputs[0]->dev, inputs[0]->type, nd, dims, false);
    NCNode *n = nc_new_node(nc_ctx(y), OP_CONCAT, n_inputs, nullptr);
    n->ia[0] = axis;
    for (int i = 0; i < n_inputs; i++) {
        NCTensor *v = nc_slice_alias(y, axis, pos, pos + inputs[i]->dims[axis]);
        nc_copy_any(v, inputs[i]);
        nc_free_tensor(v);
        n->sizes.push_back(inputs[i]->dims[axis]);
        n->parents[i] = nc_dup_node(inputs[i]->node);
        pos += inputs[i]->dims[axis];
    }
    y = nc_finish(y, n, inputs, n_inputs);
    for (int i = 0; i < n_inputs; i++) nc_free_tensor(inputs[i]);
    return y;
}

extern "C" NCTensor *nc_vconcat(NCTensor **inputs, int n) { return nc_concat(inputs, n, 0); } // libnc.h:315
extern "C" NCTensor *nc_hconcat(NCTensor **inputs, int n) { return nc_concat(inputs, n, 1); } // libnc.h:317

extern "C" void nc_split(NCTensor **tab_y, NCTensor *x, int n_outputs, const size_t *tab_size, int axis) // libnc.h:318-320
{
    size_t pos = 0;
    for (int i = 0; i < n_outputs; i++) {
        size_t sz = tab_size ? tab_size[i] : x->dims[axis] / n_outputs;
        tab_y[i] = nc_slice(nc_dup_tensor(x), axis, pos, pos + sz);
        pos += sz;
    }
    nc_free_tensor(x);
}

// libnc.h:325-335 (nncp.c:777 left-pads w_r^T q from d_pos to K rows)
extern "C" NCTensor *nc_pad(NCTensor *x, ssize_t left_len, NCPadEnum left_op, ssize_t right_len, NCPadEnum right_op)
{
    x = nc_contig(x);
    need_f32(x, "nc_pad");
    size_t dims[NC_N_DIMS_MAX];
    memcpy(dims, x->dims, sizeof(size_t) * x->n_dims);
    ssize_t n_out = (ssize_t)dims[0] + left_len + right_len;
    if (x->n_dims < 1 || n_out <= 0) nc_fatal("nc_pad: empty result");
    dims[0] = (size_t)n_out;
    NCTensor *y = new_f32(x, x->n_dims, dims);
    k_pad(nc_stream(x), nc_f32(x), nc_f32(y), (int64_t)x->dims[0], (int64_t)(nc_numel(x) / x->dims[0]),
          left_len, left_op, right_len, right_op);
    LAUNCHED(x);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_PAD, 1, args);
    n->ia[0] = (int)left_len; n->ia[1] = left_op; n->ia[2] = (int)right_len; n->ia[3] = right_op;
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

// libnc.h:353-360: result axis i is x axis axis[i], made contiguous
static NCTensor *permute_raw(const NCTensor *x, int nd, const int *axis)
{
    if (nd != x->n_dims) nc_fatal("nc_permute: rank mismatch");
    NCTensor *v = nc_view(x);
    for (int i = 0; i < nd; i++) { v->dims[i] = x->dims[axis[i]]; v->strides[i] = x->strides[axis[i]]; }
    NCTensor *y = nc_alloc(x->dev, x->type, nd, v->dims, false);
    nc_copy_any(y, v);
    nc_free_tensor(v);
    return y;
}

extern "C" NCTensor *nc_permute(NCTensor *x, int n_dims, const int *axis)
{
    x = nc_contig(x);
    need_dev(x, "nc_permute");
    NCTensor *y = permute_raw(x, n_dims, axis);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_PERMUTE, 1, args);
    for (int i = 0; i < n_dims; i++) n->ia[i] = axis[i];
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_permute_4d(NCTensor *x, int a0, int a1, int a2, int a3)
{
    int axis[4] = { a0, a1, a2, a3 };
    return nc_permute(x, 4, axis);
}

// libnc.h:396-397 (see k_rel_shift): y[j,i] = x[j - (pos + i*mult), i]
extern "C" NCTensor *nc_rel_shift(NCTensor *x, ssize_t pos, ssize_t mult)
{
    x = nc_contig(x);
    need_f32(x, "nc_rel_shift");
    if (x->n_dims < 2) nc_fatal("nc_rel_shift: at least 2 axes expected");
    NCTensor *y = nc_alloc_like(x);
    k_rel_shift(nc_stream(x), nc_f32(x), nc_f32(y), (int64_t)x->dims[0], (int64_t)x->dims[1],
                (int64_t)(nc_numel(x) / (x->dims[0] * x->dims[1])), pos, mult, 0);
    LAUNCHED(x);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_REL_SHIFT, 1, args);
    n->ia[0] = (int)pos; n->ia[1] = (int)mult;
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_cmul(NCTensor *x1, NCTensor *x2, BOOL is_conj, BOOL is_planar)
{
    (void)x1; (void)x2; (void)is_conj; (void)is_planar;
    nc_fatal("nc_cmul (rotary position embedding, nncp.c:764-770) is not supported");
}

// ---- matmul -----------------------------------------------------------------
struct MMShape {
    size_t m, n, k, batch;
    bool flat;
};

static MMShape mm_shape(const NCTensor *a, const NCTensor *b, bool ta, bool tb)
{
    MMShape s;
    if (a->n_dims < 2 || b->n_dims < 2) nc_fatal("nc_matmul: operands need at least 2 axes");
    s.m = ta ? a->dims[1] : a->dims[0];
    s.k = ta ? a->dims[0] : a->dims[1];
    s.batch = 1;
    s.flat = false;
    size_t kb;
    if (a->n_dims == 2 && b->n_dims > 2 && !tb) {
        s.flat = true;
        kb = b->dims[0];
        s.n = nc_numel(b) / kb;
    } else {
        if (a->n_dims != b->n_dims) nc_fatal("nc_matmul: rank mismatch (%d vs %d)", a->n_dims, b->n_dims);
        for (int i = 2; i < a->n_dims; i++) {
            if (a->dims[i] != b->dims[i]) nc_fatal("nc_matmul: batch axis %d mismatch", i);
            s.batch *= a->dims[i];
        }
        kb = tb ? b->dims[1] : b->dims[0];
        s.n = tb ? b->dims[0] : b->dims[1];
    }
    if (s.k != kb) nc_fatal("nc_matmul: inner dimension mismatch (%zu vs %zu)", s.k, kb);
    return s;
}

// C (contiguous m x n per batch) = alpha op(A) op(B) + beta C [+ bias, act]
// `addend` (laid out like C, or NULL) is added after the activation; beta must be 0 with it
// forward: a product of the forward pass (honours nc_set_matmul_width_invariant)
// ---- k-major copies of weight matrices (nc_ext.h) -----------------------------------------
// A product with a few columns is bound by the cache lines its workgroups bring in; for a
// matrix stored with rows contiguous that is one line per k and workgroup, for a k-major
// copy a quarter of it.  The decoder keeps such copies of its weights for the timesteps of
// a segment; the products find them by the address of the matrix.
const float *nc_k_major_of(const NCContext *m, const float *a, size_t rows, size_t k)
{
    for (const KMajorCopy &e : m->k_major)
        if (e.src == a && e.m == rows && e.k == k) return nc_f32(e.copy);
    return nullptr;
}

extern "C" void nc_keep_k_major_weight(NCTensor *w)
{
    if (w->type == NC_TYPE_BF16) { // the copy is made of, and found by, the parameter's f32 copy
        NCTensor *v = nc_operand(nc_dup_tensor(w));
        nc_keep_k_major_weight(v);
        nc_free_tensor(v);
        return;
    }
    need_f32(w, "nc_keep_k_major_weight");
    if (w->n_dims != 2 || !nc_is_contig(w)) nc_fatal("nc_keep_k_major_weight: a contiguous (m, k) matrix expected");
    NCContext *m = nc_ctx(w);
    const size_t rows = w->dims[0], k = w->dims[1];
    if (nc_k_major_of(m, nc_f32(w), rows, k)) return;
    size_t dims[2] = { k, rows };
    NCTensor *copy = new_f32(w, 2, dims);
    k_transpose_f32(m->stream, nc_f32(w), nc_f32(copy), (int)rows, (int)k);
    m->launches++;
    m->k_major.push_back(KMajorCopy{ nc_f32(w), rows, k, copy });
}

extern "C" void nc_forget_k_major_weights(NCContext *m)
{
    for (KMajorCopy &e : m->k_major) nc_free_tensor(e.copy);
    m->k_major.clear();
}

// The product through the operands' bf16 shadows (bf16 mode, plain unbatched products whose
// shape the unguarded loaders take): no operand is converted inside the product, and none is
// cast more than once however many products read it.  want_c16: also leave the result's own
// shadow (it is the operand of a later product).  Returns false when this route does not
// apply (nothing launched).
struct Bf16Extra { const float *dpre = nullptr; int dact = 0; float *rowsum = nullptr; int *rows_written = nullptr; };
static bool dev_gemm_bf16_operands(NCContext *m, bool ta, bool tb, size_t M, size_t N, size_t K, float alpha,
                                   const NCTensor *a, const NCTensor *b, NCTensor *c, const float *bias, int act,
                                   float *pre, const float *addend, bool want_c16, const Bf16Extra *ex = nullptr)
{
    static const bool off = getenv("NCHIP_BF16_SHADOWS") && atoi(getenv("NCHIP_BF16_SHADOWS")) == 0;
    if (off || !m->matmul_bf16 || K % 64 || K < 64 || M < 64 || N < 16) return false;
    const size_t lda = ta ? K : M, ldb = tb ? N : K;
    if (lda % 8 || ldb % 8 || (!ta && M % 64) || (tb && N % 64)) return false;
    const uint16_t *a16 = nc_shadow_of(m, a), *b16 = a16 ? nc_shadow_of(m, b) : nullptr;
    if (!a16 || !b16) return false;
    NchipGemmBf16Args g;
    memset(&g, 0, sizeof(g));
    g.ta = ta; g.tb = tb; g.m = (int)M; g.n = (int)N; g.k = (int)K; g.alpha = alpha;
    g.A16 = a16; g.lda = (int64_t)lda; g.B16 = b16; g.ldb = (int64_t)ldb;
    g.C = nc_f32(c); g.ldc = (int64_t)M;
    g.bias = bias; g.act = act; g.pre = pre; g.addend = addend;
    if (ex) { g.dpre = ex->dpre; g.dact = ex->dact; g.rowsum = ex->rowsum; g.rows_written = ex->rows_written; }
    // (the result's shadow is claimed only once the launch is certain: a refused shape leaves it alone)
    const bool had = c->buf->sh_valid;
    g.C16 = want_c16 ? nc_shadow_for_write(m, c) : nullptr;
    int rc = nchip_gemm_bf16_operands(m->stream, &g);
    if (rc < 0) nc_fatal("gemm failed (bf16 operands, m=%zu n=%zu k=%zu)", M, N, K);
    if (rc > 0) {
        if (g.C16) c->buf->sh_valid = had;
        return false;
    }
    if (!g.C16) nc_shadow_invalidate(c);
    m->launches++;
    return true;
}

static void dev_gemm(NCContext *m, bool ta, bool tb, size_t M, size_t N, size_t K, float alpha,
                     const NCTensor *a, const NCTensor *b, float beta, NCTensor *c, size_t batch,
                     const float *bias, int act, float *pre, const float *addend = nullptr,
                     bool forward = false, bool want_c16 = false)
{
    const bool invariant = forward && m->matmul_invariant;
    if (forward && m->bf16_copy_results) want_c16 = true; // nc_set_bf16_copy_of_results
    if (m->matmul_bf16 && !invariant && batch == 1 && beta == 0.0f &&
        dev_gemm_bf16_operands(m, ta, tb, M, N, K, alpha, a, b, c, bias, act, pre, addend, want_c16))
        return;
    nc_shadow_invalidate(c);
    const int prec = m->matmul_bf16 | (invariant ? NCHIP_GEMM_WIDTH_INVARIANT : 0);
    int ks = invariant ? 1 : nchip_gemm_pick_ksplit((int)M, (int)N, (int)K, (int)batch);
    size_t cap = 0;
    float *ws = nullptr;
    if (ks > 1) ws = nc_tmp_f32(m, batch * ks * M * N, &cap);
    int rc;
    // a few columns against a weight matrix with a k-major copy: the same chains from the copy
    const float *a_data = nc_f32(a);
    if (invariant && !ta && !tb && batch == 1 && !m->matmul_bf16 && N <= 64 && M % 32 == 0 && K % 32 == 0 && K >= 32 &&
        alpha == 1.0f && beta == 0.0f && !m->k_major.empty()) {
        if (const float *km = nc_k_major_of(m, a_data, M, K)) {
            a_data = km;
            ta = true;
        }
    }
    if (addend)
        rc = nchip_gemm_add(m->stream, ta, tb, (int)M, (int)N, (int)K, alpha,
                            a_data, (int64_t)(ta ? K : M), (int64_t)(M * K),
                            nc_f32(b), (int64_t)(tb ? N : K), (int64_t)(K * N),
                            nc_f32(c), (int64_t)M, (int64_t)(M * N), (int)batch,
                            bias, act, pre, addend, prec, ks, ws);
    else
        rc = nchip_gemm(m->stream, ta, tb, (int)M, (int)N, (int)K, alpha,
                        a_data, (int64_t)(ta ? K : M), (int64_t)(M * K),
                        nc_f32(b), (int64_t)(tb ? N : K), (int64_t)(K * N),
                        beta, nc_f32(c), (int64_t)M, (int64_t)(M * N), (int)batch,
                        bias, act, pre, prec, ks, ws);
    if (ws) nc_tmp_free(m, ws, cap);
    if (rc) nc_fatal("gemm failed (m=%zu n=%zu k=%zu)", M, N, K);
    m->launches += ks > 1 ? 2 : 1;
}

// libnc.h:365-373
extern "C" NCTensor *nc_matmul_add(NCTensor *a, NCTensor *b, NCTensor *c, BOOL ta, BOOL tb, float alpha)
{
    a = nc_contig(a); b = nc_contig(b);
    need_f32(a, "nc_matmul"); need_f32(b, "nc_matmul");
    NCContext *m = nc_ctx(a);
    MMShape s = mm_shape(a, b, ta != 0, tb != 0);
    size_t dims[NC_N_DIMS_MAX];
    memcpy(dims, b->dims, sizeof(size_t) * b->n_dims);
    dims[0] = s.m;
    if (!s.flat) dims[1] = s.n;
    NCTensor *y = new_f32(a, b->n_dims, dims);
    if (c) {
        c = nc_contig(c);
        need_f32(c, "nc_matmul_add");
        if (nc_numel(c) != nc_numel(y)) nc_fatal("nc_matmul_add: addend shape mismatch");
    }
    // the addend is read in the GEMM epilogue: no copy, no second pass
    dev_gemm(m, ta != 0, tb != 0, s.m, s.n, s.k, alpha, a, b, 0.0f, y, s.batch, nullptr, 0, nullptr,
             c ? nc_f32(c) : nullptr, true);
    NCTensor *args[3] = { a, b, c };
    NCNode *n = nc_new_node(m, OP_MATMUL, 3, args);
    if (a->node || b->node || (c && c->node)) {
        n->saved[0] = nc_view(a);
        n->saved[1] = nc_view(b);
    }
    n->ia[0] = ta != 0; n->ia[1] = tb != 0; n->ia[2] = s.flat;
    n->fa[0] = alpha;
    y = nc_finish(y, n, args, 3);
    nc_free_tensor(a); nc_free_tensor(b); nc_free_tensor(c);
    return y;
}

extern "C" NCTensor *nc_matmul(NCTensor *w, NCTensor *x) { return nc_matmul_add(w, x, nullptr, 0, 0, 1.0f); }

// During nc_backward: the gradient already delivered to parent `arg` of the
// node being processed, when a kernel can add it in its own epilogue instead of
// a separate element-wise sum.  Taking it marks it as consumed.
static const float *nc_bw_addend(NCContext *m, int arg, size_t numel)
{
    if (arg >= NC_BW_ARGS || !m->bw_prev[arg]) return nullptr;
    NCTensor *p = m->bw_prev[arg];
    if (p->type != NC_TYPE_F32 || !nc_is_contig(p) || nc_numel(p) != numel) return nullptr;
    m->bw_used[arg] = true;
    return nc_f32(p);
}

// gradients of alpha op(A) op(B): the four transposition cases
static void matmul_bw(NCNode *nd, NCTensor *g, NCTensor **ga, int ia, int ib)
{
    NCTensor *a = nd->saved[0], *b = nd->saved[1];
    if (!a || !b) nc_fatal("matmul backward: arguments were not saved");
    NCContext *m = nc_ctx(g);
    bool ta = nd->ia[0], tb = nd->ia[1];
    float alpha = nd->fa[0];
    MMShape s = mm_shape(a, b, ta, tb);
    if (nd->parents[ia]) {
        NCTensor *da = nc_alloc_like(a);
        NCNode *pa = nd->parents[ia];
        // dW = alpha * dY * X^T of a plain linear layer whose weight is used once
        // or twice (K/V of the segment and of the memory): postponed to the
        // grouped launch at the end of nc_backward; the second use joins the
        // first as a second k range of the same problem
        DeferredGemm *open_entry = nullptr;
        for (DeferredGemm &e : m->deferred)
            if (e.param == pa) open_entry = &e;
        const bool plain = m->defer_wgrad && !ta && !tb && s.batch == 1 && pa->op == OP_PARAM;
        if (plain && !open_entry && pa->consumers <= 2) {
            DeferredGemm d;
            d.a = nc_contig(nc_dup_tensor(g)); d.b = nc_dup_tensor(b); d.c = nc_dup_tensor(da);
            d.a2 = d.b2 = nullptr; d.k2 = 0;
            d.m = (int)s.m; d.n = (int)s.k; d.k = (int)s.n; d.alpha = alpha;
            d.param = pa;
            m->deferred.push_back(d);
            ga[ia] = da;
        } else if (plain && open_entry && !open_entry->a2 && open_entry->m == (int)s.m &&
                   open_entry->n == (int)s.k && open_entry->k % 64 == 0 && open_entry->alpha == alpha) {
            open_entry->a2 = nc_contig(nc_dup_tensor(g));
            open_entry->b2 = nc_dup_tensor(b);
            open_entry->k2 = (int)s.n;
            nc_free_tensor(da); // the first use's tensor receives the whole gradient
        } else {
            if (!ta) dev_gemm(m, false, !tb, s.m, s.k, s.n, alpha, g, b, 0.0f, da, s.batch, nullptr, 0, nullptr);
            else     dev_gemm(m, tb, true, s.k, s.m, s.n, alpha, b, g, 0.0f, da, s.batch, nullptr, 0, nullptr);
            ga[ia] = da;
        }
    }
    if (nd->parents[ib]) {
        NCTensor *db = nc_alloc_like(b);
        // a gradient already delivered to this parent is added in the epilogue
        const float *prev = nc_bw_addend(m, ib, nc_numel(db));
        // x came out of nc_linear's activation and feeds nothing else: its
        // backward step (times act'(pre)) rides in this GEMM's epilogue
        NCNode *px = nd->parents[ib];
        if (!prev && !tb && s.batch == 1 && px->op == OP_LINEAR && px->ia[3] != NC_ACT_NONE && px->consumers == 1 &&
            px->saved[2] && nc_numel(px->saved[2]) == nc_numel(db) && nc_is_contig(px->saved[2])) {
            int ks = nchip_gemm_pick_ksplit((int)s.k, (int)s.n, (int)s.m, 1);
            size_t cap = 0;
            float *ws = ks > 1 ? nc_tmp_f32(m, (size_t)ks * s.k * s.n, &cap) : nullptr;
            // px's bias gradient is the row sum of this product: its partial sums come out of
            // the same epilogue when px's bias can wait for the batched sum at the end
            float *rs = nullptr;
            size_t rs_cap = 0;
            int rs_rows = 0;
            if (px->n_args > 2 && px->parents.size() > 2 && px->parents[2] && nc_can_defer_sum(m, px->parents[2]) && ks == 1)
                rs = nc_tmp_f32(m, (size_t)nchip_gemm_rowsum_rows((int)s.n) * s.k, &rs_cap);
            bool done = false;
            if (m->matmul_bf16 && ks == 1) {
                // operands from their bf16 shadows; the result (the gradient of the pre-activation) is
                // the operand of the next two products, so its shadow comes out of this epilogue too
                Bf16Extra ex;
                ex.dpre = nc_f32(px->saved[2]); ex.dact = px->ia[3]; ex.rowsum = rs; ex.rows_written = &rs_rows;
                done = dev_gemm_bf16_operands(m, !ta, false, s.k, s.n, s.m, alpha, a, g, db, nullptr, 0, nullptr, nullptr,
                                              true, &ex);
                if (done) m->launches--; // (counted below)
            }
            if (!done &&
                nchip_gemm_dact_rowsum(m->stream, !ta, 0, (int)s.k, (int)s.n, (int)s.m, alpha,
                                       nc_f32(a), (int64_t)(!ta ? s.m : s.k), nc_f32(g), (int64_t)s.m,
                                       nc_f32(db), (int64_t)s.k, nc_f32(px->saved[2]), px->ia[3],
                                       m->matmul_bf16, ks, ws, rs, &rs_rows))
                nc_fatal("gemm failed (activation-gradient epilogue)");
            if (rs && rs_rows > 0) {
                px->grad_rowsum = rs; px->grad_rowsum_cap = rs_cap; px->grad_rowsum_rows = rs_rows;
            } else if (rs) {
                nc_tmp_free(m, rs, rs_cap);
            }
            if (ws) nc_tmp_free(m, ws, cap);
            m->launches += ks > 1 ? 2 : 1;
            px->ia[5] = 1; // the gradient delivered to px is already d(pre-activation)
        } else
        // (the gradient of an attention output is an operand of the bf16 attention backward:
        // its bf16 copy comes out of this product's epilogue)
        if (!tb) dev_gemm(m, !ta, false, s.k, s.n, s.m, alpha, a, g, 0.0f, db, s.batch, nullptr, 0, nullptr, prev, false,
                          px->op == OP_ATTN);
        else     dev_gemm(m, true, ta, s.n, s.k, s.m, alpha, g, a, 0.0f, db, s.batch, nullptr, 0, nullptr, prev);
        ga[ib] = db;
    }
}

// y = act(w x + bias) [+ res] in one GEMM with a fused epilogue (nc_ext.h)
static NCTensor *linear_impl(NCTensor *w, NCTensor *x, NCTensor *bias, int act, NCTensor *res)
{
    w = nc_contig(w); x = nc_contig(x);
    need_f32(w, "nc_linear"); need_f32(x, "nc_linear");
    NCContext *m = nc_ctx(w);
    if (w->n_dims != 2) nc_fatal("nc_linear: w must be (m, k)");
    MMShape s = mm_shape(w, x, false, false);
    if (bias) {
        bias = nc_contig(bias);
        need_f32(bias, "nc_linear");
        if (nc_numel(bias) != s.m) nc_fatal("nc_linear: bias must have m = %zu elements", s.m);
    }
    size_t dims[NC_N_DIMS_MAX];
    memcpy(dims, x->dims, sizeof(size_t) * x->n_dims);
    dims[0] = s.m;
    NCTensor *y = new_f32(w, x->n_dims, dims);
    if (res) {
        res = nc_contig(res);
        need_f32(res, "nc_linear_add");
        if (nc_numel(res) != nc_numel(y)) nc_fatal("nc_linear_add: res must have the shape of the result");
    }
    bool graph = w->node || x->node || (bias && bias->node) || (res && res->node);
    NCTensor *pre = (act != NC_ACT_NONE && graph) ? nc_alloc_like(y) : nullptr;
    // (an activated result feeds the next linear layer: in bf16 mode its operand copy is
    // written by this product's epilogue)
    dev_gemm(m, false, false, s.m, s.n, s.k, 1.0f, w, x, 0.0f, y, 1, bias ? nc_f32(bias) : nullptr, act,
             pre ? nc_f32(pre) : nullptr, res ? nc_f32(res) : nullptr, true, act != NC_ACT_NONE);
    NCTensor *args[4] = { w, x, bias, res };
    NCNode *n = nc_new_node(m, OP_LINEAR, 4, args);
    if (graph) {
        n->saved[0] = nc_view(w);
        n->saved[1] = nc_view(x);
        n->saved[2] = pre;
        pre = nullptr;
    }
    n->ia[0] = 0; n->ia[1] = 0; n->ia[2] = 1; n->ia[3] = act;
    n->fa[0] = 1.0f;
    y = nc_finish(y, n, args, 4);
    nc_free_tensor(pre);
    nc_free_tensor(w); nc_free_tensor(x); nc_free_tensor(bias); nc_free_tensor(res);
    return y;
}

extern "C" NCTensor *nc_linear(NCTensor *w, NCTensor *x, NCTensor *bias, int act)
{
    return linear_impl(w, x, bias, act, nullptr);
}

extern "C" NCTensor *nc_linear_add(NCTensor *w, NCTensor *x, NCTensor *bias, int act, NCTensor *res)
{
    return linear_impl(w, x, bias, act, res);
}

// nc_ext.h: the two projections of one decoder timestep in one launch.  Returns w0 x + bias0
// and writes w1 x into slice `index` of the last axis of dst.  No gradient.
extern "C" NCTensor *nc_linear_pair_into(NCTensor *w0, NCTensor *bias0, NCTensor *w1, NCTensor *x,
                                         NCTensor *dst, int index)
{
    w0 = nc_contig(w0); w1 = nc_contig(w1); x = nc_contig(x);
    need_f32(w0, "nc_linear_pair_into"); need_f32(w1, "nc_linear_pair_into"); need_f32(x, "nc_linear_pair_into");
    need_f32(dst, "nc_linear_pair_into");
    if (bias0) { bias0 = nc_contig(bias0); need_f32(bias0, "nc_linear_pair_into"); }
    NCContext *m = nc_ctx(w0);
    if (w0->n_dims != 2 || w1->n_dims != 2 || x->n_dims != 2 || w0->dims[1] != x->dims[0] || w1->dims[1] != x->dims[0])
        nc_fatal("nc_linear_pair_into: w0 (m0, k), w1 (m1, k) and x (k, n) expected");
    const size_t m0 = w0->dims[0], m1 = w1->dims[0], k = x->dims[0], n = x->dims[1];
    if (dst->n_dims != 3 || dst->dims[0] != m1 || dst->dims[1] != n || index < 0 || (size_t)index >= dst->dims[2] ||
        !nc_is_contig(dst))
        nc_fatal("nc_linear_pair_into: dst must be a contiguous (m1, n, T) tensor and 0 <= index < T");
    if (bias0 && nc_numel(bias0) != m0) nc_fatal("nc_linear_pair_into: bias0 must have m0 elements");
    size_t dims[2] = { m0, n };
    NCTensor *y0 = new_f32(w0, 2, dims);
    float *slot = nc_f32(dst) + (size_t)index * m1 * n;
    nc_shadow_invalidate(dst);
    int rc = 1;
    if (m->matmul_invariant && !m->matmul_bf16) {
        const float *k0 = nc_k_major_of(m, nc_f32(w0), m0, k), *k1 = nc_k_major_of(m, nc_f32(w1), m1, k);
        const bool km = k0 && k1;
        rc = nchip_gemm_pair_few_columns(m->stream, (int)m0, (int)m1, (int)n, (int)k, km ? k0 : nc_f32(w0), (int64_t)(km ? k : m0),
                                         km ? k1 : nc_f32(w1), (int64_t)(km ? k : m1), nc_f32(x), (int64_t)k, nc_f32(y0), (int64_t)m0,
                                         slot, (int64_t)m1, bias0 ? nc_f32(bias0) : nullptr, nullptr, km);
    }
    if (rc < 0) nc_fatal("nc_linear_pair_into: kernel rejected the shapes");
    if (rc == 0) {
        m->launches++;
    } else {
        // other shapes and modes: the two products one after the other (the second one
        // writes its columns straight into the slot: ldc = m1)
        dev_gemm(m, false, false, m0, n, k, 1.0f, w0, x, 0.0f, y0, 1, bias0 ? nc_f32(bias0) : nullptr, 0, nullptr, nullptr, true);
        NCTensor *view = nc_slice_alias(dst, 2, (size_t)index, (size_t)index + 1);
        view = nc_reshape_2d(view, m1, n);
        dev_gemm(m, false, false, m1, n, k, 1.0f, w1, x, 0.0f, view, 1, nullptr, 0, nullptr, nullptr, true);
        nc_free_tensor(view);
    }
    nc_free_tensor(w0); nc_free_tensor(bias0); nc_free_tensor(w1); nc_free_tensor(x);
    return y0;
}

// ---- embedding, softmax, loss, norms ----------------------------------------
extern "C" NCTensor *nc_get_col(NCTensor *w, NCTensor *x) // libnc.h:374-375
{
    w = nc_contig(w); x = nc_contig(x);
    need_f32(w, "nc_get_col"); need_dev(x, "nc_get_col");
    if (x->type != NC_TYPE_I32 || w->n_dims != 2) nc_fatal("nc_get_col: (D,V) f32 matrix and i32 indices expected");
    size_t dims[2] = { w->dims[0], nc_numel(x) };
    NCTensor *y = new_f32(w, 2, dims);
    if (nchip_get_col(nc_stream(w), nc_f32(w), (const int32_t *)nc_data(x), nc_f32(y), (int)dims[0],
                      (int)w->dims[1], (int64_t)dims[1]))
        nc_fatal("nc_get_col failed");
    LAUNCHED(w);
    NCTensor *args[1] = { w };
    NCNode *n = nc_new_node(nc_ctx(w), OP_GET_COL, 1, args);
    n->saved[0] = nc_view(x);
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(w); nc_free_tensor(x);
    return y;
}

// nc_ext.h: nc_get_col with the indices read by the kernel straight from pinned host memory
// (a decoder timestep's 32 tokens: an upload of their own costs a launch and its latency).
// The index tensor must stay as it is until the stream has been waited for.  The columns come
// out multiplied by `scale` (the embedding multiplier: one launch less).  No gradient.
extern "C" NCTensor *nc_get_col_host_indices(NCTensor *w, NCTensor *x, float scale)
{
    w = nc_contig(w);
    need_f32(w, "nc_get_col_host_indices");
    if (x->dev->is_hip || x->type != NC_TYPE_I32 || !nc_is_contig(x) || w->n_dims != 2)
        nc_fatal("nc_get_col_host_indices: (D,V) f32 matrix on the GPU and contiguous i32 indices on the host expected");
    size_t dims[2] = { w->dims[0], nc_numel(x) };
    NCTensor *y = new_f32(w, 2, dims);
    if (nchip_get_col_scaled(nc_stream(w), nc_f32(w), (const int32_t *)nc_data(x), nc_f32(y), (int)dims[0],
                             (int)w->dims[1], (int64_t)dims[1], scale))
        nc_fatal("nc_get_col_host_indices failed");
    LAUNCHED(w);
    nc_mark_in_flight(x); // the kernel has yet to read the indices: their buffer outlives this reference
    nc_free_tensor(w); nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_soft_max(NCTensor *x) // libnc.h:382
{
    x = nc_contig(x);
    need_f32(x, "nc_soft_max");
    NCTensor *y = nc_alloc_like(x);
    size_t v = x->n_dims ? x->dims[0] : 1;
    if (nchip_softmax_fwd(nc_stream(x), nc_f32(x), nc_f32(y), (int)v, (int64_t)(nc_numel(x) / v)))
        nc_fatal("nc_soft_max failed");
    LAUNCHED(x);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_SOFT_MAX, 1, args);
    if (x->node) n->saved[0] = nc_view(y);
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x);
    return y;
}

// libnc.h:385-388; straight after nc_soft_max the gradient goes to the logits
// as g*(onehot - p)
extern "C" NCTensor *nc_indexed_log(NCTensor *x, NCTensor *eout)
{
    x = nc_contig(x); eout = nc_contig(eout);
    need_f32(x, "nc_indexed_log"); need_dev(eout, "nc_indexed_log");
    if (eout->type != NC_TYPE_I32) nc_fatal("nc_indexed_log: i32 indices expected");
    size_t v = x->dims[0], cols = nc_numel(x) / v;
    if (nc_numel(eout) != cols) nc_fatal("nc_indexed_log: %zu indices for %zu columns", nc_numel(eout), cols);
    NCTensor *y = new_f32(x, x->n_dims - 1, x->dims + 1);
    if (nchip_indexed_log(nc_stream(x), nc_f32(x), (const int32_t *)nc_data(eout), nc_f32(y), (int)v, (int64_t)cols))
        nc_fatal("nc_indexed_log failed");
    LAUNCHED(x);
    NCTensor *args[1] = { x };
    NCNode *n = nc_new_node(nc_ctx(x), OP_INDEXED_LOG, 1, args);
    if (x->node) {
        n->saved[0] = nc_view(x);
        n->saved[1] = nc_view(eout);
        if (x->node->op == OP_SOFT_MAX && x->node->parents[0]) {
            nc_free_node(n->parents[0]);
            n->parents[0] = nc_dup_node(x->node->parents[0]);
            n->ia[0] = 1;
        }
    }
    y = nc_finish(y, n, args, 1);
    nc_free_tensor(x); nc_free_tensor(eout);
    return y;
}

// libnc.h:389-395
static NCTensor *norm_op(NCTensor *x, NCTensor *w, NCTensor *b, float eps, int avg)
{
    x = nc_contig(x);
    need_f32(x, "layer norm");
    if (w) { w = nc_contig(w); b = nc_contig(b); need_f32(w, "layer norm"); need_f32(b, "layer norm"); }
    size_t d = x->dims[0], cols = nc_numel(x) / d;
    if (w && (nc_numel(w) != d || nc_numel(b) != d)) nc_fatal("layer norm: affine parameters must have %zu elements", d);
    NCTensor *y = nc_alloc_like(x);
    NCTensor *xhat = w ? nc_alloc_like(x) : nc_dup_tensor(y);
    NCTensor *rstd = nc_alloc(x->dev, NC_TYPE_F32, 1, &cols, false);
    // bf16 products: the normalised columns are the operand of the products that follow, so
    // their bf16 copy is written here and never cast
    uint16_t *y16 = nc_ctx(x)->matmul_bf16 ? nc_shadow_for_write(nc_ctx(x), y) : nullptr;
    if (nchip_norm_fwd_bf16copy(nc_stream(x), nc_f32(x), w ? nc_f32(w) : nullptr, b ? nc_f32(b) : nullptr, nc_f32(y),
                                nc_f32(xhat), nc_f32(rstd), (int)d, (int64_t)cols, eps, avg, y16))
        nc_fatal("layer norm failed");
    LAUNCHED(x);
    NCTensor *args[3] = { x, w, b };
    NCNode *n = nc_new_node(nc_ctx(x), OP_NORM, 3, args);
    if (x->node || (w && (w->node || b->node))) {
        n->saved[0] = nc_view(xhat);
        n->saved[1] = nc_view(rstd);
        if (w) n->saved[2] = nc_view(w);
    }
    n->ia[0] = avg;
    y = nc_finish(y, n, args, 3);
    nc_free_tensor(xhat); nc_free_tensor(rstd);
    nc_free_tensor(x); nc_free_tensor(w); nc_free_tensor(b);
    return y;
}

extern "C" NCTensor *nc_layer_norm(NCTensor *x, float eps) { return norm_op(x, nullptr, nullptr, eps, 1); }
extern "C" NCTensor *nc_rms_norm(NCTensor *x, float eps) { return norm_op(x, nullptr, nullptr, eps, 0); }

extern "C" NCTensor *nc_fused_layer_norm(NCTensor *x, NCTensor *w, NCTensor *b, float eps, BOOL avg_flag)
{
    if ((w == nullptr) != (b == nullptr)) nc_fatal("nc_fused_layer_norm: w and b go together");
    return norm_op(x, w, b, eps, avg_flag != 0);
}

// nc_ext.h: one or two products of the normalised x in one launch, the decoder's way of not
// paying a launch for the layer norm between two blocks.  y0 = act0(w0 norm(x) + bias0);
// with w1, w1 norm(x) goes into slice `index` of dst; *pnormed (when asked for) is norm(x).
// Same bits as nc_fused_layer_norm + nc_linear / nc_linear_pair_into.  No gradient.
extern "C" NCTensor *nc_norm_linear_pair_into(NCTensor *x, NCTensor *g, NCTensor *b, float eps, BOOL avg_flag,
                                              NCTensor *w0, NCTensor *bias0, int act0,
                                              NCTensor *w1, NCTensor *dst, int index, NCTensor **pnormed)
{
    const char *me = "nc_norm_linear_pair_into";
    if ((g == nullptr) != (b == nullptr)) nc_fatal("%s: g and b go together", me);
    if ((w1 == nullptr) != (dst == nullptr)) nc_fatal("%s: w1 and dst go together", me);
    if (dst) nc_shadow_invalidate(dst);
    // (checked before a path is chosen: the pair kernel would apply act0 to the cache column too)
    if (w1 && act0 != NC_ACT_NONE) nc_fatal("%s: no activation on the first product of a pair", me);
    x = nc_contig(x); w0 = nc_contig(w0);
    need_f32(x, me); need_f32(w0, me);
    // (the other operands are taken as they are, so that the shapes this kernel does not
    // cover fall through to the plain ops below; bf16 parameters are widened here)
    if (g && g->type == NC_TYPE_BF16) g = nc_operand(g);
    if (b && b->type == NC_TYPE_BF16) b = nc_operand(b);
    if (bias0 && bias0->type == NC_TYPE_BF16) bias0 = nc_operand(bias0);
    if (w1 && w1->type == NC_TYPE_BF16) w1 = nc_operand(w1);
    NCContext *m = nc_ctx(w0);
    int rc = 1;
    NCTensor *y0 = nullptr, *normed = nullptr;
    if (x->n_dims == 2 && w0->n_dims == 2 && w0->dims[1] == x->dims[0] && m->matmul_invariant && !m->matmul_bf16 &&
        (!g || (g->type == NC_TYPE_F32 && b->type == NC_TYPE_F32 && nc_is_contig(g) && nc_is_contig(b) &&
                nc_numel(g) == x->dims[0] && nc_numel(b) == x->dims[0])) &&
        (!bias0 || (bias0->type == NC_TYPE_F32 && nc_is_contig(bias0) && nc_numel(bias0) == w0->dims[0])) &&
        (!w1 || (w1->type == NC_TYPE_F32 && nc_is_contig(w1) && w1->n_dims == 2 && w1->dims[1] == x->dims[0] &&
                 dst->type == NC_TYPE_F32 && nc_is_contig(dst) && dst->n_dims == 3 && dst->dims[0] == w1->dims[0] &&
                 dst->dims[1] == x->dims[1] && index >= 0 && (size_t)index < dst->dims[2])) &&
        (act0 == NC_ACT_NONE || act0 == NC_ACT_GELU || act0 == NC_ACT_RELU)) {
        const size_t k = x->dims[0], n = x->dims[1], m0 = w0->dims[0], m1 = w1 ? w1->dims[0] : 0;
        size_t d0[2] = { m0, n }, dn[2] = { k, n };
        y0 = new_f32(w0, 2, d0);
        if (pnormed) normed = new_f32(w0, 2, dn);
        const float *k0 = nc_k_major_of(m, nc_f32(w0), m0, k), *k1 = w1 ? nc_k_major_of(m, nc_f32(w1), m1, k) : nullptr;
        const bool km = k0 && (!w1 || k1);
        rc = nchip_norm_gemm_few_columns(m->stream, g ? nc_f32(g) : nullptr, b ? nc_f32(b) : nullptr, eps, avg_flag != 0,
                                         normed ? nc_f32(normed) : nullptr, (int64_t)k, (int)m0, (int)m1, (int)n, (int)k,
                                         km ? k0 : nc_f32(w0), (int64_t)(km ? k : m0), w1 ? (km ? k1 : nc_f32(w1)) : nullptr,
                                         (int64_t)(km ? k : m1), nc_f32(x), (int64_t)k,
                                         nc_f32(y0), (int64_t)m0, w1 ? nc_f32(dst) + (size_t)index * m1 * n : nullptr, (int64_t)m1,
                                         bias0 ? nc_f32(bias0) : nullptr, nullptr,
                                         act0 == NC_ACT_GELU ? NCHIP_ACT_GELU : act0 == NC_ACT_RELU ? NCHIP_ACT_RELU : NCHIP_ACT_NONE,
                                         km);
        if (rc < 0) nc_fatal("%s: kernel rejected the shapes", me);
        if (rc != 0) {
            nc_free_tensor(y0); nc_free_tensor(normed);
            y0 = normed = nullptr;
        }
    }
    if (rc == 0) {
        m->launches++;
        nc_free_tensor(x); nc_free_tensor(g); nc_free_tensor(b);
        nc_free_tensor(w0); nc_free_tensor(bias0); nc_free_tensor(w1);
    } else { // other shapes and modes: the steps one after the other
        normed = g ? nc_fused_layer_norm(x, g, b, eps, avg_flag) : nc_fused_layer_norm(x, nullptr, nullptr, eps, avg_flag);
        if (w1) {
            y0 = nc_linear_pair_into(w0, bias0, w1, nc_dup_tensor(normed), dst, index);
        } else {
            y0 = nc_linear(w0, nc_dup_tensor(normed), bias0, act0);
        }
        if (!pnormed) { nc_free_tensor(normed); normed = nullptr; }
    }
    if (pnormed) *pnormed = normed;
    return y0;
}

// ---- fused attention (nc_ext.h) ---------------------------------------------
struct AttnDims {
    int H, dk, dv, B, T, M, K, d_pos;
};

static AttnDims attn_dims(const NCTensor *q, const NCTensor *kv, const NCTensor *kvm,
                          const NCTensor *w_r, const NCTensor *b_r, int n_head, int d_key)
{
    AttnDims a;
    if (q->n_dims != 3 || kv->n_dims != 3) nc_fatal("nc_relpos_attention: q and kv must be (features, B, T)");
    a.H = n_head; a.dk = d_key;
    a.B = (int)q->dims[1]; a.T = (int)q->dims[2];
    a.M = kvm ? (int)kvm->dims[2] : 0;
    a.K = a.M + a.T;
    if ((int)q->dims[0] != n_head * d_key || kv->dims[1] != q->dims[1] || kv->dims[2] != q->dims[2])
        nc_fatal("nc_relpos_attention: q/kv shape mismatch");
    if (kv->dims[0] <= q->dims[0] || (kv->dims[0] - q->dims[0]) % n_head)
        nc_fatal("nc_relpos_attention: kv must hold H*dk key rows then H*dv value rows");
    a.dv = (int)(kv->dims[0] - q->dims[0]) / n_head;
    if (kvm && (kvm->n_dims != 3 || kvm->dims[0] != kv->dims[0] || kvm->dims[1] != kv->dims[1]))
        nc_fatal("nc_relpos_attention: kv_mem shape mismatch");
    a.d_pos = 1;
    if (w_r) {
        if (w_r->n_dims != 3 || (int)w_r->dims[0] != d_key || (int)w_r->dims[2] != n_head)
            nc_fatal("nc_relpos_attention: w_r must be (dk, d_pos, H)");
        a.d_pos = (int)w_r->dims[1];
        if (a.d_pos > a.K) nc_fatal("nc_relpos_attention: d_pos > K is not supported");
    }
    if (b_r && (b_r->n_dims != 2 || (int)b_r->dims[0] != a.K || (int)b_r->dims[1] != n_head))
        nc_fatal("nc_relpos_attention: b_r must be (K, H)");
    return a;
}

extern "C" NCTensor *nc_relpos_attention(NCTensor *q, NCTensor *kv, NCTensor *kv_mem, NCTensor *w_r,
                                         NCTensor *b_r, int n_head, int d_key, int attn_len,
                                         float b_r_scale)
{
    NCTensor *all[5] = { nc_contig(q), nc_contig(kv), kv_mem ? nc_contig(kv_mem) : nullptr,
                         w_r ? nc_contig(w_r) : nullptr, b_r ? nc_contig(b_r) : nullptr };
    for (int i = 0; i < 5; i++)
        if (all[i]) need_f32(all[i], "nc_relpos_attention");
    NCContext *m = nc_ctx(all[0]);
    AttnDims a = attn_dims(all[0], all[1], all[2], all[3], all[4], n_head, d_key);
    size_t od[3] = { (size_t)a.H * a.dv, (size_t)a.B, (size_t)a.T };
    size_t pd[4] = { (size_t)a.K, (size_t)a.T, (size_t)a.H, (size_t)a.B };
    NCTensor *y = new_f32(all[0], 3, od);
    // bf16 products: the attention runs on the bf16 matrix cores from the operands' bf16 copies
    // (left behind by the products that made q / kv and by the optimiser for w_r) when the
    // head shape is that kernel's; the probabilities are then kept as bf16
    bool on_bf16 = false;
    NCTensor *probs = nullptr;
    static const bool bf16_attn_off = getenv("NCHIP_BF16_ATTENTION") && atoi(getenv("NCHIP_BF16_ATTENTION")) == 0;
    // (not in width-invariant mode: there the per-timestep decoder must find the bits of this
    // whole-segment evaluation, and its one-query kernel computes in fp32)
    if (m->matmul_bf16 && !m->matmul_invariant && !bf16_attn_off && k_attn_bf16_shape_ok(a.dk, a.dv, a.T, a.K, a.d_pos, all[3] != nullptr) &&
        all[0]->dims[0] % 8 == 0 && all[1]->dims[0] % 8 == 0) {
        const uint16_t *q16 = nc_shadow_of(m, all[0]), *kv16 = nc_shadow_of(m, all[1]);
        const uint16_t *kvm16 = all[2] ? nc_shadow_of(m, all[2]) : nullptr;
        const uint16_t *w16 = all[3] ? nc_shadow_of(m, all[3]) : nullptr;
        if (q16 && kv16 && (!all[2] || kvm16) && (!all[3] || w16)) {
            probs = nc_alloc(all[0]->dev, NC_TYPE_U16, 4, pd, false);
            Bf16AttnFwdArgs g;
            g.q = q16; g.kv = kv16; g.kvm = kvm16; g.w_r = w16; g.b_r = all[4] ? nc_f32(all[4]) : nullptr;
            g.out = nc_f32(y); g.out16 = nc_shadow_for_write(m, y); g.probs = (uint16_t *)nc_data(probs);
            g.ldq = (int64_t)all[0]->dims[0]; g.ldkv = (int64_t)all[1]->dims[0]; g.ldo = (int64_t)od[0];
            g.H = a.H; g.B = a.B; g.T = a.T; g.M = a.M; g.K = a.K; g.d_pos = a.d_pos; g.attn_len = attn_len;
            g.b_r_scale = b_r_scale; g.scale = 1.0f / sqrtf((float)a.dk);
            if (k_attn_bf16_fwd(m->stream, g)) nc_fatal("nc_relpos_attention: bf16 kernel launch failed");
            m->launches++;
            on_bf16 = true;
        }
    }
    if (!probs) probs = new_f32(all[0], 4, pd);
    size_t cap = 0;
    float *rel = (all[3] && !on_bf16) ? nc_tmp_f32(m, (size_t)a.d_pos * a.T * a.H * a.B, &cap) : nullptr;
    int rc = on_bf16 ? 0 : nchip_relpos_attn_fwd(m->stream, nc_f32(all[0]), (int64_t)all[0]->dims[0],
                                   nc_f32(all[1]), all[2] ? nc_f32(all[2]) : nullptr, (int64_t)all[1]->dims[0],
                                   all[3] ? nc_f32(all[3]) : nullptr, all[4] ? nc_f32(all[4]) : nullptr,
                                   nc_f32(y), (int64_t)od[0], nc_f32(probs), rel,
                                   a.H, a.dk, a.dv, a.B, a.T, a.M, a.d_pos, attn_len, b_r_scale,
                                   0 /* attention stays fp32 in the bf16 variant */);
    if (rel) nc_tmp_free(m, rel, cap);
    if (rc) nc_fatal("nc_relpos_attention: kernel rejected the shapes");
    if (!on_bf16) m->launches += nchip_relpos_attn_last_launches();
    NCNode *n = nc_new_node(m, OP_ATTN, 5, all);
    bool graph = false;
    for (int i = 0; i < 5; i++)
        if (all[i] && all[i]->node) graph = true;
    if (graph) {
        for (int i = 0; i < 4; i++)
            if (all[i]) n->saved[i] = nc_view(all[i]);
        n->saved[4] = probs;
        probs = nullptr;
    }
    n->ia[0] = n_head; n->ia[1] = d_key; n->ia[2] = attn_len;
    n->ia[3] = all[3] != nullptr; n->ia[4] = all[4] != nullptr;
    n->fa[0] = b_r_scale;
    y = nc_finish(y, n, all, 5);
    nc_free_tensor(probs);
    for (int i = 0; i < 5; i++) nc_free_tensor(all[i]);
    return y;
}

// nc_ext.h: one query position against the segment's K/V cache; no graph
extern "C" NCTensor *nc_relpos_attention_step(NCTensor *q, NCTensor *kv_cache, NCTensor *kv_mem,
                                              NCTensor *w_r, NCTensor *b_r, int n_head, int d_key,
                                              int attn_len, float b_r_scale, int t)
{
    NCTensor *all[5] = { q, kv_cache, kv_mem, w_r, b_r };
    for (int i = 0; i < 5; i++)
        if (all[i]) { all[i] = nc_contig(all[i]); need_f32(all[i], "nc_relpos_attention_step"); }
    NCContext *m = nc_ctx(all[0]);
    if (all[0]->n_dims != 2 || all[1]->n_dims != 3 || all[0]->dims[1] != all[1]->dims[1])
        nc_fatal("nc_relpos_attention_step: q (H*dk, B) and kv_cache (H*dk+H*dv, B, T) expected");
    const size_t B = all[1]->dims[1], T = all[1]->dims[2];
    // the shape checks of the whole-segment op, on a view of q as one of T positions
    size_t qd[3] = { all[0]->dims[0], B, T };
    NCTensor qshape = *all[0];
    qshape.n_dims = 3;
    memcpy(qshape.dims, qd, sizeof(qd));
    AttnDims a = attn_dims(&qshape, all[1], all[2], all[3], all[4], n_head, d_key);
    size_t od[2] = { (size_t)a.H * a.dv, B };
    NCTensor *y = new_f32(all[0], 2, od);
    int rc = nchip_relpos_attn_fwd_step(m->stream, nc_f32(all[0]), (int64_t)all[0]->dims[0],
                                        nc_f32(all[1]), all[2] ? nc_f32(all[2]) : nullptr, (int64_t)all[1]->dims[0],
                                        all[3] ? nc_f32(all[3]) : nullptr, all[4] ? nc_f32(all[4]) : nullptr,
                                        nc_f32(y), (int64_t)od[0], a.H, a.dk, a.dv, a.B, a.T, a.M, a.d_pos,
                                        attn_len, b_r_scale, t);
    if (rc) nc_fatal("nc_relpos_attention_step: kernel rejected the shapes");
    m->launches++;
    for (int i = 0; i < 5; i++) nc_free_tensor(all[i]);
    return y;
}

static void attn_bw(NCNode *nd, NCTensor *g, NCTensor **ga)
{
    NCTensor *q = nd->saved[0], *kv = nd->saved[1], *kvm = nd->saved[2], *w_r = nd->saved[3];
    NCTensor *probs = nd->saved[4];
    NCContext *m = nc_ctx(g);
    AttnDims a = attn_dims(q, kv, kvm, w_r, nullptr, nd->ia[0], nd->ia[1]);
    NCTensor *gc = nc_contig(nc_dup_tensor(g));
    NCTensor *dq = nc_alloc_like(q), *dkv = nc_alloc_like(kv);
    NCTensor *dkvm = kvm ? nc_alloc_like(kvm) : nullptr;
    NCTensor *dwr = w_r ? nc_alloc_like(w_r) : nullptr;
    size_t bd[2] = { (size_t)a.K, (size_t)a.H };
    NCTensor *dbr = nd->ia[4] ? new_f32(q, 2, bd) : nullptr;
    size_t cap;
    float *scratch = nc_tmp_f32(m, nchip_relpos_attn_bwd_scratch(a.H, a.dk, a.B, a.T, a.M, a.d_pos), &cap);
    // per-stream partials may be summed late when the gradients go straight to parameters:
    // used once (one sum), or shared by several attention nodes (two-level sum)
    const bool once = (!dwr || nc_can_defer_sum(m, nd->parents[3])) && (!dbr || nc_can_defer_sum(m, nd->parents[4]));
    const bool shared = (!dwr || nc_can_defer_shared_sum(m, nd->parents[3])) &&
                        (!dbr || nc_can_defer_shared_sum(m, nd->parents[4]));
    const int keep = (dwr || dbr) && (once || shared);
    int rc;
    if (probs->type == NC_TYPE_U16) {
        // the forward ran on the bf16 matrix cores: so does the backward, from the same copies
        const uint16_t *q16 = nc_shadow_of(m, q), *kv16 = nc_shadow_of(m, kv), *kvm16 = kvm ? nc_shadow_of(m, kvm) : nullptr;
        const uint16_t *w16 = w_r ? nc_shadow_of(m, w_r) : nullptr, *go16 = nc_shadow_of(m, gc);
        if (!q16 || !kv16 || (kvm && !kvm16) || (w_r && !w16) || !go16)
            nc_fatal("nc_relpos_attention backward: an operand has no bf16 copy");
        const int64_t n_w = dwr ? (int64_t)nc_numel(dwr) : 0, n_b = dbr ? (int64_t)nc_numel(dbr) : 0;
        Bf16AttnBwdArgs g;
        g.q = q16; g.kv = kv16; g.kvm = kvm16; g.w_r = w16; g.probs = (const uint16_t *)nc_data(probs); g.dout = go16;
        g.dq = nc_f32(dq); g.dkv = nc_f32(dkv); g.dkvm = dkvm ? nc_f32(dkvm) : nullptr;
        g.dwp = dwr ? scratch : nullptr; g.dbp = dbr ? scratch + n_w * a.B : nullptr;
        g.dq16 = nc_shadow_for_write(m, dq); g.dkv16 = nc_shadow_for_write(m, dkv);
        g.dkvm16 = dkvm ? nc_shadow_for_write(m, dkvm) : nullptr;
        g.ldq = (int64_t)q->dims[0]; g.ldkv = (int64_t)kv->dims[0]; g.ldo = (int64_t)gc->dims[0];
        g.H = a.H; g.B = a.B; g.T = a.T; g.M = a.M; g.K = a.K; g.d_pos = a.d_pos; g.attn_len = nd->ia[2];
        g.b_r_scale = nd->fa[0]; g.scale = 1.0f / sqrtf((float)a.dk);
        if (k_attn_bf16_bwd(m->stream, g)) nc_fatal("nc_relpos_attention backward: bf16 kernel launch failed");
        m->launches++;
        rc = keep ? 1 : 0;
        if (!keep && (dwr || dbr)) {
            if (k_attn_param_grad_reduce(m->stream, scratch, dwr ? nc_f32(dwr) : nullptr, n_w, scratch + n_w * a.B,
                                         dbr ? nc_f32(dbr) : nullptr, n_b, a.B))
                nc_fatal("nc_relpos_attention backward: partial sums failed");
            m->launches++;
        }
    } else
    rc = nchip_relpos_attn_bwd(m->stream, nc_f32(q), (int64_t)q->dims[0], nc_f32(kv),
                                   kvm ? nc_f32(kvm) : nullptr, (int64_t)kv->dims[0],
                                   w_r ? nc_f32(w_r) : nullptr, nc_f32(probs), nc_f32(gc),
                                   (int64_t)gc->dims[0], nc_f32(dq), nc_f32(dkv),
                                   dkvm ? nc_f32(dkvm) : nullptr, dwr ? nc_f32(dwr) : nullptr,
                                   dbr ? nc_f32(dbr) : nullptr, a.H, a.dk, a.dv, a.B, a.T, a.M, a.d_pos,
                                   nd->ia[2], nd->fa[0], 0, scratch, keep);
    if (rc < 0) nc_fatal("nc_relpos_attention backward failed");
    if (rc == 1) {
        // per-stream dw_r / db_r partials stay in scratch until the batched sum
        const int64_t n_w = dwr ? (int64_t)nc_numel(dwr) : 0, n_b = dbr ? (int64_t)nc_numel(dbr) : 0;
        if (once) {
            if (dwr) defer_sum(m, scratch, dwr, a.B, n_w, (int)n_w, nd->parents[3]);
            if (dbr) defer_sum(m, scratch + n_w * a.B, dbr, a.B, n_b, (int)n_b, nd->parents[4]);
        } else {
            if (dwr) { NCTensor *t = defer_shared_sum(m, scratch, dwr, a.B, n_w, nd->parents[3]); nc_free_tensor(dwr); dwr = t; }
            if (dbr) { NCTensor *t = defer_shared_sum(m, scratch + n_w * a.B, dbr, a.B, n_b, nd->parents[4]); nc_free_tensor(dbr); dbr = t; }
        }
        DeferredTmp dt = { scratch, cap };
        m->deferred_tmp.push_back(dt);
    } else {
        nc_tmp_free(m, scratch, cap);
    }
    if (probs->type != NC_TYPE_U16) m->launches += nchip_relpos_attn_last_launches();
    nc_free_tensor(gc);
    NCTensor *out[5] = { dq, dkv, dkvm, dwr, dbr };
    for (int i = 0; i < 5; i++) {
        if (out[i] && nd->parents[i]) ga[i] = out[i];
        else nc_free_tensor(out[i]);
    }
}

// ---- integer CDF path (nc_ext.h) --------------------------------------------
extern "C" NCTensor *nc_soft_max_cdf16(NCTensor *logits)
{
    logits = nc_contig(logits);
    need_f32(logits, "nc_soft_max_cdf16");
    size_t v = logits->dims[0];
    NCTensor *y = nc_alloc(logits->dev, NC_TYPE_U16, logits->n_dims, logits->dims, false);
    if (nchip_softmax_cdf16(nc_stream(logits), nc_f32(logits), (uint16_t *)nc_data(y), (int)v,
                            (int64_t)(nc_numel(logits) / v)))
        nc_fatal("nc_soft_max_cdf16 failed");
    LAUNCHED(logits);
    nc_free_tensor(logits);
    return y;
}

// nc_ext.h: the same CDFs written by the kernel straight into pinned host memory (the rows
// of a decoder timestep are 16 KB: a copy of their own costs a launch and its latency).  The
// tensor is on the host device; its contents are there after the next nc_synchronize.
extern "C" NCTensor *nc_soft_max_cdf16_to_host(NCTensor *logits)
{
    logits = nc_contig(logits);
    need_f32(logits, "nc_soft_max_cdf16_to_host");
    NCContext *m = nc_ctx(logits);
    size_t v = logits->dims[0];
    NCTensor *y = nc_alloc(&m->cpu, NC_TYPE_U16, logits->n_dims, logits->dims, false);
    if (nchip_softmax_cdf16(m->stream, nc_f32(logits), (uint16_t *)nc_data(y), (int)v, (int64_t)(nc_numel(logits) / v)))
        nc_fatal("nc_soft_max_cdf16_to_host failed");
    m->launches++;
    nc_mark_in_flight(y); // freed before the next wait, the buffer must not serve another tensor yet
    nc_free_tensor(logits);
    return y;
}

extern "C" NCTensor *nc_soft_max_int(NCTensor *x, float mult) // libnc.h:383-384
{
    x = nc_contig(x);
    need_f32(x, "nc_soft_max_int");
    size_t v = x->dims[0];
    NCTensor *y = nc_alloc(x->dev, NC_TYPE_I32, x->n_dims, x->dims, false);
    if (nchip_softmax_int(nc_stream(x), nc_f32(x), (int32_t *)nc_data(y), (int)v, (int64_t)(nc_numel(x) / v), mult))
        nc_fatal("nc_soft_max_int failed");
    LAUNCHED(x);
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_cdf_lookup(NCTensor *cdf, NCTensor *targets)
{
    cdf = nc_contig(cdf); targets = nc_contig(targets);
    need_dev(cdf, "nc_cdf_lookup"); need_dev(targets, "nc_cdf_lookup");
    if (cdf->type != NC_TYPE_U16 || targets->type != NC_TYPE_U16) nc_fatal("nc_cdf_lookup: u16 tensors expected");
    size_t v = cdf->dims[0], cols = nc_numel(cdf) / v, mm = targets->dims[0];
    if (nc_numel(targets) != mm * cols) nc_fatal("nc_cdf_lookup: targets must be (m, n) for a (V, n) cdf");
    NCTensor *y = nc_alloc_like(targets);
    if (nchip_cdf_lookup(nc_stream(cdf), (const uint16_t *)nc_data(cdf), (const uint16_t *)nc_data(targets),
                         (uint16_t *)nc_data(y), (int)v, (int64_t)mm, (int64_t)cols))
        nc_fatal("nc_cdf_lookup failed");
    LAUNCHED(cdf);
    nc_free_tensor(cdf); nc_free_tensor(targets);
    return y;
}

static int cdf_path_levels(size_t v)
{
    int levels = 1;
    while (((size_t)1 << levels) < v) levels++;
    return levels;
}

extern "C" NCTensor *nc_cdf_path(NCTensor *cdf, NCTensor *symbols)
{
    cdf = nc_contig(cdf); symbols = nc_contig(symbols);
    need_dev(cdf, "nc_cdf_path"); need_dev(symbols, "nc_cdf_path");
    if (cdf->type != NC_TYPE_U16 || symbols->type != NC_TYPE_I32) nc_fatal("nc_cdf_path: a u16 cdf and i32 symbols expected");
    size_t v = cdf->dims[0], cols = v ? nc_numel(cdf) / v : 0;
    if (v == 0 || nc_numel(symbols) != cols) nc_fatal("nc_cdf_path: one symbol per column of the cdf expected");
    size_t dims[2] = { (size_t)cdf_path_levels(v), cols };
    NCTensor *y = nc_alloc(cdf->dev, NC_TYPE_U16, 2, dims, false);
    if (nchip_cdf_path(nc_stream(cdf), (const uint16_t *)nc_data(cdf), (const int32_t *)nc_data(symbols),
                       (uint16_t *)nc_data(y), (int)v, (int64_t)cols, (int)dims[0]))
        nc_fatal("nc_cdf_path failed");
    LAUNCHED(cdf);
    nc_free_tensor(cdf); nc_free_tensor(symbols);
    return y;
}

static NCTensor *soft_max_cdf16_path(NCTensor *logits, NCTensor *symbols, bool to_host);
extern "C" NCTensor *nc_soft_max_cdf16_path(NCTensor *logits, NCTensor *symbols) { return soft_max_cdf16_path(logits, symbols, false); }
extern "C" NCTensor *nc_soft_max_cdf16_path_to_host(NCTensor *logits, NCTensor *symbols) { return soft_max_cdf16_path(logits, symbols, true); }

static NCTensor *soft_max_cdf16_path(NCTensor *logits, NCTensor *symbols, bool to_host)
{
    logits = nc_contig(logits); symbols = nc_contig(symbols);
    need_dev(logits, "nc_soft_max_cdf16_path"); need_dev(symbols, "nc_soft_max_cdf16_path");
    if (logits->type != NC_TYPE_F32 || symbols->type != NC_TYPE_I32) nc_fatal("nc_soft_max_cdf16_path: f32 logits and i32 symbols expected");
    size_t v = logits->dims[0], cols = v ? nc_numel(logits) / v : 0;
    if (v == 0 || v > 65535) nc_fatal("nc_soft_max_cdf16_path: 1..65535 symbols expected");
    if (nc_numel(symbols) != cols) nc_fatal("nc_soft_max_cdf16_path: one symbol per column of the logits expected");
    size_t dims[2] = { (size_t)cdf_path_levels(v), cols };
    NCTensor *y = nc_alloc(to_host ? &nc_ctx(logits)->cpu : logits->dev, NC_TYPE_U16, 2, dims, false);
    if (nchip_softmax_cdf16_path(nc_stream(logits), nc_f32(logits), (const int32_t *)nc_data(symbols),
                                 (uint16_t *)nc_data(y), (int)v, (int64_t)cols, (int)dims[0]))
        nc_fatal("nc_soft_max_cdf16_path failed");
    LAUNCHED(logits);
    if (to_host) nc_mark_in_flight(y); // freed before the next wait, the buffer must not serve another tensor yet
    nc_free_tensor(logits); nc_free_tensor(symbols);
    return y;
}

// same arithmetic as the device exponential of k_cdf.hip, for host callers
extern "C" float nc_exp_det(float x)
{
    const float log2e = 0x1.715476p+0f, ln2_hi = 0x1.63p-1f, ln2_lo = -0x1.bd0106p-13f;
    float n = rintf(x * log2e);
    float r = fmaf(-n, ln2_hi, x);
    r = fmaf(-n, ln2_lo, r);
    float p = 0x1.6c16c2p-10f;
    p = fmaf(p, r, 0x1.111112p-7f);
    p = fmaf(p, r, 0x1.555556p-5f);
    p = fmaf(p, r, 0x1.555556p-3f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    union { float f; uint32_t u; } v = { p };
    v.u += (uint32_t)((int32_t)n * (1 << 23));
    return v.f;
}

static void flush_deferred_gemms(NCContext *m)
{
    if (m->deferred.empty()) return;
    std::vector<NchipGemmProblem> tab;
    int tiles = 0;
    double flops = 0.0;
    // longest reductions first: their tiles run longest and would otherwise
    // form the tail of the launch
    std::stable_sort(m->deferred.begin(), m->deferred.end(), [](const DeferredGemm &x, const DeferredGemm &y) {
        return x.k + (x.a2 ? x.k2 : 0) > y.k + (y.a2 ? y.k2 : 0);
    });
    // bf16 mode: when every problem fits the unguarded loaders, the operands are read from
    // their bf16 shadows (which the forward and input-gradient products of the same tensors
    // have left behind, or one cast each makes now)
    bool from_shadows = m->matmul_bf16 != 0 && !(getenv("NCHIP_BF16_SHADOWS") && atoi(getenv("NCHIP_BF16_SHADOWS")) == 0);
    for (const DeferredGemm &d : m->deferred)
        if (d.m % 128 || d.n % 128 || d.k % 64 || (d.a2 && d.k2 % 64) || d.k < 64) from_shadows = false;
    std::vector<const uint16_t *> sh;
    if (from_shadows) {
        for (const DeferredGemm &d : m->deferred) {
            const NCTensor *ops[4] = { d.a, d.b, d.a2, d.b2 };
            for (const NCTensor *t : ops) {
                const uint16_t *q = t ? nc_shadow_of(m, t) : nullptr;
                if (t && !q) from_shadows = false;
                sh.push_back(q);
            }
        }
    }
    size_t di = 0;
    for (DeferredGemm &d : m->deferred) {
        NchipGemmProblem p;
        if (from_shadows) {
            p.A = (const float *)sh[4 * di]; p.B = (const float *)sh[4 * di + 1]; p.C = nc_f32(d.c);
            p.A2 = (const float *)sh[4 * di + 2]; p.B2 = (const float *)sh[4 * di + 3];
        } else {
            p.A = nc_f32(d.a); p.B = nc_f32(d.b); p.C = nc_f32(d.c);
            p.A2 = d.a2 ? nc_f32(d.a2) : nullptr; p.B2 = d.b2 ? nc_f32(d.b2) : nullptr;
        }
        di++;
        nc_shadow_invalidate(d.c);
        p.m = d.m; p.n = d.n; p.k = d.k; p.k2 = d.a2 ? d.k2 : 0;
        flops += 2.0 * d.m * d.n * (double)(d.k + p.k2);
        p.lda = d.m; p.ldb = d.n; p.ldc = d.m;
        p.tile_start = tiles; p.alpha = d.alpha;
        tiles += nchip_gemm_grouped_tiles(d.m, d.n);
        tab.push_back(p);
    }
    size_t bytes = tab.size() * sizeof(NchipGemmProblem), hcap, dcap;
    void *host = m->host_pool.get(bytes, &hcap);
    void *dev = m->dev_pool.get(bytes, &dcap);
    memcpy(host, tab.data(), bytes);
    hip_check(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, m->stream), "hipMemcpyAsync gemm table");
    if (nchip_gemm_grouped(m->stream, 0, 1, (const NchipGemmProblem *)dev, (int)tab.size(), tiles,
                           from_shadows ? 2 : m->matmul_bf16, flops))
        nc_fatal("grouped weight-gradient GEMM failed");
    m->launches++;
    // pinned staging is recycled one flush later, after a wait for the stream
    nc_staging_retire(m, m->grp_staging, m->grp_staging_cap, m->grp_staging_stamp);
    m->grp_staging = host; m->grp_staging_cap = hcap; m->grp_staging_stamp = m->sync_count;
    m->dev_pool.put(dev, dcap);
    for (DeferredGemm &d : m->deferred) {
        nc_free_tensor(d.a); nc_free_tensor(d.b); nc_free_tensor(d.c);
        nc_free_tensor(d.a2); nc_free_tensor(d.b2);
    }
    m->deferred.clear();
}

// one launch over a table of row sums; the pinned copy of the table is retired one launch later
static void launch_row_sums(NCContext *m, const std::vector<KReduceRowsEntry> &tab, int max_n)
{
    size_t bytes = tab.size() * sizeof(KReduceRowsEntry), hcap, dcap;
    void *host = m->host_pool.get(bytes, &hcap);
    void *dev = m->dev_pool.get(bytes, &dcap);
    memcpy(host, tab.data(), bytes);
    hip_check(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, m->stream), "hipMemcpyAsync sum table");
    k_reduce_rows_multi(m->stream, (const KReduceRowsEntry *)dev, (int)tab.size(), max_n);
    m->launches++;
    nc_staging_retire(m, m->red_staging, m->red_staging_cap, m->red_staging_stamp);
    m->red_staging = host; m->red_staging_cap = hcap; m->red_staging_stamp = m->sync_count;
    m->dev_pool.put(dev, dcap);
}

static void flush_deferred_sums(NCContext *m)
{
    if (m->deferred_red.empty()) return;
    std::vector<KReduceRowsEntry> tab;
    int max_n = 0;
    for (DeferredReduce &d : m->deferred_red) {
        KReduceRowsEntry e;
        e.src = d.src; e.dst = d.dst; e.stride = d.stride; e.rows = d.rows; e.n = d.n;
        if (d.n > max_n) max_n = d.n;
        tab.push_back(e);
    }
    launch_row_sums(m, tab, max_n);
    if (!m->deferred_shared.empty()) {
        // second level: the rows of each shared parameter's stage (one per use that was
        // reached, in that order) into its gradient tensor
        tab.clear();
        max_n = 0;
        for (DeferredShared &d : m->deferred_shared) {
            KReduceRowsEntry e;
            e.src = d.stage; e.dst = nc_f32(d.dst); e.stride = d.n; e.rows = d.next; e.n = d.n;
            if (d.n > max_n) max_n = d.n;
            tab.push_back(e);
        }
        launch_row_sums(m, tab, max_n);
        for (DeferredShared &d : m->deferred_shared) { nc_tmp_free(m, d.stage, d.cap); nc_free_tensor(d.dst); }
        m->deferred_shared.clear();
    }
    for (DeferredTmp &t : m->deferred_tmp) nc_tmp_free(m, t.ptr, t.cap);
    for (NCTensor *t : m->deferred_keep) nc_free_tensor(t);
    m->deferred_red.clear(); m->deferred_tmp.clear(); m->deferred_keep.clear();
}

// Runs every postponed weight-gradient GEMM in one grouped launch and every
// postponed sum of partial rows in another.  The gradient tensors were handed
// to the parameter callback earlier, so with nc_set_deferred_weight_grad()
// enabled they hold valid data only once nc_backward() has returned.
void nc_flush_deferred(NCContext *m)
{
    flush_deferred_gemms(m);
    flush_deferred_sums(m);
}

bool nc_has_deferred(const NCContext *m, const NCNode *param)
{
    for (const DeferredGemm &e : m->deferred)
        if (e.param == param) return true;
    for (const DeferredReduce &e : m->deferred_red)
        if (e.param == param) return true;
    for (const DeferredShared &e : m->deferred_shared)
        if (e.param == param) return true;
    return false;
}

// a gradient that goes straight to a parameter used once may be finished late
bool nc_can_defer_sum(const NCContext *m, const NCNode *parent)
{
    return m->defer_wgrad && parent && parent->op == OP_PARAM && parent->consumers == 1;
}

static void defer_sum(NCContext *m, const float *src, NCTensor *dst, int rows, int64_t stride, int n,
                      const NCNode *param)
{
    DeferredReduce d;
    d.src = src; d.dst = nc_f32(dst); d.rows = rows; d.stride = stride; d.n = n; d.param = param;
    m->deferred_red.push_back(d);
    m->deferred_keep.push_back(nc_dup_tensor(dst));
}

// a gradient that goes straight to a parameter with several uses in this graph
bool nc_can_defer_shared_sum(const NCContext *m, const NCNode *parent)
{
    return m->defer_wgrad && parent && parent->op == OP_PARAM && parent->consumers > 1;
}

// One use's partial rows of a shared parameter.  Returns the tensor to hand to the graph: the
// gradient tensor itself at the first use, nullptr afterwards (the same tensor gets the total).
static NCTensor *defer_shared_sum(NCContext *m, const float *src, NCTensor *like, int rows, int64_t stride,
                                  const NCNode *param)
{
    const int n = (int)nc_numel(like);
    DeferredShared *d = nullptr;
    for (DeferredShared &e : m->deferred_shared)
        if (e.param == param) d = &e;
    NCTensor *ret = nullptr;
    if (!d) {
        DeferredShared e;
        e.param = param; e.n = n; e.uses = param->consumers; e.next = 0;
        e.stage = nc_tmp_f32(m, (size_t)e.uses * n, &e.cap);
        e.dst = nc_alloc_like(like);
        m->deferred_shared.push_back(e);
        d = &m->deferred_shared.back();
        ret = nc_dup_tensor(d->dst);
    }
    if (d->n != n || d->next >= d->uses) nc_fatal("shared gradient sum: unexpected use of a parameter");
    DeferredReduce r;
    r.src = src; r.dst = d->stage + (size_t)d->next * n; r.rows = rows; r.stride = stride; r.n = n; r.param = param;
    m->deferred_red.push_back(r);
    d->next++;
    return ret;
}

// ---- backward dispatch --------------------------------------------------------
void nc_node_backward(NCNode *nd, NCTensor *g, NCTensor **ga)
{
    NCContext *m = nc_ctx(g);
    hipStream_t st = m->stream;
    g = nc_contig(nc_dup_tensor(g));
    int64_t cnt = (int64_t)nc_numel(g);
    switch (nd->op) {
    case OP_ADD:
        for (int w = 0; w < 2; w++)
            if (nd->parents[w]) ga[w] = dev_unbroadcast(nc_dup_tensor(g), nd->arg_shape[w]);
        break;
    case OP_MUL:
        for (int w = 0; w < 2; w++)
            if (nd->parents[w]) ga[w] = dev_unbroadcast(dev_binary(KB_MUL, g, nd->saved[1 - w]), nd->arg_shape[w]);
        break;
    case OP_MASKED_FILL: {
        NCTensor *mask = nd->saved[0], *t = nc_alloc_like(g);
        // (mask ? 0 : g) is masked_fill of g with c = 0
        k_masked_fill(st, nc_f32(g), (const int8_t *)nc_data(mask), nc_f32(t), cnt, (int64_t)nc_numel(mask), 0.0f, nd->ia[0]);
        m->launches++;
        ga[0] = t;
        break;
    }
    case OP_UNARY: {
        NCTensor *t = nc_alloc_like(g);
        k_unary_bwd(st, nd->ia[0], nc_f32(nd->saved[0]), nc_f32(g), nc_f32(t), cnt);
        m->launches++;
        ga[0] = t;
        break;
    }
    case OP_GATED_SWISH: {
        NCTensor *dg = nc_alloc_like(g), *dx = nc_alloc_like(g);
        k_gated_swish_bwd(st, nc_f32(nd->saved[0]), nc_f32(nd->saved[1]), nc_f32(g), nc_f32(dg), nc_f32(dx), cnt, nd->fa[0]);
        m->launches++;
        if (nd->parents[0]) ga[0] = dg; else nc_free_tensor(dg);
        if (nd->parents[1]) ga[1] = dx; else nc_free_tensor(dx);
        break;
    }
    case OP_LSTM_CLAMPED: {
        NCTensor *t[4];
        for (int i = 0; i < 4; i++) t[i] = nc_alloc_like(g);
        k_lstm_clamped_bwd(st, nc_f32(nd->saved[0]), nc_f32(nd->saved[1]), nc_f32(nd->saved[2]), nc_f32(nd->saved[3]),
                           nc_f32(g), nc_f32(t[0]), nc_f32(t[1]), nc_f32(t[2]), nc_f32(t[3]), cnt);
        m->launches++;
        for (int i = 0; i < 4; i++)
            if (nd->parents[i]) ga[i] = t[i]; else nc_free_tensor(t[i]);
        break;
    }
    case OP_LERP: {
        NCTensor *t[3];
        for (int i = 0; i < 3; i++) t[i] = nc_alloc_like(g);
        k_lerp_bwd(st, nc_f32(nd->saved[0]), nc_f32(nd->saved[1]), nc_f32(nd->saved[2]), nc_f32(g),
                   nc_f32(t[0]), nc_f32(t[1]), nc_f32(t[2]), cnt);
        m->launches++;
        for (int i = 0; i < 3; i++)
            if (nd->parents[i]) ga[i] = t[i]; else nc_free_tensor(t[i]);
        break;
    }
    case OP_RESHAPE:
        ga[0] = nc_reshape_view(nc_dup_tensor(g), nd->arg_shape[0].nd, nd->arg_shape[0].d);
        break;
    case OP_REPEAT:
        ga[0] = dev_unbroadcast(nc_dup_tensor(g), nd->arg_shape[0]);
        break;
    case OP_REDUCE_SUM:
        if (nd->parents[0]) ga[0] = nc_dup_tensor(g);
        if (nd->parents[1])
            ga[1] = repeat_raw(g, nd->arg_shape[1].nd - g->n_dims, nd->arg_shape[1].d + g->n_dims);
        break;
    case OP_SUM: {
        // broadcast the scalar gradient: 0-stride source copy
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, nd->arg_shape[0].nd, nd->arg_shape[0].d, false);
        NCTensor *v = nc_view(g);
        v->n_dims = t->n_dims;
        for (int i = 0; i < t->n_dims; i++) { v->dims[i] = t->dims[i]; v->strides[i] = 0; }
        nc_copy_any(t, v);
        nc_free_tensor(v);
        ga[0] = t;
        break;
    }
    case OP_SLICE: {
        NCTensor *t = nc_alloc(g->dev, g->type, nd->arg_shape[0].nd, nd->arg_shape[0].d, true);
        NCTensor *v = nc_slice_alias(t, nd->ia[0], (size_t)nd->ia[1], (size_t)nd->ia[1] + g->dims[nd->ia[0]]);
        nc_copy_any(v, g);
        nc_free_tensor(v);
        ga[0] = t;
        break;
    }
    case OP_CONCAT: case OP_CONCAT_NODE: {
        size_t pos = 0;
        for (int i = 0; i < nd->n_args; i++) {
            if (nd->parents[i]) {
                NCTensor *v = nc_slice_alias(g, nd->ia[0], pos, pos + nd->sizes[i]);
                ga[i] = nc_alloc(g->dev, g->type, v->n_dims, v->dims, false);
                nc_copy_any(ga[i], v);
                nc_free_tensor(v);
            }
            pos += nd->sizes[i];
        }
        break;
    }
    case OP_PAD: {
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, nd->arg_shape[0].nd, nd->arg_shape[0].d, false);
        int64_t n_in = (int64_t)nd->arg_shape[0].d[0];
        k_pad_bwd(st, nc_f32(g), nc_f32(t), n_in, (int64_t)nc_numel(t) / n_in, nd->ia[0], nd->ia[1], nd->ia[2], nd->ia[3]);
        m->launches++;
        ga[0] = t;
        break;
    }
    case OP_PERMUTE: {
        int inv[NC_N_DIMS_MAX];
        for (int i = 0; i < g->n_dims; i++) inv[nd->ia[i]] = i;
        ga[0] = permute_raw(g, g->n_dims, inv);
        break;
    }
    case OP_REL_SHIFT: {
        NCTensor *t = nc_alloc_like(g);
        k_rel_shift(st, nc_f32(g), nc_f32(t), (int64_t)g->dims[0], (int64_t)g->dims[1],
                    cnt / (int64_t)(g->dims[0] * g->dims[1]), nd->ia[0], nd->ia[1], 1);
        m->launches++;
        ga[0] = t;
        break;
    }
    case OP_MATMUL:
        matmul_bw(nd, g, ga, 0, 1);
        if (nd->parents[2]) ga[2] = nc_dup_tensor(g);
        break;
    case OP_LINEAR: {
        if (nd->n_args > 3 && nd->parents[3]) ga[3] = nc_dup_tensor(g); // residual input
        NCTensor *gz = nc_dup_tensor(g);
        const bool already = nd->ia[5] != 0; // the producer of g applied act'(pre) in its epilogue
        nd->ia[5] = 0;
        if (nd->ia[3] != NC_ACT_NONE && !already) {
            NCTensor *t = nc_alloc_like(g);
            k_unary_bwd(st, nd->ia[3] == NC_ACT_GELU ? KU_GELU : KU_RELU, nc_f32(nd->saved[2]), nc_f32(g), nc_f32(t), cnt);
            m->launches++;
            nc_free_tensor(gz);
            gz = t;
        }
        matmul_bw(nd, gz, ga, 0, 1);
        if (nd->parents[2] && nd->grad_rowsum && (already || nd->ia[3] == NC_ACT_NONE)) {
            // the kernel that produced gz left its partial row sums: they join the batched sum
            size_t nb = nd->saved[0]->dims[0];
            NCTensor *dbias = nc_alloc(g->dev, NC_TYPE_F32, 1, &nb, false);
            defer_sum(m, nd->grad_rowsum, dbias, nd->grad_rowsum_rows, (int64_t)nb, (int)nb, nd->parents[2]);
            DeferredTmp dt = { nd->grad_rowsum, nd->grad_rowsum_cap };
            m->deferred_tmp.push_back(dt);
            nd->grad_rowsum = nullptr;
            ga[2] = dbias;
        } else if (nd->parents[2]) {
            Shape bs;
            bs.nd = 1; bs.d[0] = nd->saved[0]->dims[0];
            ga[2] = dev_unbroadcast(nc_dup_tensor(gz), bs, nd->parents[2]);
        }
        if (nd->grad_rowsum) { nc_tmp_free(m, nd->grad_rowsum, nd->grad_rowsum_cap); nd->grad_rowsum = nullptr; }
        nc_free_tensor(gz);
        break;
    }
    case OP_GET_COL: {
        NCTensor *idx = nd->saved[0];
        NCTensor *t = nc_alloc(g->dev, NC_TYPE_F32, nd->arg_shape[0].nd, nd->arg_shape[0].d, false);
        if (nchip_add_col(st, nc_f32(g), (const int32_t *)nc_data(idx), nc_f32(t), (int)t->dims[0], (int)t->dims[1],
                          (int64_t)nc_numel(idx)))
            nc_fatal("get_col backward failed");
        m->launches++;
        ga[0] = t;
        break;
    }
    case OP_SOFT_MAX: {
        NCTensor *y = nd->saved[0], *t = nc_alloc_like(g);
        int v = (int)y->dims[0];
        if (nchip_softmax_bwd(st, nc_f32(y), nc_f32(g), nc_f32(t), v, cnt / v)) nc_fatal("softmax backward failed");
        m->launches++;
        ga[0] = t;
        break;
    }
    case OP_INDEXED_LOG: {
        NCTensor *p = nd->saved[0], *idx = nd->saved[1];
        NCTensor *t = nc_alloc_like(p);
        int v = (int)p->dims[0];
        if (nchip_nll_bwd(st, nc_f32(p), (const int32_t *)nc_data(idx), nc_f32(g), nc_f32(t), v,
                          (int64_t)nc_numel(p) / v, nd->ia[0]))
            nc_fatal("indexed_log backward failed");
        m->launches++;
        ga[0] = t;
        break;
    }
    case OP_NORM: {
        NCTensor *xhat = nd->saved[0], *rstd = nd->saved[1], *w = nd->saved[2];
        int d = (int)xhat->dims[0];
        int64_t cols = (int64_t)nc_numel(xhat) / d;
        NCTensor *dx = nd->parents[0] ? nc_alloc_like(xhat) : nullptr;
        size_t dd = (size_t)d, cap = 0;
        NCTensor *dw = (w && nd->parents[1]) ? nc_alloc(g->dev, NC_TYPE_F32, 1, &dd, false) : nullptr;
        NCTensor *db = (w && nd->parents[2]) ? nc_alloc(g->dev, NC_TYPE_F32, 1, &dd, false) : nullptr;
        float *partial = (dw || db) ? nc_tmp_f32(m, (size_t)nchip_norm_bwd_partial_rows(cols) * 2 * d, &cap) : nullptr;
        const float *prev = dx ? nc_bw_addend(m, 0, nc_numel(dx)) : nullptr;
        // dw / db that go straight to once-used parameters: their sums over the
        // partial rows join the batched sum at the end of nc_backward
        const bool late = dw && db && nc_can_defer_sum(m, nd->parents[1]) && nc_can_defer_sum(m, nd->parents[2]);
        // the input came straight out of a linear layer with a bias (and feeds nothing else):
        // that bias gradient is the row sum of dx, whose partial sums this kernel can leave
        NCNode *pl = nd->parents[0];
        float *dxp = nullptr;
        size_t dxp_cap = 0;
        if (dx && pl && pl->op == OP_LINEAR && pl->ia[3] == NC_ACT_NONE && pl->consumers == 1 && !pl->grad_rowsum &&
            pl->parents.size() > 2 && pl->parents[2] && nc_can_defer_sum(m, pl->parents[2]) &&
            nchip_norm_bwd_has_dx_rowsum(d) && pl->saved[0] && (int)pl->saved[0]->dims[0] == d)
            dxp = nc_tmp_f32(m, (size_t)nchip_norm_bwd_rows(d, cols) * d, &dxp_cap);
        // (bf16 products: dx is the operand of the products behind the layer that fed this norm)
        uint16_t *dx16 = (dx && m->matmul_bf16) ? nc_shadow_for_write(m, dx) : nullptr;
        if (nchip_norm_bwd_bf16copy(st, nc_f32(g), nc_f32(xhat), nc_f32(rstd), w ? nc_f32(w) : nullptr,
                                    dx ? nc_f32(dx) : nullptr, prev, (dw && !late) ? nc_f32(dw) : nullptr,
                                    (db && !late) ? nc_f32(db) : nullptr, partial, d, cols, nd->ia[0], dxp, dx16))
            nc_fatal("layer norm backward failed");
        if (dxp) {
            pl->grad_rowsum = dxp; pl->grad_rowsum_cap = dxp_cap; pl->grad_rowsum_rows = nchip_norm_bwd_rows(d, cols);
        }
        if (late) {
            const int rows = nchip_norm_bwd_rows(d, cols);
            defer_sum(m, partial, dw, rows, 2 * (int64_t)d, d, nd->parents[1]);
            defer_sum(m, partial + d, db, rows, 2 * (int64_t)d, d, nd->parents[2]);
            DeferredTmp dt = { partial, cap };
            m->deferred_tmp.push_back(dt);
            m->launches += 1;
        } else {
            if (partial) nc_tmp_free(m, partial, cap);
            m->launches += (dw || db) ? 2 : 1;
        }
        ga[0] = dx; ga[1] = dw; ga[2] = db;
        break;
    }
    case OP_ATTN:
        attn_bw(nd, g, ga);
        break;
    default:
        nc_fatal("backward: op %d not handled", nd->op);
    }
    nc_free_tensor(g);
}
