/*
 * libnc_ref core: context, tensors, views, copies, RNG, parameters, optimiser.
 *
 * TEST INFRASTRUCTURE ONLY (CPU checker + timed CPU baseline).  The reference
 * ships libnc as a header only (libnc.h); what each function must do is taken
 * from that header's comments and from how nncp.c uses it (cited per function).
 * Behaviour the header does not fix is defined here and marked "build-defined".
 * What each such function computes is pinned by tests (the random fills against
 * an independent statement of Marsaglia's xorwow and the uniform law, the
 * optimisers against torch.optim in float64, vec_sum_f32 as a left-to-right
 * sum); that libnc's own choice is the same one cannot be known from the
 * header, so against libnc itself parity stays unpinned for:
 * nc_tensor_set_rnd_unif, nc_tensor_set_dropout (which generator and stream),
 * nc_sgd_opt_update (bias correction / clip semantics), vec_sum_f32 order.
 * nc_cmul (rotary position embedding) is not implemented on either side.
 */
#include <stdarg.h>
#include <stdio.h>
#include <omp.h>
#include <time.h>
#include "nc_ref_internal.h"

void nc_fatal(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    fprintf(stderr, "libnc_ref: ");
    vfprintf(stderr, fmt, ap);
    fprintf(stderr, "\n");
    va_end(ap);
    abort();
}

/* libnc.h:117-119 */
void *nc_malloc(size_t size)
{
    void *p = malloc(size ? size : 1);
    if (!p)
        nc_fatal("out of memory (%zu bytes)", size);
    return p;
}

void *nc_mallocz(size_t size)
{
    void *p = nc_malloc(size);
    memset(p, 0, size);
    return p;
}

void nc_free(void *ptr)
{
    free(ptr);
}

/* libnc.h:124-130; nncp.c:2770-2777 creates one context, one CPU device and
   optionally one accelerator device. */
NCContext *nc_context_init(int nb_threads)
{
    NCContext *m = nc_mallocz(sizeof(*m));
    m->nb_threads = nb_threads > 0 ? nb_threads : 1;
    omp_set_num_threads(m->nb_threads);
    m->cpu = nc_mallocz(sizeof(NCDevice));
    m->cpu->ctx = m;
    /* the bf16 operand emulation is one switch for the whole checker: a new context starts
       in fp32, as a context of the product does, whatever an earlier one left behind */
    nc_set_matmul_bf16(m, 0);
    return m;
}

void nc_context_end(NCContext *m)
{
    if (!m)
        return;
    nc_free(m->cpu);
    nc_free(m);
}

NCDevice *nc_new_cpu_device(NCContext *m) { return m->cpu; }
NCDevice *nc_new_cuda_device(NCContext *m, int device_index) { (void)device_index; return m->cpu; }
NCDevice *nc_new_device(NCContext *m, const char *name) { (void)name; return m->cpu; }
void nc_synchronize(NCDevice *d) { (void)d; }
/* libnc.h:14-67: the section timers (nanoseconds of wall clock); no marker ranges here */
int64_t prof_cycles[PROF_COUNT], prof_samples[PROF_COUNT], prof_ops[PROF_COUNT];
static int64_t prof_clock(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (int64_t)ts.tv_sec * 1000000000 + ts.tv_nsec;
}
void nc_prof_begin(int idx)
{
    if (idx >= 0 && idx < PROF_COUNT)
        prof_cycles[idx] -= prof_clock();
}
void nc_prof_finish(int idx, int n_ops)
{
    if (idx < 0 || idx >= PROF_COUNT)
        return;
    prof_cycles[idx] += prof_clock();
    prof_samples[idx]++;
    prof_ops[idx] += n_ops;
}
void nc_prof_dump(void)
{
    static const char *const names[PROF_COUNT] = { "EVAL", "GRAD", "SGD", "UPDATE", "WRITE_SYM", "PROBE", "TOTAL" };
    const char *on = getenv("NC_PROFILE");
    if (!on || !*on)
        return;
    for (int i = 0; i < PROF_COUNT; i++)
        if (prof_samples[i])
            fprintf(stderr, "%-10s %10lld samples %14.3f ms\n", names[i], (long long)prof_samples[i], prof_cycles[i] * 1e-6);
}
int nc_set_matmul_bf16(NCContext *m, int enable);
int64_t nc_get_launch_count(NCContext *m) { (void)m; return 0; }
void *nc_context_stream(NCContext *m) { (void)m; return NULL; }
int nc_set_deferred_weight_grad(NCContext *m, int enable) { (void)m; (void)enable; return 0; }
int nc_set_matmul_width_invariant(NCContext *m, int enable) { (void)m; (void)enable; return 0; }
int64_t nc_get_bf16_cast_count(NCContext *m) { (void)m; return 0; }
int nc_set_bf16_shadow_check(int enable) { (void)enable; return 0; }
int nc_set_bf16_copy_of_results(NCContext *m, int enable) { (void)m; (void)enable; return 0; }

size_t nc_type_size(NCTypeEnum t)
{
    switch (t) {
    case NC_TYPE_F32: case NC_TYPE_I32: case NC_TYPE_U32: return 4;
    case NC_TYPE_BF16: case NC_TYPE_F16: case NC_TYPE_I16: case NC_TYPE_U16: return 2;
    case NC_TYPE_I8: case NC_TYPE_U8: return 1;
    default: nc_fatal("unsupported tensor type %d", t);
    }
}

size_t nc_numel(const NCTensor *x)
{
    size_t n = 1;
    for (int i = 0; i < x->n_dims; i++)
        n *= x->dims[i];
    return n;
}

int nc_is_contig(const NCTensor *x)
{
    size_t s = 1;
    for (int i = 0; i < x->n_dims; i++) {
        if (x->dims[i] != 1 && x->strides[i] != s)
            return 0;
        s *= x->dims[i];
    }
    return 1;
}

NCTensor *nc_alloc(NCDevice *d, NCTypeEnum type, int n_dims, const size_t *dims, int zero)
{
    NCTensor *x = nc_mallocz(sizeof(*x));
    size_t n = 1;
    if (n_dims > NC_N_DIMS_MAX)
        nc_fatal("too many dimensions");
    x->ref = 1;
    x->dev = d;
    x->type = type;
    x->n_dims = n_dims;
    for (int i = 0; i < n_dims; i++) {
        x->dims[i] = dims[i];
        x->strides[i] = n;
        n *= dims[i];
    }
    x->buf = nc_mallocz(sizeof(*x->buf));
    x->buf->ref = 1;
    x->buf->size = n * nc_type_size(type);
    x->buf->data = zero ? nc_mallocz(x->buf->size + 64) : nc_malloc(x->buf->size + 64);
    return x;
}

NCTensor *nc_alloc_like(const NCTensor *x)
{
    return nc_alloc(x->dev, x->type, x->n_dims, x->dims, 0);
}

NCTensor *nc_view(const NCTensor *x)
{
    NCTensor *y = nc_mallocz(sizeof(*y));
    *y = *x;
    y->ref = 1;
    y->node = NULL;
    y->buf->ref++;
    return y;
}

float *nc_f32(const NCTensor *x)
{
    /* a 2-byte tensor read as floats would be read out of bounds: ops widen bf16 operands
       before they come here (nc_operand) */
    if (nc_type_size(x->type) != sizeof(float))
        nc_fatal("f32 access to a tensor of type %d", (int)x->type);
    return (float *)x->buf->data + x->off;
}

static void *elem_ptr(const NCTensor *x)
{
    return (uint8_t *)x->buf->data + x->off * nc_type_size(x->type);
}

/* libnc.h:153-171.  The plain constructors zero the data: nncp.c relies on it
   for b_r, b_q, the FF/out biases and ln_b (nncp.c:369-372, 275-276). */
NCTensor *nc_new_tensor(NCDevice *d, NCTypeEnum t, int n, const size_t *dims) { return nc_alloc(d, t, n, dims, 1); }
NCTensor *nc_new_tensor_nz(NCDevice *d, NCTypeEnum t, int n, const size_t *dims) { return nc_alloc(d, t, n, dims, 0); }
NCTensor *nc_new_tensor_from_tensor_nz(const NCTensor *x) { return nc_alloc_like(x); }
NCTensor *nc_new_scalar(NCDevice *d, NCTypeEnum t) { return nc_alloc(d, t, 0, NULL, 1); }
NCTensor *nc_new_tensor_1d(NCDevice *d, NCTypeEnum t, size_t n0) { size_t s[1] = { n0 }; return nc_alloc(d, t, 1, s, 1); }
NCTensor *nc_new_tensor_2d(NCDevice *d, NCTypeEnum t, size_t n0, size_t n1) { size_t s[2] = { n0, n1 }; return nc_alloc(d, t, 2, s, 1); }
NCTensor *nc_new_tensor_3d(NCDevice *d, NCTypeEnum t, size_t n0, size_t n1, size_t n2) { size_t s[3] = { n0, n1, n2 }; return nc_alloc(d, t, 3, s, 1); }
NCTensor *nc_new_tensor_4d(NCDevice *d, NCTypeEnum t, size_t n0, size_t n1, size_t n2, size_t n3) { size_t s[4] = { n0, n1, n2, n3 }; return nc_alloc(d, t, 4, s, 1); }

NCTensor *nc_new_f32(NCDevice *d, float val) /* libnc.h:278 */
{
    NCTensor *x = nc_new_scalar(d, NC_TYPE_F32);
    nc_f32(x)[0] = val;
    return x;
}

NCTensor *nc_tensor_set_name(NCTensor *x, const char *fmt, ...) { (void)fmt; return x; }

NCTensor *nc_dup_tensor(const NCTensor *x) /* libnc.h:173 */
{
    if (x)
        ((NCTensor *)x)->ref++;
    return (NCTensor *)x;
}

void nc_free_tensor(NCTensor *x) /* libnc.h:174; NULL is accepted (nncp.c:532-534) */
{
    if (!x)
        return;
    if (--x->ref > 0)
        return;
    nc_free_node(x->node);
    if (--x->buf->ref == 0) {
        free(x->buf->data);
        free(x->buf);
    }
    free(x);
}

NCNode *nc_get_node(NCTensor *x) { return x->node; }           /* libnc.h:180, borrowed */
NCTypeEnum nc_tensor_get_item_type(const NCTensor *x) { return x->type; }
NCDevice *nc_get_tensor_device(const NCTensor *x) { return x->dev; }

int nc_tensor_get_dims(const NCTensor *x, size_t *dims) /* libnc.h:189 */
{
    if (dims)
        for (int i = 0; i < x->n_dims; i++)
            dims[i] = x->dims[i];
    return x->n_dims;
}

/* libnc.h:183-185: base pointer and the element stride of axis 1
   (process_block reads one stream's V probabilities at output + stream*stride,
   nncp.c:3005-3013). */
void *nc_tensor_get_ptr(const NCTensor *x, size_t *pstride)
{
    if (pstride)
        *pstride = x->n_dims >= 2 ? x->strides[1] : (x->n_dims ? x->dims[0] : 1);
    return elem_ptr(x);
}

/* generic strided element copy with type conversion between F32/I32/I8/U16 */
static double load_elem(const NCTensor *x, size_t off)
{
    const uint8_t *p = (const uint8_t *)x->buf->data;
    switch (x->type) {
    case NC_TYPE_F32: return ((const float *)p)[x->off + off];
    case NC_TYPE_I32: return ((const int32_t *)p)[x->off + off];
    case NC_TYPE_I8: return ((const int8_t *)p)[x->off + off];
    case NC_TYPE_U16: return ((const uint16_t *)p)[x->off + off];
    case NC_TYPE_BF16: return nc_bf16_widen(((const uint16_t *)p)[x->off + off]);
    default: nc_fatal("load: unsupported type");
    }
}

static void store_elem(NCTensor *x, size_t off, double v)
{
    uint8_t *p = (uint8_t *)x->buf->data;
    switch (x->type) {
    case NC_TYPE_F32: ((float *)p)[x->off + off] = (float)v; break;
    case NC_TYPE_I32: ((int32_t *)p)[x->off + off] = (int32_t)v; break;
    case NC_TYPE_I8: ((int8_t *)p)[x->off + off] = (int8_t)v; break;
    case NC_TYPE_U16: ((uint16_t *)p)[x->off + off] = (uint16_t)v; break;
    case NC_TYPE_BF16: ((uint16_t *)p)[x->off + off] = nc_bf16_bits((float)v); break;
    default: nc_fatal("store: unsupported type");
    }
}

void nc_copy_strided(NCTensor *dst, const NCTensor *src)
{
    size_t n = nc_numel(dst), idx[NC_N_DIMS_MAX] = { 0 };
    if (nc_numel(src) != n || dst->n_dims != src->n_dims)
        nc_fatal("copy: shape mismatch");
    for (int i = 0; i < dst->n_dims; i++)
        if (dst->dims[i] != src->dims[i])
            nc_fatal("copy: shape mismatch on axis %d (%zu vs %zu)", i, dst->dims[i], src->dims[i]);
    if (n == 0)
        return;
    /* fast path: both F32 and axis 0 contiguous */
    size_t n0 = dst->n_dims ? dst->dims[0] : 1;
    int fast = dst->type == NC_TYPE_F32 && src->type == NC_TYPE_F32 &&
               (dst->n_dims == 0 || (dst->strides[0] == 1 && src->strides[0] == 1));
    size_t so = 0, dof = 0;
    for (size_t c = 0; c < n / n0; c++) {
        if (fast) {
            memcpy(nc_f32(dst) + dof, nc_f32(src) + so, n0 * sizeof(float));
        } else {
            for (size_t i = 0; i < n0; i++)
                store_elem(dst, dof + i * (dst->n_dims ? dst->strides[0] : 0),
                           load_elem(src, so + i * (src->n_dims ? src->strides[0] : 0)));
        }
        /* odometer over axes >= 1 */
        for (int a = 1; a < dst->n_dims; a++) {
            idx[a]++;
            so += src->strides[a];
            dof += dst->strides[a];
            if (idx[a] < dst->dims[a])
                break;
            so -= src->strides[a] * dst->dims[a];
            dof -= dst->strides[a] * dst->dims[a];
            idx[a] = 0;
        }
    }
}

NCTensor *nc_contig(NCTensor *x)
{
    NCTensor *y;
    if (nc_is_contig(x)) {
        /* normalise the strides of size-1 axes so raw indexing is safe */
        return x;
    }
    y = nc_alloc_like(x);
    nc_copy_strided(y, x);
    y->node = nc_dup_node(x->node);
    nc_free_tensor(x);
    return y;
}

/* libnc.h:218: element copy, shapes equal, both borrowed (nncp.c:655-657) */
void nc_tensor_copy(NCTensor *dst, NCTensor *src)
{
    nc_copy_strided(dst, src);
}

/* libnc.h:219-220: dst[.., dst_start:dst_end, ..] = src[.., src_start:.., ..]
   on 'axis'; overlapping self-copy towards lower indices is used by
   mem_update (nncp.c:1212). */
void nc_tensor_copy_slice(NCTensor *dst, NCTensor *src, int axis,
                          size_t dst_start, size_t dst_end, size_t src_start)
{
    NCTensor *d = nc_slice_alias(dst, axis, dst_start, dst_end);
    NCTensor *s = nc_slice_alias(src, axis, src_start, src_start + (dst_end - dst_start));
    if (dst->buf == src->buf) {
        NCTensor *tmp = nc_alloc_like(s);
        nc_copy_strided(tmp, s);
        nc_copy_strided(d, tmp);
        nc_free_tensor(tmp);
    } else {
        nc_copy_strided(d, s);
    }
    nc_free_tensor(d);
    nc_free_tensor(s);
}

void nc_tensor_set_zero(NCTensor *y) /* libnc.h:192 */
{
    if (nc_is_contig(y)) {
        memset(elem_ptr(y), 0, nc_numel(y) * nc_type_size(y->type));
    } else {
        NCTensor *z = nc_alloc(y->dev, y->type, y->n_dims, y->dims, 1);
        nc_copy_strided(y, z);
        nc_free_tensor(z);
    }
}

void nc_tensor_set_f32(NCTensor *y, float val) /* libnc.h:194 */
{
    size_t n = nc_numel(y);
    if (!nc_is_contig(y) || (y->type != NC_TYPE_F32 && y->type != NC_TYPE_BF16))
        nc_fatal("set_f32: contiguous f32 or bf16 tensor expected");
    for (size_t i = 0; i < n; i++)
        store_elem(y, i, val);
}

/* libnc.h:206: host-side single element write with conversion to the item
   type; used for the I8 masks and the I32 token inputs (nncp.c:361, 2998). */
void nc_set1_i32_2d(NCTensor *y, size_t i0, size_t i1, int32_t val)
{
    if (y->n_dims != 2 || i0 >= y->dims[0] || i1 >= y->dims[1])
        nc_fatal("set1_i32_2d: index out of range");
    store_elem(y, i0 * y->strides[0] + i1 * y->strides[1], val);
}

float nc_get_scalar_f32(const NCTensor *x) /* libnc.h:214 */
{
    if (nc_numel(x) != 1)
        nc_fatal("get_scalar: not a scalar");
    return (float)load_elem(x, 0);
}

/* libnc.h:226-228: single CPU device here, so both are identity moves that
   hand the consumed reference back. */
NCTensor *nc_tensor_to_device(NCTensor *x, NCDevice *d) { (void)d; return x; }
NCTensor *nc_tensor_to_cpu_device(NCTensor *x) { return nc_contig(x); }

/* libnc.h:177: any stable 32-bit hash; FNV-1a over the raw contiguous bytes */
uint32_t nc_tensor_get_hash(const NCTensor *x)
{
    NCTensor *c = nc_contig(nc_dup_tensor(x));
    const uint8_t *p = elem_ptr(c);
    size_t n = nc_numel(c) * nc_type_size(c->type);
    uint32_t h = 2166136261u;
    for (size_t i = 0; i < n; i++)
        h = (h ^ p[i]) * 16777619u;
    nc_free_tensor(c);
    return h;
}

/* ---- RNG (build-defined: xorwow, the generator the RNDState fields of
   libnc.h:584-589 suggest; the reference stream itself is not visible) ---- */
struct NCRNDState {
    uint32_t x, y, z, w, v, d;
};

static uint32_t xorwow(NCRNDState *s)
{
    uint32_t t = s->x ^ (s->x >> 2);
    s->x = s->y; s->y = s->z; s->z = s->w; s->w = s->v;
    s->v = (s->v ^ (s->v << 4)) ^ (t ^ (t << 1));
    s->d += 362437;
    return s->d + s->v;
}

NCRNDState *nc_rnd_init(NCDevice *d, uint32_t seed) /* libnc.h:195 */
{
    NCRNDState *s = nc_mallocz(sizeof(*s));
    (void)d;
    s->x = 123456789 ^ seed; s->y = 362436069; s->z = 521288629;
    s->w = 88675123; s->v = 5783321; s->d = 6615241 + seed * 2654435761u;
    for (int i = 0; i < 16; i++)
        xorwow(s);
    return s;
}

void nc_rnd_end(NCRNDState *s) { nc_free(s); }

/* libnc.h:197: uniform in [avg - range, avg + range) (half-width reading) */
void nc_tensor_set_rnd_unif(NCTensor *y, float avg, float range, NCRNDState *rs)
{
    size_t n = nc_numel(y);
    if (!nc_is_contig(y) || (y->type != NC_TYPE_F32 && y->type != NC_TYPE_BF16))
        nc_fatal("set_rnd_unif: contiguous f32 or bf16 tensor expected");
    for (size_t i = 0; i < n; i++) {
        float u = (float)(xorwow(rs) >> 8) * (1.0f / 16777216.0f); /* [0,1) */
        store_elem(y, i, avg + range * (2.0f * u - 1.0f)); /* (a bf16 tensor keeps the rounding) */
    }
}

/* libnc.h:201: 0 with probability prob, else 1/(1-prob) */
void nc_tensor_set_dropout(NCTensor *y, float prob, NCRNDState *rs)
{
    size_t n = nc_numel(y);
    float keep = 1.0f / (1.0f - prob);
    for (size_t i = 0; i < n; i++) {
        float u = (float)(xorwow(rs) >> 8) * (1.0f / 16777216.0f);
        nc_f32(y)[i] = u < prob ? 0.0f : keep;
    }
}

/* ---- parameters (libnc.h:501-525) ---------------------------------------- */
static void list_add_tail_(struct list_head *el, struct list_head *head)
{
    el->prev = head->prev;
    el->next = head;
    head->prev->next = el;
    head->prev = el;
}

void nc_param_list_init(NCContext *m, NCParamList *pl)
{
    pl->ctx = m;
    pl->param_list.prev = pl->param_list.next = &pl->param_list;
    pl->add_graph = 1;
}

/* Registers the ADDRESS of the model's tensor pointer (nncp.c:273, 371, ...)
   and turns the tensor into a graph leaf whose gradient is reported with the
   NCParam as opaque (libnc.h:453-457). */
NCParam *nc_new_param(NCParamList *pl, NCTensor **pval, const char *fmt, ...)
{
    char buf[128];
    va_list ap;
    NCParam *p = nc_mallocz(sizeof(*p));
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    p->pval = pval;
    p->name = strdup(buf);
    p->lr_mult = 1.0f;
    list_add_tail_(&p->link, &pl->param_list);
    nc_set_param(*pval, p);
    return p;
}

size_t nc_get_param_count(NCParamList *pl)
{
    size_t n = 0;
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next)
        n += nc_numel(*((NCParam *)el)->pval);
    return n;
}

/* frees the list AND the parameter tensors (trf_end never frees them,
   nncp.c:522-550) */
void nc_param_list_end(NCParamList *pl)
{
    struct list_head *el = pl->param_list.next, *next;
    for (; el != &pl->param_list; el = next) {
        NCParam *p = (NCParam *)el;
        next = el->next;
        nc_free_tensor(*p->pval);
        *p->pval = NULL;
        free(p->name);
        nc_free(p);
    }
    pl->param_list.prev = pl->param_list.next = &pl->param_list;
}

/* ---- optimiser (libnc.h:540-572) ------------------------------------------
   Build-defined where the header is silent:
   sgd_opt_update_var() only ACCUMULATES the reported gradient (tied tensors
   are reported once per use); nc_sgd_opt_update() applies the update to every
   parameter that received one and advances the step counter t.
     ADAM   : g = clamp(g, -clip, clip) if clip != 0 (element-wise);
              m = b1*m + (1-b1)*g ; v = b2*v + (1-b2)*g*g ;
              w -= lr * (m/(1-b1^t)) / (sqrt(v/(1-b2^t)) + eps)
     RMSPROP: v = b2*v + (1-b2)*g*g ; w -= lr * g / (sqrt(v) + eps)
     BASIC  : w -= lr * g                                                    */
struct SGDOptVarState {
    NCSGDOptState *opt;
    NCParam *param;
    float *m, *v, *g;
    float *master; /* bf16 parameters: the fp32 values the update works on */
    size_t n;
    int has_grad;
    struct SGDOptVarState *next;
};

struct NCSGDOptState {
    NCContext *ctx;
    SGDOptParams p;
    int64_t step;
    struct SGDOptVarState *vars;
};

NCSGDOptState *nc_sgd_opt_init(NCContext *m, const SGDOptParams *p)
{
    NCSGDOptState *s = nc_mallocz(sizeof(*s));
    s->ctx = m;
    s->p = *p;
    return s;
}

void nc_sgd_opt_end(NCSGDOptState *s)
{
    nc_free(s);
}

void nc_sgd_opt_set_all(NCParamList *pl, NCSGDOptState *s)
{
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next) {
        NCParam *p = (NCParam *)el;
        if (p->sgd_opt) {
            struct SGDOptVarState *vs = p->sgd_opt, **pp;
            for (pp = &vs->opt->vars; *pp; pp = &(*pp)->next)
                if (*pp == vs) { *pp = vs->next; break; }
            free(vs->m); free(vs->v); free(vs->g); free(vs->master);
            nc_free(vs);
            p->sgd_opt = NULL;
        }
        if (s) {
            struct SGDOptVarState *vs = nc_mallocz(sizeof(*vs)), **pp;
            vs->opt = s;
            vs->param = p;
            vs->n = nc_numel(*p->pval);
            vs->m = nc_mallocz(vs->n * sizeof(float));
            vs->v = nc_mallocz(vs->n * sizeof(float));
            vs->g = nc_mallocz(vs->n * sizeof(float));
            if ((*p->pval)->type == NC_TYPE_BF16) {
                /* the update works on an fp32 master that starts as the parameter's value;
                   the parameter itself holds the master's rounding */
                NCTensor *c = nc_contig(nc_dup_tensor(*p->pval));
                vs->master = nc_malloc(vs->n * sizeof(float));
                for (size_t i = 0; i < vs->n; i++)
                    vs->master[i] = (float)load_elem(c, i);
                nc_free_tensor(c);
            }
            for (pp = &s->vars; *pp; pp = &(*pp)->next)
                ;
            *pp = vs;
            p->sgd_opt = vs;
        }
    }
}

void nc_sgd_opt_set_lr(NCSGDOptState *s, float lr) { s->p.lr = lr; }

/* nc_ext.h: a parameter's moments as tensors (the checker keeps both for every algorithm;
   the ones an algorithm never touches read as NULL, as in the product) */
static float *moment_of(NCParam *p, int which)
{
    struct SGDOptVarState *vs = p->sgd_opt;
    if (!vs)
        return NULL;
    int algo = (int)vs->opt->p.algo;
    if (which == 0)
        return algo == SGD_OPT_ADAM && vs->opt->p.u.adam.beta1 != 0.0f ? vs->m : NULL;
    if (which == 1)
        return algo != SGD_OPT_BASIC ? vs->v : NULL;
    if (which == 2)
        return vs->master;
    return NULL;
}

NCTensor *nc_sgd_opt_get_state(NCParam *p, int which)
{
    float *src = moment_of(p, which);
    if (!src)
        return NULL;
    NCTensor *t = nc_new_tensor_1d(nc_new_cpu_device((*p->pval)->dev->ctx), NC_TYPE_F32, p->sgd_opt->n);
    memcpy(nc_f32(t), src, p->sgd_opt->n * sizeof(float));
    return t;
}

void nc_sgd_opt_set_state(NCParam *p, int which, const NCTensor *v)
{
    float *dst = moment_of(p, which);
    if (!dst)
        nc_fatal("nc_sgd_opt_set_state: '%s' keeps no moment %d", p->name, which);
    if (v->type != NC_TYPE_F32 || nc_numel(v) != p->sgd_opt->n)
        nc_fatal("nc_sgd_opt_set_state: %zu f32 values expected for '%s'", p->sgd_opt->n, p->name);
    NCTensor *c = nc_contig(nc_dup_tensor(v));
    memcpy(dst, nc_f32(c), p->sgd_opt->n * sizeof(float));
    nc_free_tensor(c);
}

int64_t nc_sgd_opt_get_step(NCSGDOptState *s) { return s->step; }
void nc_sgd_opt_set_step(NCSGDOptState *s, int64_t step) { s->step = step; }

/* libnc.h:563: the NCParamUpdateFunc nncp.c forwards to (nncp.c:1095);
   opaque is the NCParam, yg is consumed. */
void sgd_opt_update_var(void *opaque, NCTensor *yg, NCTensor *get_col_index)
{
    NCParam *p = opaque;
    struct SGDOptVarState *vs = p->sgd_opt;
    if (get_col_index)
        nc_fatal("sparse gradients are not supported");
    if (vs) {
        yg = nc_contig(yg);
        if (nc_numel(yg) != vs->n)
            nc_fatal("gradient size mismatch for %s", p->name);
        const float *g = nc_f32(yg);
        if (!vs->has_grad) {
            memcpy(vs->g, g, vs->n * sizeof(float));
            vs->has_grad = 1;
        } else {
            for (size_t i = 0; i < vs->n; i++)
                vs->g[i] += g[i];
        }
    }
    nc_free_tensor(yg);
}

void nc_sgd_opt_update(NCSGDOptState *s)
{
    const SGDOptParams *p = &s->p;
    float b1 = p->u.adam.beta1, b2 = p->u.adam.beta2, eps = p->u.adam.eps;
    float clip = p->u.adam.gradient_clip;
    s->step++;
    float c1 = 1.0f / (1.0f - powf(b1, (float)s->step));
    float c2 = 1.0f / (1.0f - powf(b2, (float)s->step));
    for (struct SGDOptVarState *vs = s->vars; vs; vs = vs->next) {
        if (!vs->has_grad)
            continue;
        NCTensor *wt = *vs->param->pval;
        float lr = p->lr * vs->param->lr_mult;
        if (!nc_is_contig(wt) || (wt->type != NC_TYPE_F32 && !vs->master))
            nc_fatal("optimiser: contiguous f32 or bf16 parameter expected");
        float *w = vs->master ? vs->master : nc_f32(wt);
        #pragma omp parallel for if (vs->n > 65536)
        for (size_t i = 0; i < vs->n; i++) {
            float g = vs->g[i];
            switch ((int)p->algo) {
            case SGD_OPT_BASIC:
                w[i] -= lr * g;
                break;
            case SGD_OPT_ADAM: {
                if (clip != 0.0f)
                    g = fminf(fmaxf(g, -clip), clip);
                float m = b1 * vs->m[i] + (1.0f - b1) * g;
                float v = b2 * vs->v[i] + (1.0f - b2) * g * g;
                vs->m[i] = m;
                vs->v[i] = v;
                w[i] -= lr * (m * c1) / (sqrtf(v * c2) + eps);
                break;
            }
            case SGD_OPT_RMSPROP: {
                float v = b2 * vs->v[i] + (1.0f - b2) * g * g;
                vs->v[i] = v;
                w[i] -= lr * g / (sqrtf(v) + eps);
                break;
            }
            default:
                nc_fatal("unsupported optimiser %d", p->algo);
            }
        }
        if (vs->master) {
            uint16_t *w16 = (uint16_t *)wt->buf->data + wt->off;
            for (size_t i = 0; i < vs->n; i++)
                w16[i] = nc_bf16_bits(vs->master[i]);
        }
        vs->has_grad = 0;
    }
}

/* libnc.h:600; fixed left-to-right order so encoder and decoder agree */
float vec_sum_f32(const float *tab, size_t n)
{
    float s = 0;
    for (size_t i = 0; i < n; i++)
        s += tab[i];
    return s;
}
