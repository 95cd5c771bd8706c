// libnc_hip core: context, devices, pooled memory, tensors and views, host <->
// device moves, RNG fills, parameter lists, optimiser, graph nodes and the
// backward walk.  Semantics follow libnc.h (cited per function) and the way
// nncp.c drives it; behaviour the header leaves open is defined in
// include/nc_api.h.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <dlfcn.h>
#include <time.h>
#include "nc_hip_internal.h"

[[noreturn]] void nc_fatal(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    fprintf(stderr, "libnc_hip: ");
    vfprintf(stderr, fmt, ap);
    fprintf(stderr, "\n");
    va_end(ap);
    abort();
}

void hip_check(hipError_t e, const char *what)
{
    if (e != hipSuccess)
        nc_fatal("%s: %s", what, hipGetErrorString(e));
}

// ---- pools ----------------------------------------------------------------
size_t Pool::round_size(size_t n)
{
    if (n <= 256) return 256;
    if (n <= (2u << 20)) {
        size_t p = 256;
        while (p < n) p <<= 1;
        return p;
    }
    const size_t g = 2u << 20;
    return (n + g - 1) / g * g;
}

void *Pool::get(size_t n, size_t *cap)
{
    size_t c = round_size(n);
    *cap = c;
    auto it = free_lists.find(c);
    if (it != free_lists.end() && !it->second.empty()) {
        void *p = it->second.back();
        it->second.pop_back();
        return p;
    }
    void *p = nullptr;
    if (device)
        hip_check(hipMalloc(&p, c), "hipMalloc");
    else
        hip_check(hipHostMalloc(&p, c, hipHostMallocDefault), "hipHostMalloc");
    all.push_back(p);
    bytes += (int64_t)c;
    return p;
}

void Pool::put(void *p, size_t cap)
{
    free_lists[cap].push_back(p);
}

void Pool::release_all()
{
    for (void *p : all) {
        if (device) (void)hipFree(p);
        else (void)hipHostFree(p);
    }
    all.clear();
    free_lists.clear();
    bytes = 0;
}

// ---- memory / context (libnc.h:117-130) -------------------------------------
extern "C" void *nc_malloc(size_t size)
{
    void *p = malloc(size ? size : 1);
    if (!p) nc_fatal("out of host memory (%zu bytes)", size);
    return p;
}

extern "C" void *nc_mallocz(size_t size)
{
    void *p = nc_malloc(size);
    memset(p, 0, size);
    return p;
}

extern "C" void nc_free(void *ptr) { free(ptr); }

extern "C" NCContext *nc_context_init(int nb_threads)
{
    NCContext *m = new NCContext();
    m->nb_threads = nb_threads;
    m->cpu.ctx = m; m->cpu.is_hip = false;
    m->hip.ctx = m; m->hip.is_hip = true;
    m->hip_ready = false;
    m->stream = nullptr;
    m->dev_pool.device = true;
    m->host_pool.device = false;
    m->matmul_bf16 = 0;
    m->matmul_invariant = 0;
    m->bf16_copy_results = 0;
    m->launches = 0;
    m->shadow_casts = 0;
    m->node_seq = 0;
    m->epoch = 0;
    m->defer_wgrad = false;
    for (int i = 0; i < NC_BW_ARGS; i++) { m->bw_prev[i] = nullptr; m->bw_used[i] = false; }
    m->grp_staging = nullptr;
    m->grp_staging_cap = 0;
    m->red_staging = nullptr;
    m->red_staging_cap = 0;
    m->grp_staging_stamp = m->red_staging_stamp = 0;
    m->sync_count = 0;
    const char *e = getenv("NCHIP_MATMUL_BF16");
    if (e && atoi(e) != 0)
        m->matmul_bf16 = 1;
    return m;
}

static void staging_reclaim(NCContext *m);

extern "C" void nc_context_end(NCContext *m)
{
    if (!m) return;
    nc_forget_k_major_weights(m);
    if (m->hip_ready) {
        (void)hipStreamSynchronize(m->stream);
        m->sync_count++;
        staging_reclaim(m);
        m->dev_pool.release_all();
        m->host_pool.release_all();
        (void)hipStreamDestroy(m->stream);
    }
    delete m;
}

static void hip_init(NCContext *m, int index)
{
    if (m->hip_ready) return;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= index)
        nc_fatal("no HIP device %d (found %d): this library has no CPU compute path", index, n);
    hip_check(hipSetDevice(index), "hipSetDevice");
    hip_check(hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking), "hipStreamCreate");
    m->hip_ready = true;
}

// Host staging memory is pinned (hipHostMalloc), so creating the first host
// tensor already needs the HIP runtime.
extern "C" NCDevice *nc_new_cpu_device(NCContext *m) { return &m->cpu; }

// nncp.c:2773-2774 calls this for --cuda; here it is the MI355X.
extern "C" NCDevice *nc_new_cuda_device(NCContext *m, int device_index)
{
    hip_init(m, device_index);
    return &m->hip;
}

extern "C" NCDevice *nc_new_device(NCContext *m, const char *name)
{
    if (name && (!strcmp(name, "hip") || !strcmp(name, "cuda")))
        return nc_new_cuda_device(m, 0);
    return &m->cpu;
}

// pinned tables whose upload the stream has consumed (a wait has happened since it was
// enqueued) go back to the host pool
static void staging_reclaim(NCContext *m)
{
    size_t kept = 0;
    for (const StagingRetired &r : m->staging_retired) {
        if (r.stamp < m->sync_count) m->host_pool.put(r.p, r.cap);
        else m->staging_retired[kept++] = r;
    }
    m->staging_retired.resize(kept);
}

void nc_stream_wait(NCContext *m)
{
    hip_check(hipStreamSynchronize(m->stream), "hipStreamSynchronize");
    m->sync_count++;
    staging_reclaim(m);
    if (nchip_index_error())
        nc_fatal("a token index outside its table reached nc_get_col or nc_indexed_log");
}

// A pinned table that an asynchronous upload reads may be rewritten only after the stream
// has executed that upload.  The host runs ahead of the stream, so "enough later launches
// were issued" says nothing: the buffer waits in a list until the stream has been waited for
// at least once since the upload was enqueued (stamp = the wait count at that moment).
// No wait is forced here - a training step waits twice on its own (distributions to the
// host, loss) - unless the list grows long.
void nc_staging_retire(NCContext *m, void *p, size_t cap, uint64_t stamp)
{
    if (!p) return;
    m->staging_retired.push_back(StagingRetired{ p, cap, stamp });
    if (m->staging_retired.size() > 64) nc_stream_wait(m);
    else staging_reclaim(m);
}

void nc_mark_in_flight(NCTensor *x)
{
    x->buf->in_flight = x->buf->dev->ctx->sync_count + 1;
}

extern "C" void nc_synchronize(NCDevice *d)
{
    if (d->ctx->hip_ready)
        nc_stream_wait(d->ctx);
}

// ---- profiling hooks (libnc.h:14-67) -----------------------------------------------------
// Section timers of the host code above the ABI: wall-clock nanoseconds per section (the
// kernels of a section run asynchronously, so a section's time is the time the host spent
// in it, waits included), plus - with NC_PROFILE set - a roctx range per section for
// rocprofv3's marker trace.  The roctx library is looked up at run time and only then.
extern "C" {
int64_t prof_cycles[PROF_COUNT], prof_samples[PROF_COUNT], prof_ops[PROF_COUNT];
}
static const char *const PROF_NAMES[PROF_COUNT] = { "EVAL", "GRAD", "SGD", "UPDATE", "WRITE_SYM", "PROBE", "TOTAL" };
static bool prof_enabled() { static const bool on = getenv("NC_PROFILE") && *getenv("NC_PROFILE"); return on; }
typedef int (*RoctxPush)(const char *);
typedef int (*RoctxPop)(void);
static RoctxPush roctx_push;
static RoctxPop roctx_pop;
static void roctx_lookup()
{
    static bool done = false;
    if (done) return;
    done = true;
    for (const char *name : { "libroctx64.so.4", "libroctx64.so", "librocprofiler-sdk-roctx.so.1" }) {
        if (void *h = dlopen(name, RTLD_NOW | RTLD_LOCAL)) {
            roctx_push = (RoctxPush)dlsym(h, "roctxRangePushA");
            roctx_pop = (RoctxPop)dlsym(h, "roctxRangePop");
            if (roctx_push && roctx_pop) return;
            roctx_push = nullptr; roctx_pop = nullptr;
        }
    }
}
static int64_t prof_now()
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (int64_t)ts.tv_sec * 1000000000 + ts.tv_nsec;
}

extern "C" void nc_prof_begin(int idx)
{
    if (idx < 0 || idx >= PROF_COUNT) return;
    if (prof_enabled()) {
        roctx_lookup();
        if (roctx_push) roctx_push(PROF_NAMES[idx]);
    }
    prof_cycles[idx] -= prof_now();
}

extern "C" void nc_prof_finish(int idx, int n_ops)
{
    if (idx < 0 || idx >= PROF_COUNT) return;
    prof_cycles[idx] += prof_now();
    prof_samples[idx]++;
    prof_ops[idx] += n_ops;
    if (prof_enabled() && roctx_pop) roctx_pop();
}

extern "C" void nc_prof_dump(void) // libnc.h:67
{
    if (!prof_enabled()) return;
    fprintf(stderr, "%-10s %10s %14s %12s %12s\n", "section", "samples", "total ms", "us/sample", "ops");
    for (int i = 0; i < PROF_COUNT; i++) {
        if (!prof_samples[i]) continue;
        fprintf(stderr, "%-10s %10lld %14.3f %12.2f %12lld\n", PROF_NAMES[i], (long long)prof_samples[i],
                prof_cycles[i] * 1e-6, prof_cycles[i] * 1e-3 / prof_samples[i], (long long)prof_ops[i]);
    }
}

extern "C" int nc_set_matmul_width_invariant(NCContext *m, int enable) // nc_ext.h
{
    int old = m->matmul_invariant;
    m->matmul_invariant = enable != 0;
    return old;
}

extern "C" int nc_set_bf16_copy_of_results(NCContext *m, int enable) // nc_ext.h
{
    int old = m->bf16_copy_results;
    m->bf16_copy_results = enable != 0;
    return old;
}

extern "C" int nc_set_matmul_bf16(NCContext *m, int enable)
{
    int old = m->matmul_bf16;
    m->matmul_bf16 = enable != 0;
    return old;
}

extern "C" int64_t nc_get_launch_count(NCContext *m) { return m->launches; }

extern "C" void *nc_context_stream(NCContext *m) { return m->hip_ready ? (void *)m->stream : nullptr; }

extern "C" int nc_set_deferred_weight_grad(NCContext *m, int enable)
{
    int old = m->defer_wgrad;
    m->defer_wgrad = enable != 0;
    return old;
}

// ---- tensors ----------------------------------------------------------------
size_t nc_type_size(NCTypeEnum t)
{
    switch (t) {
    case NC_TYPE_F32: case NC_TYPE_I32: case NC_TYPE_U32: return 4;
    case NC_TYPE_BF16: case NC_TYPE_F16: case NC_TYPE_I16: case NC_TYPE_U16: return 2;
    case NC_TYPE_I8: case NC_TYPE_U8: return 1;
    default: nc_fatal("unsupported tensor type %d", (int)t);
    }
}

size_t nc_numel(const NCTensor *x)
{
    size_t n = 1;
    for (int i = 0; i < x->n_dims; i++) n *= x->dims[i];
    return n;
}

bool nc_is_contig(const NCTensor *x)
{
    size_t s = 1;
    for (int i = 0; i < x->n_dims; i++) {
        if (x->dims[i] != 1 && x->strides[i] != s) return false;
        s *= x->dims[i];
    }
    return true;
}

void *nc_data(const NCTensor *x)
{
    return (uint8_t *)x->buf->ptr + x->off * nc_type_size(x->type);
}

NCContext *nc_ctx(const NCTensor *x) { return x->dev->ctx; }

void need_dev(const NCTensor *x, const char *op)
{
    if (!x->dev->is_hip)
        nc_fatal("%s on a host tensor: libnc_hip computes on the GPU only "
                 "(create the model with nc_new_cuda_device / nncp --cuda)", op);
}

static Pool &pool_of(NCDevice *d)
{
    NCContext *m = d->ctx;
    if (!m->hip_ready) {
        // host staging buffers are pinned, which needs the runtime
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess || n < 1)
            nc_fatal("no HIP device found: this library has no CPU compute path");
        hip_check(hipSetDevice(0), "hipSetDevice");
        hip_check(hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking), "hipStreamCreate");
        m->hip_ready = true;
    }
    return d->is_hip ? m->dev_pool : m->host_pool;
}

NCTensor *nc_alloc(NCDevice *d, NCTypeEnum t, int nd, const size_t *dims, bool zero)
{
    if (nd > NC_N_DIMS_MAX) nc_fatal("too many dimensions (%d)", nd);
    NCTensor *x = (NCTensor *)nc_mallocz(sizeof(NCTensor));
    size_t n = 1;
    x->ref = 1; x->dev = d; x->type = t; x->n_dims = nd;
    for (int i = 0; i < nd; i++) { x->dims[i] = dims[i]; x->strides[i] = n; n *= dims[i]; }
    x->buf = (NCTensorBuffer *)nc_mallocz(sizeof(NCTensorBuffer));
    x->buf->ref = 1;
    x->buf->dev = d;
    size_t bytes = n * nc_type_size(t);
    x->buf->elems = n;
    x->buf->ptr = pool_of(d).get(bytes ? bytes : 4, &x->buf->cap);
    if (zero && bytes) {
        if (d->is_hip) { k_fill_bytes(d->ctx->stream, x->buf->ptr, 0, (int64_t)bytes); d->ctx->launches++; }
        else memset(x->buf->ptr, 0, bytes);
    }
    return x;
}

NCTensor *nc_alloc_like(const NCTensor *x) { return nc_alloc(x->dev, x->type, x->n_dims, x->dims, false); }

NCTensor *nc_view(const NCTensor *x)
{
    NCTensor *y = (NCTensor *)nc_mallocz(sizeof(NCTensor));
    *y = *x;
    y->ref = 1;
    y->node = nullptr;
    y->buf->ref++;
    return y;
}

NCTensor *nc_reshape_view(NCTensor *x, int nd, const size_t *dims)
{
    x = nc_contig(x);
    NCTensor *y = nc_view(x);
    size_t s = 1;
    y->n_dims = nd;
    for (int i = 0; i < nd; i++) { y->dims[i] = dims[i]; y->strides[i] = s; s *= dims[i]; }
    if (s != nc_numel(x)) nc_fatal("reshape: element count mismatch (%zu vs %zu)", s, nc_numel(x));
    nc_free_tensor(x);
    return y;
}

// ---- bf16 shadows --------------------------------------------------------------------------
static bool shadow_capable(const NCTensor *x)
{
    return x->dev->is_hip && x->type == NC_TYPE_F32 && nc_is_contig(x) && x->off % 8 == 0 && x->buf->elems > 0;
}

static void shadow_alloc(NCContext *m, NCTensorBuffer *b)
{
    if (!b->sh) {
        b->sh = (uint16_t *)m->dev_pool.get(b->elems * sizeof(uint16_t) + 64, &b->sh_cap);
        b->sh_valid = false;
    }
}

static int g_shadow_check = getenv("NCHIP_SHADOW_CHECK") ? atoi(getenv("NCHIP_SHADOW_CHECK")) : 0;
static int shadow_check_mode() { return g_shadow_check; }

extern "C" int nc_set_bf16_shadow_check(int enable) // nc_ext.h
{
    int old = g_shadow_check;
    g_shadow_check = enable != 0;
    return old;
}

extern "C" int64_t nc_get_bf16_cast_count(NCContext *m) { return m->shadow_casts; } // nc_ext.h

const uint16_t *nc_shadow_of(NCContext *m, const NCTensor *x)
{
    if (!shadow_capable(x)) return nullptr;
    NCTensorBuffer *b = x->buf;
    if (b->sh_valid && shadow_check_mode()) {
        // debugging aid: a shadow that claims to be valid must equal a fresh cast
        size_t cap;
        uint16_t *tmp = (uint16_t *)m->dev_pool.get(b->elems * sizeof(uint16_t) + 64, &cap);
        if (nchip_cast_bf16(m->stream, (const float *)b->ptr, tmp, (int64_t)b->elems)) nc_fatal("bf16 cast failed");
        std::vector<uint16_t> h0(b->elems), h1(b->elems);
        hip_check(hipMemcpyAsync(h0.data(), tmp, b->elems * 2, hipMemcpyDeviceToHost, m->stream), "shadow check copy");
        hip_check(hipMemcpyAsync(h1.data(), b->sh, b->elems * 2, hipMemcpyDeviceToHost, m->stream), "shadow check copy");
        nc_stream_wait(m);
        m->dev_pool.put(tmp, cap);
        if (memcmp(h0.data(), h1.data(), b->elems * 2) != 0)
            nc_fatal("bf16 shadow of a buffer of %zu elements is stale (a writer did not invalidate it)", b->elems);
    }
    if (!b->sh_valid) {
        shadow_alloc(m, b);
        if (nchip_cast_bf16(m->stream, (const float *)b->ptr, b->sh, (int64_t)b->elems)) nc_fatal("bf16 cast failed");
        m->launches++;
        m->shadow_casts++;
        b->sh_valid = true;
        static const bool trace = getenv("NCHIP_SHADOW_TRACE") != nullptr;
        if (trace) fprintf(stderr, "[cast] %zu elements, tensor dims %zu x %zu (rank %d)\n", b->elems,
                           x->n_dims > 0 ? x->dims[0] : 1, x->n_dims > 1 ? x->dims[1] : 1, x->n_dims);
    }
    return b->sh + x->off;
}

uint16_t *nc_shadow_for_write(NCContext *m, NCTensor *x)
{
    if (!shadow_capable(x) || x->off != 0 || nc_numel(x) != x->buf->elems) return nullptr;
    shadow_alloc(m, x->buf);
    x->buf->sh_valid = true;
    return x->buf->sh;
}

void nc_shadow_invalidate(NCTensor *x)
{
    if (!x || !x->buf) return;
    x->buf->sh_valid = false;
    x->buf->wide_valid = false;
    x->buf->version++;
}

// ---- bf16 tensors as operands --------------------------------------------------------------
NCTensor *nc_operand(NCTensor *x)
{
    if (x->type != NC_TYPE_BF16) return nc_contig(x);
    need_dev(x, "an op on a bf16 tensor");
    NCContext *m = nc_ctx(x);
    NCTensorBuffer *b = x->buf;
    if (!b->wide) {
        size_t n = b->elems ? b->elems : 1;
        b->wide = nc_alloc(x->dev, NC_TYPE_F32, 1, &n, false);
        NCTensorBuffer *wb = b->wide->buf;
        wb->sh = (uint16_t *)b->ptr;
        wb->sh_cap = 0;
        wb->sh_alias = true;
        wb->sh_valid = false;
        b->wide_valid = false;
    }
    if (!b->wide_valid) {
        if (nchip_widen_bf16(m->stream, (const uint16_t *)b->ptr, (float *)b->wide->buf->ptr, (int64_t)b->elems))
            nc_fatal("bf16 widening failed");
        m->launches++;
        b->wide_valid = true;
        b->wide->buf->sh_valid = true; // the bf16 buffer IS the rounding of its own widening
    }
    NCTensor *y = nc_view(b->wide);
    y->off = x->off;
    y->n_dims = x->n_dims;
    for (int i = 0; i < x->n_dims; i++) { y->dims[i] = x->dims[i]; y->strides[i] = x->strides[i]; }
    y->node = nc_dup_node(x->node);
    nc_free_tensor(x);
    return nc_contig(y);
}

float *nc_tmp_f32(NCContext *m, size_t n, size_t *cap)
{
    return (float *)m->dev_pool.get(n * sizeof(float), cap);
}

void nc_tmp_free(NCContext *m, void *p, size_t cap) { m->dev_pool.put(p, cap); }

// libnc.h:153-171; the plain constructors zero the data (nncp.c relies on it
// for b_r, b_q, the biases and ln_b: nncp.c:369-372, 275-276)
extern "C" NCTensor *nc_new_tensor(NCDevice *d, NCTypeEnum t, int n, const size_t *dims) { return nc_alloc(d, t, n, dims, true); }
extern "C" NCTensor *nc_new_tensor_nz(NCDevice *d, NCTypeEnum t, int n, const size_t *dims) { return nc_alloc(d, t, n, dims, false); }
extern "C" NCTensor *nc_new_tensor_from_tensor_nz(const NCTensor *x) { return nc_alloc_like(x); }
extern "C" NCTensor *nc_new_scalar(NCDevice *d, NCTypeEnum t) { return nc_alloc(d, t, 0, nullptr, true); }
extern "C" NCTensor *nc_new_tensor_1d(NCDevice *d, NCTypeEnum t, size_t n0) { size_t s[1] = { n0 }; return nc_alloc(d, t, 1, s, true); }
extern "C" NCTensor *nc_new_tensor_2d(NCDevice *d, NCTypeEnum t, size_t n0, size_t n1) { size_t s[2] = { n0, n1 }; return nc_alloc(d, t, 2, s, true); }
extern "C" NCTensor *nc_new_tensor_3d(NCDevice *d, NCTypeEnum t, size_t n0, size_t n1, size_t n2) { size_t s[3] = { n0, n1, n2 }; return nc_alloc(d, t, 3, s, true); }
extern "C" NCTensor *nc_new_tensor_4d(NCDevice *d, NCTypeEnum t, size_t n0, size_t n1, size_t n2, size_t n3) { size_t s[4] = { n0, n1, n2, n3 }; return nc_alloc(d, t, 4, s, true); }

extern "C" NCTensor *nc_new_f32(NCDevice *d, float val) // libnc.h:278
{
    NCTensor *x = nc_alloc(d, NC_TYPE_F32, 0, nullptr, false);
    if (d->is_hip) { k_fill_f32(d->ctx->stream, nc_f32(x), val, 1); d->ctx->launches++; }
    else nc_f32(x)[0] = val;
    return x;
}

extern "C" NCTensor *nc_tensor_set_name(NCTensor *x, const char *fmt, ...) { (void)fmt; return x; }

extern "C" NCTensor *nc_dup_tensor(const NCTensor *x) // libnc.h:173
{
    if (x) ((NCTensor *)x)->ref++;
    return (NCTensor *)x;
}

extern "C" void nc_free_tensor(NCTensor *x) // libnc.h:174; NULL accepted (nncp.c:532-534)
{
    if (!x || --x->ref > 0) return;
    nc_free_node(x->node);
    if (--x->buf->ref == 0) {
        NCContext *m = x->buf->dev->ctx;
        if (x->buf->sh && !x->buf->sh_alias) m->dev_pool.put(x->buf->sh, x->buf->sh_cap); // stream ordered, like the buffer itself
        if (NCTensor *wide = x->buf->wide) {
            // the f32 copy of a bf16 buffer borrowed this buffer as its shadow: views of the
            // copy may outlive it, and make a shadow of their own from then on
            wide->buf->sh = nullptr; wide->buf->sh_cap = 0;
            wide->buf->sh_alias = false; wide->buf->sh_valid = false;
            x->buf->wide = nullptr;
            nc_free_tensor(wide);
        }
        if (x->buf->in_flight && !x->buf->dev->is_hip && x->buf->in_flight > m->sync_count)
            nc_staging_retire(m, x->buf->ptr, x->buf->cap, x->buf->in_flight - 1); // a queued kernel may still use it
        else
            pool_of(x->buf->dev).put(x->buf->ptr, x->buf->cap);
        free(x->buf);
    }
    free(x);
}

extern "C" NCNode *nc_get_node(NCTensor *x) { return x->node; }
extern "C" NCTypeEnum nc_tensor_get_item_type(const NCTensor *x) { return x->type; }
extern "C" NCDevice *nc_get_tensor_device(const NCTensor *x) { return x->dev; }

extern "C" int nc_tensor_get_dims(const NCTensor *x, size_t *dims)
{
    if (dims) for (int i = 0; i < x->n_dims; i++) dims[i] = x->dims[i];
    return x->n_dims;
}

// libnc.h:183-185.  Host tensors: the address the coder reads (nncp.c:3005).
// Device tensors: the device address, for callers of the nchip_* kernel ABI.
extern "C" void *nc_tensor_get_ptr(const NCTensor *x, size_t *pstride)
{
    if (pstride) *pstride = x->n_dims >= 2 ? x->strides[1] : (x->n_dims ? x->dims[0] : 1);
    nc_shadow_invalidate((NCTensor *)x); // the address leaves the library: whoever holds it may write
    return nc_data(x);
}

// ---- strided copies ---------------------------------------------------------
static void host_copy_strided(NCTensor *dst, const NCTensor *src)
{
    size_t n = nc_numel(dst), es = nc_type_size(dst->type);
    size_t idx[NC_N_DIMS_MAX] = { 0 }, so = 0, dof = 0;
    const uint8_t *sp = (const uint8_t *)nc_data(src);
    uint8_t *dp = (uint8_t *)nc_data(dst);
    for (size_t e = 0; e < n; e++) {
        memcpy(dp + dof * es, sp + so * es, es);
        for (int a = 0; a < dst->n_dims; a++) {
            idx[a]++; so += src->strides[a]; dof += dst->strides[a];
            if (idx[a] < dst->dims[a]) break;
            so -= src->strides[a] * dst->dims[a];
            dof -= dst->strides[a] * dst->dims[a];
            idx[a] = 0;
        }
    }
}

void nc_copy_any(NCTensor *dst, const NCTensor *src)
{
    if (dst->n_dims != src->n_dims || dst->type != src->type)
        nc_fatal("copy: rank or type mismatch");
    for (int i = 0; i < dst->n_dims; i++)
        if (dst->dims[i] != src->dims[i])
            nc_fatal("copy: shape mismatch on axis %d (%zu vs %zu)", i, dst->dims[i], src->dims[i]);
    if (dst->dev != src->dev)
        nc_fatal("copy: tensors live on different devices");
    if (nc_numel(dst) == 0) return;
    // A contiguous range written into a buffer whose bf16 copy is in use (the memory of a layer,
    // which takes a new segment per step): the copy is brought up to date over that range - from
    // the source's own copy when it has one, else by a cast of the range - instead of being
    // dropped and rebuilt over the whole buffer at its next use.
    const bool keep_shadow = dst->dev->is_hip && dst->dev->ctx->matmul_bf16 && dst->buf->sh && dst->buf->sh_valid &&
                             shadow_capable(dst) && nc_is_contig(src) && nc_numel(dst) < dst->buf->elems;
    nc_shadow_invalidate(dst);
    if (!dst->dev->is_hip) { host_copy_strided(dst, src); return; }
    NCContext *m = dst->dev->ctx;
    if (nc_is_contig(dst) && nc_is_contig(src)) {
        const size_t n = nc_numel(dst);
        hip_check(hipMemcpyAsync(nc_data(dst), nc_data(src), n * nc_type_size(dst->type),
                                 hipMemcpyDeviceToDevice, m->stream), "hipMemcpyAsync d2d");
        if (keep_shadow) {
            uint16_t *range = dst->buf->sh + dst->off;
            // (within one buffer the flag was just cleared: a cast of the range then)
            if (src->buf != dst->buf && src->buf->sh && src->buf->sh_valid && shadow_capable(src))
                hip_check(hipMemcpyAsync(range, src->buf->sh + src->off, n * sizeof(uint16_t), hipMemcpyDeviceToDevice, m->stream),
                          "hipMemcpyAsync d2d (bf16 copy)");
            else {
                if (nchip_cast_bf16(m->stream, nc_f32(dst), range, (int64_t)n)) nc_fatal("bf16 cast failed");
                m->launches++;
                m->shadow_casts++;
            }
            dst->buf->sh_valid = true;
        }
        return;
    }
    NdDesc d;
    d.nd = 0;
    // merge axes that are contiguous in both tensors to cut index arithmetic
    for (int a = 0; a < dst->n_dims; a++) {
        if (dst->dims[a] == 1) continue;
        if (d.nd > 0 && src->strides[a] == d.sa[d.nd - 1] * d.dims[d.nd - 1] &&
            dst->strides[a] == d.sb[d.nd - 1] * d.dims[d.nd - 1]) {
            d.dims[d.nd - 1] *= (int64_t)dst->dims[a];
            continue;
        }
        d.dims[d.nd] = (int64_t)dst->dims[a];
        d.sa[d.nd] = (int64_t)src->strides[a];
        d.sb[d.nd] = (int64_t)dst->strides[a];
        d.nd++;
    }
    if (d.nd == 0) { d.nd = 1; d.dims[0] = 1; d.sa[0] = d.sb[0] = 1; }
    k_copy_nd(m->stream, nc_data(src), nc_data(dst), &d, (int)nc_type_size(dst->type));
    m->launches++;
}

NCTensor *nc_contig(NCTensor *x)
{
    if (nc_is_contig(x)) return x;
    NCTensor *y = nc_alloc_like(x);
    nc_copy_any(y, x);
    y->node = nc_dup_node(x->node);
    nc_free_tensor(x);
    return y;
}

extern "C" void nc_tensor_copy(NCTensor *dst, NCTensor *src) { nc_copy_any(dst, src); } // libnc.h:218

// libnc.h:219-220; mem_update shifts a memory onto itself (nncp.c:1212), which
// goes through a temporary
extern "C" void nc_tensor_copy_slice(NCTensor *dst, NCTensor *src, int axis, size_t dst_start,
                                     size_t dst_end, size_t src_start)
{
    if (dst == src && src_start > dst_start && dst_start < dst_end) {
        // A shift towards the front of the same tensor (the memory update): pieces no longer than
        // the shift distance do not overlap their own source, and copied front to back (the
        // stream keeps the order) each piece reads data no earlier piece has written - no
        // temporary, and every element moves once.
        const size_t dist = src_start - dst_start;
        for (size_t a = dst_start; a < dst_end; a += dist) {
            const size_t b = a + dist < dst_end ? a + dist : dst_end;
            NCTensor *dp = nc_slice_alias(dst, axis, a, b);
            NCTensor *sp = nc_slice_alias(src, axis, a + dist, b + dist);
            nc_copy_any(dp, sp);
            nc_free_tensor(dp);
            nc_free_tensor(sp);
        }
        return;
    }
    NCTensor *d = nc_slice_alias(dst, axis, dst_start, dst_end);
    NCTensor *s = nc_slice_alias(src, axis, src_start, src_start + (dst_end - dst_start));
    if (dst->buf == src->buf) {
        NCTensor *tmp = nc_alloc_like(s);
        nc_copy_any(tmp, s);
        nc_copy_any(d, tmp);
        nc_free_tensor(tmp);
    } else {
        nc_copy_any(d, s);
    }
    nc_free_tensor(d);
    nc_free_tensor(s);
}

extern "C" void nc_tensor_set_zero(NCTensor *y) // libnc.h:192
{
    size_t bytes = nc_numel(y) * nc_type_size(y->type);
    if (!bytes) return;
    nc_shadow_invalidate(y);
    if (nc_is_contig(y)) {
        if (y->dev->is_hip) { k_fill_bytes(nc_stream(y), nc_data(y), 0, (int64_t)bytes); nc_ctx(y)->launches++; }
        else memset(nc_data(y), 0, bytes);
    } else {
        NCTensor *z = nc_alloc(y->dev, y->type, y->n_dims, y->dims, true);
        nc_copy_any(y, z);
        nc_free_tensor(z);
    }
}

static void upload_values(NCTensor *y, const float *host);

extern "C" void nc_tensor_set_f32(NCTensor *y, float val) // libnc.h:194
{
    if (y->type == NC_TYPE_BF16 && nc_is_contig(y)) { // every element the same 16 bits
        size_t n = nc_numel(y);
        float *tmp = (float *)nc_malloc((n ? n : 1) * sizeof(float));
        for (size_t i = 0; i < n; i++) tmp[i] = val;
        upload_values(y, tmp);
        free(tmp);
        return;
    }
    if (!nc_is_contig(y) || y->type != NC_TYPE_F32) nc_fatal("set_f32: contiguous f32 or bf16 tensor expected");
    nc_shadow_invalidate(y);
    if (y->dev->is_hip) { k_fill_f32(nc_stream(y), nc_f32(y), val, (int64_t)nc_numel(y)); nc_ctx(y)->launches++; }
    else for (size_t i = 0; i < nc_numel(y); i++) nc_f32(y)[i] = val;
}

// libnc.h:206: host-side element write with conversion to the item type
// (I8 masks nncp.c:361, I32 tokens nncp.c:2998)
extern "C" void nc_set1_i32_2d(NCTensor *y, size_t i0, size_t i1, int32_t val)
{
    if (y->dev->is_hip) nc_fatal("nc_set1_i32_2d: host tensor expected");
    if (y->n_dims != 2 || i0 >= y->dims[0] || i1 >= y->dims[1]) nc_fatal("set1_i32_2d: index out of range");
    size_t off = y->off + i0 * y->strides[0] + i1 * y->strides[1];
    switch (y->type) {
    case NC_TYPE_I32: ((int32_t *)y->buf->ptr)[off] = val; break;
    case NC_TYPE_I8: ((int8_t *)y->buf->ptr)[off] = (int8_t)val; break;
    case NC_TYPE_U16: ((uint16_t *)y->buf->ptr)[off] = (uint16_t)val; break;
    case NC_TYPE_F32: ((float *)y->buf->ptr)[off] = (float)val; break;
    default: nc_fatal("set1_i32_2d: unsupported type");
    }
}

// libnc.h:226-227.  x is consumed.  Transfers are ordered on the stream and
// completed before returning, so the host buffer may be reused at once
// (process_block rewrites `input` every step, nncp.c:2998).
extern "C" NCTensor *nc_tensor_to_device(NCTensor *x, NCDevice *d)
{
    if (x->dev == d) return x;
    NCContext *m = d->ctx;
    if (x->node) nc_fatal("to_device: tensor carries a graph");
    x = nc_contig(x);
    NCTensor *y = nc_alloc(d, x->type, x->n_dims, x->dims, false);
    size_t bytes = nc_numel(x) * nc_type_size(x->type);
    if (bytes) {
        hip_check(hipMemcpyAsync(nc_data(y), nc_data(x), bytes,
                                 d->is_hip ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost, m->stream),
                  "hipMemcpyAsync");
        // An upload from a pinned host tensor that ends here (this was its last reference, so no
        // caller can write it again): the copy stays queued and the buffer is recycled after the
        // next wait.  Any other transfer is complete on return.
        if (d->is_hip && x->ref == 1 && x->buf->ref == 1) nc_mark_in_flight(x);
        else nc_stream_wait(m);
    }
    nc_free_tensor(x);
    return y;
}

extern "C" NCTensor *nc_tensor_to_cpu_device(NCTensor *x)
{
    NCContext *m = x->dev->ctx;
    if (!x->dev->is_hip) return nc_contig(x);
    // the graph of x stays with x's other references; the host copy has none
    NCTensor *c = nc_contig(x);
    NCTensor *y = nc_alloc(&m->cpu, c->type, c->n_dims, c->dims, false);
    size_t bytes = nc_numel(c) * nc_type_size(c->type);
    if (bytes) {
        hip_check(hipMemcpyAsync(nc_data(y), nc_data(c), bytes, hipMemcpyDeviceToHost, m->stream), "hipMemcpyAsync d2h");
        nc_stream_wait(m);
    }
    nc_free_tensor(c);
    return y;
}

extern "C" NCTensor *nc_tensor_to_cpu_device_queued(NCTensor *x) // nc_ext.h: valid after the next wait
{
    NCContext *m = x->dev->ctx;
    if (!x->dev->is_hip) return nc_contig(x);
    NCTensor *c = nc_contig(x);
    NCTensor *y = nc_alloc(&m->cpu, c->type, c->n_dims, c->dims, false);
    size_t bytes = nc_numel(c) * nc_type_size(c->type);
    if (bytes) {
        hip_check(hipMemcpyAsync(nc_data(y), nc_data(c), bytes, hipMemcpyDeviceToHost, m->stream), "hipMemcpyAsync d2h");
        nc_mark_in_flight(y);
    }
    nc_free_tensor(c);
    return y;
}

extern "C" float nc_get_scalar_f32(const NCTensor *x) // libnc.h:214 (synchronises)
{
    if (nc_numel(x) != 1 || x->type != NC_TYPE_F32) nc_fatal("get_scalar_f32: f32 scalar expected");
    if (!x->dev->is_hip) return nc_f32(x)[0];
    float v;
    NCContext *m = x->dev->ctx;
    hip_check(hipMemcpyAsync(&v, nc_data(x), sizeof(float), hipMemcpyDeviceToHost, m->stream), "hipMemcpyAsync");
    nc_stream_wait(m);
    return v;
}

extern "C" uint32_t nc_tensor_get_hash(const NCTensor *x) // libnc.h:177, FNV-1a of the bytes
{
    NCTensor *h = nc_tensor_to_cpu_device(nc_dup_tensor(x));
    const uint8_t *p = (const uint8_t *)nc_data(h);
    size_t n = nc_numel(h) * nc_type_size(h->type);
    uint32_t v = 2166136261u;
    for (size_t i = 0; i < n; i++) v = (v ^ p[i]) * 16777619u;
    nc_free_tensor(h);
    return v;
}

// ---- RNG (same build-defined xorwow stream as documented in nc_api.h) -------
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

extern "C" NCRNDState *nc_rnd_init(NCDevice *d, uint32_t seed)
{
    (void)d;
    NCRNDState *s = (NCRNDState *)nc_mallocz(sizeof(NCRNDState));
    s->x = 123456789 ^ seed; s->y = 362436069; s->z = 521288629;
    s->w = 88675123; s->v = 5783321; s->d = 6615241 + seed * 2654435761u;
    for (int i = 0; i < 16; i++) xorwow(s);
    return s;
}

extern "C" void nc_rnd_end(NCRNDState *s) { nc_free(s); }

static uint16_t host_bf16(float f) // nearest even; NaN stays a quiet NaN
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fff + ((u >> 16) & 1);
    return (uint16_t)(u >> 16);
}

static void upload_f32(NCTensor *y, const float *host);

// host values into contiguous f32 or bf16 tensor y (a bf16 tensor keeps their rounding)
static void upload_values(NCTensor *y, const float *host)
{
    nc_shadow_invalidate(y);
    if (y->type == NC_TYPE_F32) { upload_f32(y, host); return; }
    NCContext *m = y->dev->ctx;
    size_t n = nc_numel(y);
    if (!y->dev->is_hip) {
        for (size_t i = 0; i < n; i++) ((uint16_t *)nc_data(y))[i] = host_bf16(host[i]);
        return;
    }
    size_t cap;
    uint16_t *pin = (uint16_t *)m->host_pool.get((n ? n : 1) * sizeof(uint16_t), &cap);
    for (size_t i = 0; i < n; i++) pin[i] = host_bf16(host[i]);
    hip_check(hipMemcpyAsync(nc_data(y), pin, n * sizeof(uint16_t), hipMemcpyHostToDevice, m->stream), "hipMemcpyAsync h2d");
    nc_stream_wait(m);
    m->host_pool.put(pin, cap);
}

static void upload_f32(NCTensor *y, const float *host)
{
    NCContext *m = y->dev->ctx;
    size_t bytes = nc_numel(y) * sizeof(float);
    if (!y->dev->is_hip) { memcpy(nc_data(y), host, bytes); return; }
    hip_check(hipMemcpyAsync(nc_data(y), host, bytes, hipMemcpyHostToDevice, m->stream), "hipMemcpyAsync h2d");
    nc_stream_wait(m);
}

// libnc.h:197: uniform in [avg - range, avg + range); generated on the host in
// element order and uploaded (initialisation only)
extern "C" void nc_tensor_set_rnd_unif(NCTensor *y, float avg, float range, NCRNDState *rs)
{
    if (!nc_is_contig(y) || (y->type != NC_TYPE_F32 && y->type != NC_TYPE_BF16))
        nc_fatal("set_rnd_unif: contiguous f32 or bf16 tensor expected");
    size_t n = nc_numel(y);
    float *tmp = (float *)nc_malloc((n ? n : 1) * sizeof(float));
    for (size_t i = 0; i < n; i++) {
        float u = (float)(xorwow(rs) >> 8) * (1.0f / 16777216.0f);
        tmp[i] = avg + range * (2.0f * u - 1.0f);
    }
    upload_values(y, tmp);
    free(tmp);
}

extern "C" void nc_tensor_set_dropout(NCTensor *y, float prob, NCRNDState *rs) // libnc.h:201
{
    if (!nc_is_contig(y) || y->type != NC_TYPE_F32) nc_fatal("set_dropout: contiguous f32 tensor expected");
    nc_shadow_invalidate(y);
    size_t n = nc_numel(y);
    float *tmp = (float *)nc_malloc(n * sizeof(float)), keep = 1.0f / (1.0f - prob);
    for (size_t i = 0; i < n; i++) {
        float u = (float)(xorwow(rs) >> 8) * (1.0f / 16777216.0f);
        tmp[i] = u < prob ? 0.0f : keep;
    }
    upload_f32(y, tmp);
    free(tmp);
}

// ---- parameters (libnc.h:501-525) -------------------------------------------
extern "C" void nc_param_list_init(NCContext *m, NCParamList *pl)
{
    pl->ctx = m;
    pl->param_list.prev = pl->param_list.next = &pl->param_list;
    pl->add_graph = 1;
}

extern "C" NCParam *nc_new_param(NCParamList *pl, NCTensor **pval, const char *fmt, ...)
{
    char buf[128];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    NCParam *p = (NCParam *)nc_mallocz(sizeof(NCParam));
    p->pval = pval;
    p->name = strdup(buf);
    p->lr_mult = 1.0f;
    struct list_head *head = &pl->param_list, *el = &p->link;
    el->prev = head->prev; el->next = head; head->prev->next = el; head->prev = el;
    nc_set_param(*pval, p);
    return p;
}

extern "C" size_t nc_get_param_count(NCParamList *pl)
{
    size_t n = 0;
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next)
        n += nc_numel(*((NCParam *)el)->pval);
    return n;
}

// frees the list and the parameter tensors (nncp.c:522-550 never frees them)
extern "C" void nc_param_list_end(NCParamList *pl)
{
    struct list_head *el = pl->param_list.next, *next;
    for (; el != &pl->param_list; el = next) {
        NCParam *p = (NCParam *)el;
        next = el->next;
        nc_free_tensor(*p->pval);
        *p->pval = nullptr;
        free(p->name);
        nc_free(p);
    }
    pl->param_list.prev = pl->param_list.next = &pl->param_list;
}

// ---- optimiser (libnc.h:540-572; update rule defined in nc_api.h) ----------
struct SGDOptVarState {
    NCSGDOptState *opt;
    NCParam *param;
    NCTensor *m, *v, *g;
    // a bf16 parameter: the fp32 values the update works on (the parameter holds their
    // rounding), and the buffer version they were last taken from or written at
    NCTensor *master;
    uint64_t master_version;
    size_t n;
    bool has_grad;
};

struct NCSGDOptState {
    NCContext *ctx;
    SGDOptParams p;
    int64_t step;
    std::vector<SGDOptVarState *> vars;
    void *staging = nullptr; // pinned table of the previous update, recycled one update later
    size_t staging_cap = 0;
    uint64_t staging_stamp = 0;
};

extern "C" NCSGDOptState *nc_sgd_opt_init(NCContext *m, const SGDOptParams *p)
{
    NCSGDOptState *s = new NCSGDOptState();
    s->ctx = m; s->p = *p; s->step = 0;
    return s;
}

extern "C" void nc_sgd_opt_end(NCSGDOptState *s)
{
    nc_staging_retire(s->ctx, s->staging, s->staging_cap, s->staging_stamp);
    delete s;
}

// the master copy of a bf16 parameter starts as (and, after anyone else wrote the parameter,
// goes back to) the parameter's own value
static void master_from_param(SGDOptVarState *vs, NCTensor *w)
{
    NCContext *m = nc_ctx(w);
    if (nchip_widen_bf16(m->stream, (const uint16_t *)nc_data(w), nc_f32(vs->master), (int64_t)vs->n))
        nc_fatal("bf16 widening failed");
    m->launches++;
    vs->master_version = w->buf->version;
}

extern "C" void nc_sgd_opt_set_all(NCParamList *pl, NCSGDOptState *s)
{
    for (struct list_head *el = pl->param_list.next; el != &pl->param_list; el = el->next) {
        NCParam *p = (NCParam *)el;
        if (p->sgd_opt) {
            SGDOptVarState *vs = p->sgd_opt;
            auto &v = vs->opt->vars;
            for (size_t i = 0; i < v.size(); i++)
                if (v[i] == vs) { v.erase(v.begin() + i); break; }
            nc_free_tensor(vs->m); nc_free_tensor(vs->v); nc_free_tensor(vs->g); nc_free_tensor(vs->master);
            delete vs;
            p->sgd_opt = nullptr;
        }
        if (s) {
            NCTensor *w = *p->pval;
            if ((w->type != NC_TYPE_F32 && w->type != NC_TYPE_BF16) || !nc_is_contig(w))
                nc_fatal("optimiser: contiguous f32 or bf16 parameter expected");
            SGDOptVarState *vs = new SGDOptVarState();
            vs->opt = s; vs->param = p; vs->n = nc_numel(w); vs->has_grad = false;
            size_t n1 = vs->n;
            vs->master = nullptr;
            if (w->type == NC_TYPE_BF16) {
                need_dev(w, "optimiser on a bf16 parameter");
                vs->master = nc_alloc(w->dev, NC_TYPE_F32, 1, &n1, false);
                master_from_param(vs, w);
            }
            bool need_m = s->p.algo == SGD_OPT_ADAM && s->p.u.adam.beta1 != 0.0f;
            vs->m = need_m ? nc_alloc(w->dev, NC_TYPE_F32, 1, &n1, true) : nullptr;
            vs->v = (int)s->p.algo != SGD_OPT_BASIC ? nc_alloc(w->dev, NC_TYPE_F32, 1, &n1, true) : nullptr;
            vs->g = nullptr;
            s->vars.push_back(vs);
            p->sgd_opt = vs;
        }
    }
}

extern "C" void nc_sgd_opt_set_lr(NCSGDOptState *s, float lr) { s->p.lr = lr; }

// nc_ext.h: the moments of one parameter, out as a host copy and in from any f32 tensor
extern "C" NCTensor *nc_sgd_opt_get_state(NCParam *p, int which)
{
    SGDOptVarState *vs = p->sgd_opt;
    NCTensor *t = !vs ? nullptr : which == 0 ? vs->m : which == 1 ? vs->v : which == 2 ? vs->master : nullptr;
    if (t && which == 2 && vs->master_version != (*p->pval)->buf->version) master_from_param(vs, *p->pval);
    return t ? nc_tensor_to_cpu_device(nc_dup_tensor(t)) : nullptr;
}

extern "C" void nc_sgd_opt_set_state(NCParam *p, int which, const NCTensor *v)
{
    SGDOptVarState *vs = p->sgd_opt;
    NCTensor *t = !vs ? nullptr : which == 0 ? vs->m : which == 1 ? vs->v : which == 2 ? vs->master : nullptr;
    if (!t) nc_fatal("nc_sgd_opt_set_state: '%s' keeps no moment %d", p->name, which);
    if (which == 2) vs->master_version = (*p->pval)->buf->version; // (the caller sets the parameter to its rounding)
    if (v->type != NC_TYPE_F32 || nc_numel(v) != vs->n) nc_fatal("nc_sgd_opt_set_state: %zu f32 values expected for '%s'", vs->n, p->name);
    size_t n1 = vs->n;
    NCTensor *src = nc_reshape_view(nc_tensor_to_device(nc_dup_tensor(v), t->dev), 1, &n1);
    nc_tensor_copy(t, src);
    nc_free_tensor(src);
}

extern "C" int64_t nc_sgd_opt_get_step(NCSGDOptState *s) { return s->step; }
extern "C" void nc_sgd_opt_set_step(NCSGDOptState *s, int64_t step) { s->step = step; }

// libnc.h:563: the NCParamUpdateFunc nncp.c forwards to (nncp.c:1095); yg is
// consumed.  Only accumulates; nc_sgd_opt_update applies.
extern "C" void sgd_opt_update_var(void *opaque, NCTensor *yg, NCTensor *get_col_index)
{
    NCParam *p = (NCParam *)opaque;
    SGDOptVarState *vs = p->sgd_opt;
    if (get_col_index) nc_fatal("sparse gradients are not supported");
    if (!vs) { nc_free_tensor(yg); return; }
    yg = nc_contig(yg);
    if (nc_numel(yg) != vs->n) nc_fatal("gradient size mismatch for %s", p->name);
    if (!vs->has_grad) {
        nc_free_tensor(vs->g);
        vs->g = yg;
        vs->has_grad = true;
    } else {
        need_dev(yg, "sgd_opt_update_var");
        // a second gradient before the update (accumulation): with deferred weight gradients
        // yg, or the gradient kept from the first pass, may still wait for the grouped launch
        nc_flush_deferred(nc_ctx(yg));
        NCTensor *sum = nc_alloc_like(yg);
        k_binary_prefix(nc_stream(yg), KB_ADD, nc_f32(vs->g), nc_f32(yg), nc_f32(sum), (int64_t)vs->n, (int64_t)vs->n);
        nc_ctx(yg)->launches++;
        nc_free_tensor(vs->g);
        nc_free_tensor(yg);
        vs->g = sum;
    }
}

extern "C" void nc_sgd_opt_update(NCSGDOptState *s)
{
    const SGDOptParams *p = &s->p;
    float b1 = p->u.adam.beta1, b2 = p->u.adam.beta2;
    s->step++;
    float c1 = 1.0f / (1.0f - powf(b1, (float)s->step));
    float c2 = 1.0f / (1.0f - powf(b2, (float)s->step));
    // one launch over every parameter that received a gradient
    const int chunk = 8192;
    std::vector<NchipOptTensor> tab;
    std::vector<int> prefix(1, 0);
    for (SGDOptVarState *vs : s->vars) {
        if (!vs->has_grad) continue;
        NCTensor *w = *vs->param->pval;
        need_dev(w, "nc_sgd_opt_update");
        NchipOptTensor t;
        t.wide = nullptr;
        if (vs->master) {
            // bf16 parameter: update the master, leave its rounding in the parameter and, if
            // ops have taken the parameter as an operand before, in its f32 copy as well
            NCTensorBuffer *b = w->buf;
            if (vs->master_version != b->version) master_from_param(vs, w);
            t.w = nc_f32(vs->master);
            t.w16 = (uint16_t *)nc_data(w);
            const bool whole = b->wide && w->off == 0 && vs->n == b->elems;
            nc_shadow_invalidate(w);
            vs->master_version = b->version;
            if (whole) {
                t.wide = nc_f32(b->wide);
                b->wide_valid = true;
                b->wide->buf->sh_valid = true;
            }
        } else
        t.w = nc_f32(w);
        t.m = vs->m ? nc_f32(vs->m) : nullptr; // with beta1 == 0 the first moment is the gradient
        t.v = vs->v ? nc_f32(vs->v) : nullptr;
        t.g = nc_f32(vs->g);
        t.n = (int64_t)vs->n;
        t.lr = p->lr * vs->param->lr_mult;
        t.pad_ = 0;
        // matrices are operands of the bf16 products: their shadow is written with the update
        // (vectors - biases, gains - are not, and a shadow they may have is stale from here on)
        if (!vs->master) {
            t.w16 = (s->ctx->matmul_bf16 && w->n_dims >= 2) ? nc_shadow_for_write(s->ctx, w) : nullptr;
            if (!t.w16) nc_shadow_invalidate(w);
        }
        tab.push_back(t);
        prefix.push_back(prefix.back() + (int)((vs->n + chunk - 1) / chunk));
    }
    if (tab.empty()) return;
    NCContext *m = s->ctx;
    size_t tb = tab.size() * sizeof(NchipOptTensor), pb = prefix.size() * sizeof(int);
    size_t hcap, dcap;
    // pinned staging and device table; both go back to the pools only after
    // the stream has consumed them (the synchronize below is cheap here: the
    // host has nothing else to enqueue before the next step's token upload)
    uint8_t *host = (uint8_t *)m->host_pool.get(tb + pb, &hcap);
    uint8_t *dev = (uint8_t *)m->dev_pool.get(tb + pb, &dcap);
    memcpy(host, tab.data(), tb);
    memcpy(host + tb, prefix.data(), pb);
    hip_check(hipMemcpyAsync(dev, host, tb + pb, hipMemcpyHostToDevice, m->stream), "hipMemcpyAsync opt table");
    if (nchip_opt_update_multi(m->stream, (int)p->algo, (const NchipOptTensor *)dev, (const int *)(dev + tb),
                               (int)tab.size(), prefix.back(), chunk, b1, b2, p->u.adam.eps,
                               p->u.adam.gradient_clip, c1, c2))
        nc_fatal("optimiser update failed");
    m->launches++;
    // the copy must have read the staging buffer before it is recycled
    nc_staging_retire(m, s->staging, s->staging_cap, s->staging_stamp);
    s->staging = host; s->staging_cap = hcap; s->staging_stamp = m->sync_count;
    m->dev_pool.put(dev, dcap); // stream ordered: next user is enqueued after the kernel
    for (SGDOptVarState *vs : s->vars) {
        if (!vs->has_grad) continue;
        nc_free_tensor(vs->g);
        vs->g = nullptr;
        vs->has_grad = false;
    }
}

extern "C" float vec_sum_f32(const float *tab, size_t n) // libnc.h:600, fixed order
{
    float s = 0;
    for (size_t i = 0; i < n; i++) s += tab[i];
    return s;
}
