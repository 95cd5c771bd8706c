// Internal structures of libnc_hip: the libnc-compatible front end over the
// gfx950 kernels.  Host tensors exist only for staging (token ids, masks,
// probabilities copied back for the coder); every compute op requires device
// tensors and aborts otherwise - there is no CPU compute path in this library.
#ifndef NC_HIP_INTERNAL_H
#define NC_HIP_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <unordered_map>
#include <vector>
#include "../../include/nc_api.h"
#include "../../include/nc_ext.h"
#include "../../include/nchip_kernels.h"
#include "k_internal.h"

#define NC_MAX_SAVED 6
#define NC_SHAPE_ARGS 5

struct Shape {
    int nd = 0;
    size_t d[NC_N_DIMS_MAX] = { 0 };
};

// size-class caching allocator; a freed block is reusable at once because all
// work is ordered on one stream
struct Pool {
    bool device = false;
    std::unordered_map<size_t, std::vector<void *>> free_lists;
    std::vector<void *> all;
    int64_t bytes = 0;
    static size_t round_size(size_t n);
    void *get(size_t n, size_t *cap);
    void put(void *p, size_t cap);
    void release_all();
};

struct NCDevice {
    NCContext *ctx;
    bool is_hip;
};

// weight-gradient GEMM postponed to one grouped launch at the end of nc_backward
struct NCNode;
struct DeferredGemm {
    NCTensor *a, *b, *c;   // c (m x n) = alpha * (a (m x k) * b^T + a2 (m x k2) * b2^T), b is n x k
    NCTensor *a2, *b2;     // second use of the same weight (or NULL)
    int m, n, k, k2;
    float alpha;
    const NCNode *param;   // the parameter this gradient belongs to
};

// a gradient that is a sum of partial rows, summed with all others of its kind
// in one launch at the end of nc_backward
struct DeferredReduce {
    const float *src;
    float *dst;
    int64_t stride;
    int rows, n;
    const NCNode *param;
};
struct DeferredTmp { float *ptr; size_t cap; };
// A parameter used by several nodes of one graph (position vectors and biases tied over the
// layers): every use leaves its partial rows to a first-level sum into one row of `stage`
// (one row per use, in the order the backward pass reaches them), and a second-level sum
// over those rows gives the gradient tensor that the first use handed to the graph.
struct DeferredShared {
    const NCNode *param;
    float *stage;
    size_t cap;
    NCTensor *dst;
    int n, uses, next;
};

#define NC_BW_ARGS 8 // node arguments for which nc_backward offers the existing gradient

// a pinned table that was released while its upload may still be queued
struct StagingRetired { void *p; size_t cap; uint64_t stamp; };
// a weight matrix (m x k, rows contiguous) and its k-major copy (nc_keep_k_major_weight)
struct KMajorCopy { const float *src; size_t m, k; NCTensor *copy; };

struct NCContext {
    int nb_threads;
    NCDevice cpu, hip;
    bool hip_ready;
    hipStream_t stream;
    Pool dev_pool, host_pool;
    int matmul_bf16;
    int matmul_invariant; // forward products use the width-invariant GEMM class
    int bf16_copy_results; // bf16 mode: forward products also leave the bf16 copy of their result
    int64_t launches;
    int64_t shadow_casts; // bf16 shadows made by a cast of their own (not by the producing kernel)
    int64_t node_seq;
    int epoch;
    bool defer_wgrad;
    // set by nc_backward around each node: gradients its parents already hold
    // (bw_prev) and whether the node's backward folded them in (bw_used)
    NCTensor *bw_prev[NC_BW_ARGS];
    bool bw_used[NC_BW_ARGS];
    std::vector<DeferredShared> deferred_shared;
    std::vector<DeferredGemm> deferred;
    std::vector<DeferredReduce> deferred_red;
    std::vector<DeferredTmp> deferred_tmp;    // scratch the partial rows live in
    std::vector<NCTensor *> deferred_keep;    // destination tensors
    // pinned tables of the last grouped launches; each goes back to the pool
    // one flush later, and only once the stream has been waited for since its
    // upload was enqueued (nc_staging_retire)
    std::vector<StagingRetired> staging_retired; // released tables the stream may still read
    std::vector<KMajorCopy> k_major;             // copies the few-column products read instead of their weights
    void *grp_staging;
    size_t grp_staging_cap;
    uint64_t grp_staging_stamp;
    void *red_staging;
    size_t red_staging_cap;
    uint64_t red_staging_stamp;
    uint64_t sync_count; // completed waits for the stream (nc_stream_wait)
};

struct NCTensorBuffer {
    int ref;
    NCDevice *dev;
    void *ptr;
    size_t cap;
    // host buffers that a queued kernel reads or writes in place (nc_mark_in_flight): the
    // wait count when that kernel was enqueued, plus one (0 = never handed to a kernel)
    uint64_t in_flight;
    // bf16 shadow of a device f32 buffer (bf16-operand products only): the same elements in
    // the same order, rounded to nearest even.  Written either by the kernel that produces
    // the f32 values (norms, product epilogues, the optimiser) or by one cast the first time
    // a product asks for it; every later product reads 2 bytes per element instead of 4.
    // sh_valid says that sh holds the rounding of what the buffer holds NOW: whatever writes
    // into an existing buffer clears it (nc_shadow_invalidate).
    uint16_t *sh;
    size_t sh_cap;
    bool sh_valid;
    size_t elems; // elements the buffer was allocated for
    // A bf16 device buffer (NC_TYPE_BF16: 2 bytes per element are the tensor's value): `wide`
    // is the f32 copy of all its elements that kernels reading f32 use (made by one widening
    // pass when an op first takes the tensor as an operand, kept until the buffer goes;
    // wide_valid: it holds what the buffer holds NOW).  The copy's own shadow is the bf16
    // buffer itself (sh_alias: borrowed, never returned to the pool), so a bf16-operand
    // product reads the parameter's 2 bytes directly.
    NCTensor *wide;
    bool wide_valid;
    bool sh_alias;
    uint64_t version; // counts in-place writes (nc_shadow_invalidate): lets a holder of derived data notice them
};

struct NCTensor {
    int ref;
    NCDevice *dev;
    NCTensorBuffer *buf;
    size_t off; // in elements
    NCTypeEnum type;
    int n_dims;
    size_t dims[NC_N_DIMS_MAX];
    size_t strides[NC_N_DIMS_MAX]; // in elements
    NCNode *node;
};

enum NCOp {
    OP_PARAM, OP_ADD, OP_MUL, OP_MASKED_FILL, OP_UNARY, OP_GATED_SWISH, OP_LSTM_CLAMPED,
    OP_LERP, OP_RESHAPE, OP_REPEAT, OP_REDUCE_SUM, OP_SUM, OP_SLICE, OP_CONCAT, OP_PAD,
    OP_PERMUTE, OP_MATMUL, OP_GET_COL, OP_SOFT_MAX, OP_INDEXED_LOG, OP_NORM, OP_REL_SHIFT,
    OP_CONCAT_NODE, OP_ATTN, OP_LINEAR,
};

struct NCNode {
    int ref = 1;
    int op = 0;
    int n_args = 0;
    std::vector<NCNode *> parents;
    NCTensor *saved[NC_MAX_SAVED] = { nullptr };
    Shape arg_shape[NC_SHAPE_ARGS];
    int ia[8] = { 0 };
    float fa[4] = { 0 };
    std::vector<size_t> sizes;
    void *opaque = nullptr;
    NCContext *ctx = nullptr;
    // backward-walk state
    NCTensor *grad = nullptr;
    int pending = 0;
    int consumers = 0; // edges into this node in the current backward walk
    int mark = 0;
    // Partial row sums of the gradient this node is about to receive, left by the kernel that
    // produced that gradient (rows x n floats from the scratch pool): the node's backward step
    // takes its bias gradient from them instead of summing the gradient again.
    float *grad_rowsum = nullptr;
    size_t grad_rowsum_cap = 0;
    int grad_rowsum_rows = 0;
};

// nc_core.cpp
[[noreturn]] void nc_fatal(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void hip_check(hipError_t e, const char *what);
size_t nc_type_size(NCTypeEnum t);
size_t nc_numel(const NCTensor *x);
bool nc_is_contig(const NCTensor *x);
NCTensor *nc_alloc(NCDevice *d, NCTypeEnum t, int nd, const size_t *dims, bool zero);
NCTensor *nc_alloc_like(const NCTensor *x);
NCTensor *nc_view(const NCTensor *x);
NCTensor *nc_contig(NCTensor *x);                  // consumes
// What an op does to each operand (consumes): contiguous, and a bf16 tensor replaced by the
// same view of its buffer's f32 copy, carrying the same graph node (the gradient of a
// conversion is the identity, and it stays f32).
NCTensor *nc_operand(NCTensor *x);
void nc_copy_any(NCTensor *dst, const NCTensor *src); // strided, same device
void *nc_data(const NCTensor *x);
static inline float *nc_f32(const NCTensor *x)
{
    // (a 2-byte tensor taken for floats would be read out of bounds: ops widen first)
    if (x->type == NC_TYPE_BF16) nc_fatal("f32 access to a bf16 tensor");
    return (float *)nc_data(x);
}
void need_dev(const NCTensor *x, const char *op);
NCContext *nc_ctx(const NCTensor *x);
static inline hipStream_t nc_stream(const NCTensor *x) { return x->dev->ctx->stream; }
// the k-major copy kept for the m x k matrix at `a`, or NULL
const float *nc_k_major_of(const NCContext *m, const float *a, size_t rows, size_t k);
extern "C" void nc_forget_k_major_weights(NCContext *m);
float *nc_tmp_f32(NCContext *m, size_t n, size_t *cap); // pool scratch; give back with nc_tmp_free
void nc_tmp_free(NCContext *m, void *p, size_t cap);
NCTensor *nc_reshape_view(NCTensor *x, int nd, const size_t *dims); // consumes, no graph
// Every wait for the stream goes through here, so that sync_count tells whether
// work enqueued at an earlier moment has certainly finished.
void nc_stream_wait(NCContext *m);
// Gives a pinned table back to the host pool.  Its upload was enqueued when
// sync_count read `stamp`; if the stream has not been waited for since (a
// caller that enqueues step after step without reading anything back), waits
// first, so the buffer is never rewritten under a copy that has yet to run.
void nc_staging_retire(NCContext *m, void *p, size_t cap, uint64_t stamp);
// A kernel that was just enqueued reads or writes the pinned memory of host tensor x in
// place: when the last reference goes, the buffer returns to the pool only after the stream
// has been waited for (nc_free_tensor retires it like a pinned table).
void nc_mark_in_flight(NCTensor *x);

// bf16 shadows (nc_core.cpp).  nc_shadow_of: the shadow of contiguous f32 device tensor x,
// made by one cast of the whole buffer if it is not valid yet; NULL when x cannot have one
// (not f32, not on the device, not contiguous, offset not a multiple of 8 elements).
// nc_shadow_for_write: the place where a kernel that is about to write ALL of x's buffer may
// leave the shadow (marks it valid); NULL when x does not cover its buffer.
// nc_shadow_invalidate: x's buffer is about to be written in place.
const uint16_t *nc_shadow_of(NCContext *m, const NCTensor *x);
uint16_t *nc_shadow_for_write(NCContext *m, NCTensor *x);
void nc_shadow_invalidate(NCTensor *x);

// nc_autodiff.cpp
NCNode *nc_new_node(NCContext *m, int op, int n_args, NCTensor **args);
NCTensor *nc_finish(NCTensor *y, NCNode *n, NCTensor **args, int n_args);
void nc_node_backward(NCNode *nd, NCTensor *g, NCTensor **ga); // nc_ops.cpp
void nc_flush_deferred(NCContext *m);                          // nc_ops.cpp
bool nc_has_deferred(const NCContext *m, const NCNode *param);  // nc_ops.cpp
bool nc_can_defer_sum(const NCContext *m, const NCNode *parent); // nc_ops.cpp

#endif
