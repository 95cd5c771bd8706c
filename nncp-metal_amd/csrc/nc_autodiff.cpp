// Reverse-mode differentiation for libnc_hip: graph nodes, the node-surgery
// calls nncp.c uses to merge the per-timestep attention products into one
// batched backward (nncp.c:1111-1165), and nc_backward.
#include "nc_hip_internal.h"

extern "C" NCNode *nc_dup_node(const NCNode *n) // libnc.h:462
{
    if (n) ((NCNode *)n)->ref++;
    return (NCNode *)n;
}

extern "C" void nc_free_node(NCNode *n) // libnc.h:463, NULL accepted (nncp.c:1047)
{
    if (!n || --n->ref > 0) return;
    for (NCNode *p : n->parents) nc_free_node(p);
    for (int i = 0; i < NC_MAX_SAVED; i++) nc_free_tensor(n->saved[i]);
    nc_free_tensor(n->grad);
    delete n;
}

NCNode *nc_new_node(NCContext *m, int op, int n_args, NCTensor **args)
{
    NCNode *n = new NCNode();
    n->op = op;
    n->ctx = m;
    n->n_args = n_args;
    n->parents.assign(n_args, nullptr);
    for (int i = 0; i < n_args; i++) {
        if (!args || !args[i]) continue;
        n->parents[i] = nc_dup_node(args[i]->node);
        if (i < NC_SHAPE_ARGS) {
            n->arg_shape[i].nd = args[i]->n_dims;
            memcpy(n->arg_shape[i].d, args[i]->dims, sizeof(size_t) * args[i]->n_dims);
        }
    }
    return n;
}

// attach the node when any argument carries a graph, otherwise drop it
NCTensor *nc_finish(NCTensor *y, NCNode *n, NCTensor **args, int n_args)
{
    bool need = false;
    for (int i = 0; i < n_args; i++)
        if (args[i] && args[i]->node) need = true;
    if (need) {
        nc_free_node(y->node);
        y->node = n;
    } else {
        nc_free_node(n);
    }
    return y;
}

extern "C" NCTensor *nc_set_param(NCTensor *x, void *opaque) // libnc.h:457
{
    NCNode *n = nc_new_node(x->dev->ctx, OP_PARAM, 0, nullptr);
    n->opaque = opaque;
    nc_free_node(x->node);
    x->node = n;
    return x;
}

// libnc.h:470: x becomes the saved argument arg_index of n (nncp.c:827, 860)
extern "C" void nc_node_set_arg(NCNode *n, int arg_index, const NCTensor *x)
{
    if (arg_index < 0 || arg_index >= NC_MAX_SAVED) nc_fatal("node_set_arg: bad index");
    nc_free_tensor(n->saved[arg_index]);
    n->saved[arg_index] = nc_view(x);
}

// libnc.h:469: the gradient of argument arg_index of n goes to n1
// (nncp.c:1137, 1152)
extern "C" void nc_node_set_parent(NCNode *n, int arg_index, const NCNode *n1)
{
    if (arg_index < 0 || arg_index >= n->n_args) nc_fatal("node_set_parent: bad index");
    nc_free_node(n->parents[arg_index]);
    n->parents[arg_index] = nc_dup_node(n1);
}

// libnc.h:466: synthetic node whose incoming gradient is split along `axis`
// into pieces of tab_size[] for inputs[] (nncp.c:1128-1131)
extern "C" NCNode *nc_concat_node(NCContext *m, NCNode **inputs, int count, int axis,
                                  const size_t *tab_size)
{
    NCNode *n = nc_new_node(m, OP_CONCAT_NODE, count, nullptr);
    for (int i = 0; i < count; i++) n->parents[i] = nc_dup_node(inputs[i]);
    n->ia[0] = axis;
    n->sizes.assign(tab_size, tab_size + count);
    return n;
}

// libnc.h:468 / libnc.h:464: permissions to merge sibling backward passes;
// they carry no semantics of their own
extern "C" void nc_concat_optimization(NCContext *m, NCNode **nodes, int count)
{
    (void)m; (void)nodes; (void)count;
}

extern "C" void nc_combine_nodes(NCContext *m, NCNode **tab, int count, int axis, int elem_size,
                                 const size_t *tab_elem_size)
{
    (void)m; (void)tab; (void)count; (void)axis; (void)elem_size; (void)tab_elem_size;
}

static void count_edges(NCNode *root, int epoch)
{
    std::vector<NCNode *> stack;
    root->mark = epoch;
    root->pending = 0;
    stack.push_back(root);
    while (!stack.empty()) {
        NCNode *c = stack.back();
        stack.pop_back();
        for (NCNode *p : c->parents) {
            if (!p) continue;
            if (p->mark != epoch) {
                p->mark = epoch;
                p->pending = 0;
                stack.push_back(p);
            }
            p->pending++;
            p->consumers = p->pending;
        }
    }
}

static void accumulate(NCNode *p, NCTensor *g)
{
    g = nc_contig(g);
    if (!p->grad) { p->grad = g; return; }
    // a postponed weight gradient holds no data yet: run it before summing
    if (p->op == OP_PARAM && nc_has_deferred(p->ctx, p)) nc_flush_deferred(p->ctx);
    size_t n = nc_numel(g);
    if (n != nc_numel(p->grad))
        nc_fatal("backward: gradient size mismatch at op %d (%zu vs %zu)", p->op, n, nc_numel(p->grad));
    NCTensor *sum = nc_alloc_like(p->grad);
    k_binary_prefix(nc_stream(g), KB_ADD, nc_f32(p->grad), nc_f32(g), nc_f32(sum), (int64_t)n, (int64_t)n);
    nc_ctx(g)->launches++;
    nc_free_tensor(p->grad);
    nc_free_tensor(g);
    p->grad = sum;
}

// libnc.h:480-481: x borrowed, grad consumed.  Nodes are processed once all
// their consumers have delivered (Kahn order, LIFO among ready nodes), so the
// walk and every gradient sum run in an order fixed by how the graph was
// built.  A parameter used several times (tied w_r / b_r, nncp.c:742-760) is
// reported once with the summed gradient.
extern "C" void nc_backward(const NCTensor *x, NCTensor *grad, NCParamUpdateFunc *cb, int flags)
{
    (void)flags;
    if (!x->node) { nc_free_tensor(grad); return; }
    NCContext *m = x->dev->ctx;
    int epoch = ++m->epoch;
    count_edges(x->node, epoch);
    std::vector<NCNode *> ready;
    if (grad->dev != x->dev) grad = nc_tensor_to_device(grad, x->dev);
    x->node->grad = grad;
    ready.push_back(x->node);
    while (!ready.empty()) {
        NCNode *nd = ready.back();
        ready.pop_back();
        nc_dup_node(nd); // keep alive while its gradient is processed
        NCTensor *g = nd->grad;
        nd->grad = nullptr;
        if (nd->op == OP_PARAM) {
            if (g) {
                if (cb) cb(nd->opaque, g, nullptr);
                else nc_free_tensor(g);
            }
            nc_free_node(nd);
            continue;
        }
        std::vector<NCTensor *> ga(nd->n_args > 0 ? nd->n_args : 1, nullptr);
        // offer the gradients the parents already hold: a backward kernel that
        // can add one in its epilogue returns the finished sum (existing + new,
        // the same two terms accumulate() would add)
        for (int i = 0; i < NC_BW_ARGS; i++) {
            NCNode *p = i < nd->n_args ? nd->parents[i] : nullptr;
            bool again = false; // the same parent twice: only the first slot may take it
            for (int j = 0; j < i && p; j++) again |= nd->parents[j] == p;
            m->bw_prev[i] = (p && !again && p->op != OP_PARAM) ? p->grad : nullptr;
            m->bw_used[i] = false;
        }
        if (g) nc_node_backward(nd, g, ga.data());
        for (int i = 0; i < nd->n_args; i++) {
            NCNode *p = nd->parents[i];
            if (!p) { nc_free_tensor(ga[i]); continue; }
            if (ga[i]) {
                if (i < NC_BW_ARGS && m->bw_used[i]) {
                    nc_free_tensor(p->grad);
                    p->grad = ga[i];
                } else {
                    accumulate(p, ga[i]);
                }
            }
            if (--p->pending == 0) ready.push_back(p);
        }
        for (int i = 0; i < NC_BW_ARGS; i++) { m->bw_prev[i] = nullptr; m->bw_used[i] = false; }
        nc_free_tensor(g);
        nc_free_node(nd);
    }
    nc_flush_deferred(m);
}
