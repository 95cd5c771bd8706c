"""Op-level cases shared by the CPU tests (checker vs numpy / finite
differences) and the GPU tests (product vs checker).  Each case builds a small
graph through the C ABI from float inputs that are all registered as
parameters, and has an independent float64 numpy restatement.

numpy shapes are the reverse of libnc dims (see nputil.py)."""
import ctypes as C

import numpy as np

import nputil as U

_P = C.c_void_p


class Case:
    def __init__(self, name, shapes, build, ref, scale=1.0, fd=True):
        self.name, self.shapes, self.build, self.ref = name, shapes, build, ref
        self.scale, self.fd = scale, fd

    def inputs(self, rng):
        return [(rng.standard_normal(s) * self.scale).astype(np.float32) for s in self.shapes]

    def run(self, nc, arrays, weight):
        """Returns (output ndarray, [grad ndarray per input]) for
        loss = sum(output * weight)."""
        holders = [nc.param(a, "p%d" % i) for i, a in enumerate(arrays)]
        y = self.build(nc, *[nc.dup(h.value) for h, _ in holders])
        out = nc.numpy(y)
        w = nc.tensor(weight.astype(np.float32))
        loss = nc.nc_sum(nc.nc_mul(y, w))
        grads = nc.backward(loss)
        nc.free(loss)
        gl = [grads.get(p, np.zeros_like(a)) for (h, p), a in zip(holders, arrays)]
        return out, gl


def _arr(nc, lst):
    return (_P * len(lst))(*lst)


def _i32(nc, a):
    return nc.tensor(np.asarray(a, dtype=np.int32))


# ---- builders ---------------------------------------------------------------
def _mm(ta, tb):
    def build(nc, a, b):
        return nc.nc_matmul_add(a, b, None, ta, tb, 0.5)

    def ref(a, b):
        # numpy (..., c, r) holds a column-major r x c matrix: math matrix = swapaxes
        A = np.swapaxes(a, -1, -2)
        B = np.swapaxes(b, -1, -2)
        if ta:
            A = np.swapaxes(A, -1, -2)
        if tb:
            B = np.swapaxes(B, -1, -2)
        return np.swapaxes(0.5 * (A @ B), -1, -2)
    return build, ref


def _mm_shapes(ta, tb, m, k, n, batch=()):
    a = batch + ((m, k) if ta else (k, m))
    b = batch + ((k, n) if tb else (n, k))
    return [a, b]


def _perm_build(nc, x):
    return nc.nc_permute_4d(x, 0, 3, 1, 2)


def _perm_ref(x):
    # libnc result axis i = x axis axis[i]; numpy axes are reversed
    nd = 4
    ax = [0, 3, 1, 2]
    np_ax = [nd - 1 - ax[nd - 1 - j] for j in range(nd)]
    return np.transpose(x, np_ax)


def _pad_ref(left, lop, right, rop):
    def ref(x):
        n = x.shape[-1]
        out = np.zeros(x.shape[:-1] + (n + left + right,))
        for i in range(n + left + right):
            s = i - left
            if s < 0:
                if lop != 1:
                    continue
                s = 0
            elif s >= n:
                if rop != 1:
                    continue
                s = n - 1
            out[..., i] += x[..., s]
        if left < 0 and lop == 1:
            out[..., 0] += x[..., :-left].sum(axis=-1)
        if right < 0 and rop == 1:
            out[..., -1] += x[..., n + right:].sum(axis=-1)
        return out
    return ref


def _rel_shift_ref(pos, mult):
    def ref(x):
        out = np.zeros_like(x)
        n0, n1 = x.shape[-1], x.shape[-2]
        for i in range(n1):
            s = pos + i * mult
            for j in range(n0):
                if 0 <= j - s < n0:
                    out[..., i, j] = x[..., i, j - s]
        return out
    return ref


_MASK = (np.arange(6)[None, :] > np.arange(4)[:, None] + 2).astype(np.int8)  # numpy (T=4,K=6)


def _split_build(nc, x):
    tab = (_P * 2)()
    nc.nc_split(tab, x, 2, None, 0)
    return nc.nc_mul(nc.nc_gelu(tab[0]), tab[1])


def _concat_build(nc, a, b):
    return nc.nc_concat(_arr(nc, [a, b]), 2, 2)


def _reduce_build(nc, y0, x):
    return nc.nc_reduce_sum(y0, x, 2)


_IDX = np.array([3, 0, 3, 5, 1], dtype=np.int32)
_TGT = np.array([[1, 0, 2], [3, 3, 0]], dtype=np.int32)  # numpy (T=2,B=3)


def _nll_build(nc, x):
    return nc.nc_indexed_log(nc.nc_soft_max(x), _i32(nc, _TGT))


def _nll_ref(x):
    p = U.softmax(x)
    T, B, V = x.shape
    return np.log(np.array([[p[t, b, _TGT[t, b]] for b in range(B)] for t in range(T)]))


def _nll_unfused_build(nc, x):
    # the seq_eval form: softmax outputs are concatenated before the log
    # (nncp.c:1160-1170), so the fused-gradient shortcut does not apply
    p = nc.nc_soft_max(x)
    a = nc.nc_slice(nc.dup(p), 2, 0, 1)
    b = nc.nc_slice(p, 2, 1, 2)
    return nc.nc_indexed_log(nc.nc_concat(_arr(nc, [a, b]), 2, 2), _i32(nc, _TGT))


def _ln_affine(avg):
    def build(nc, x, w, b):
        return nc.nc_fused_layer_norm(x, w, b, 1e-5, avg)

    def ref(x, w, b):
        return U.layer_norm(x, 1e-5, avg) * w + b
    return build, ref


def _ln_unfused_build(nc, x, w, b):
    # layer_norm() of nncp.c:279-288
    return nc.nc_add(nc.nc_mul(nc.nc_layer_norm(x, 1e-5), w), b)


def _attn(H, dk, attn_len, use_wr, use_br, use_mem):
    def build(nc, q, kv, kvm, w_r, b_r):
        if not use_mem:
            nc.free(kvm)
        if not use_wr:
            nc.free(w_r)
        if not use_br:
            nc.free(b_r)
        return nc.nc_relpos_attention(q, kv, kvm if use_mem else None,
                                      w_r if use_wr else None, b_r if use_br else None,
                                      H, dk, attn_len, 3.0)

    def ref(q, kv, kvm, w_r, b_r):
        return U.relpos_attention(q, kv, kvm if use_mem else None, w_r if use_wr else None,
                                  b_r if use_br else None, H, dk, attn_len, 3.0)
    return build, ref


def _attn_shapes(H, dk, dv, B, T, M, d_pos, use_mem=True):
    K = (M if use_mem else 0) + T
    return [(T, B, H * dk), (T, B, H * dk + H * dv), (M, B, H * dk + H * dv),
            (H, d_pos, dk), (H, K)]


def unfused_attention(nc, q, kv, kvm, w_r, b_r, H, dk, attn_len, b_r_scale):
    """The op sequence of trf_eval for output_index < 0 (nncp.c:663-800,
    869), written with the same nc_* calls.  q (H*dk,B,T), kv, kvm as in
    nc_relpos_attention.  Returns (H*dv, B, T)."""
    HDk = H * dk
    dq = nc.dims(q)
    B, T = dq[1], dq[2]
    dkv = nc.dims(kv)
    HDv = dkv[0] - HDk
    dv = HDv // H
    M = nc.dims(kvm)[2]
    K = M + T
    d_pos = nc.dims(w_r)[1]

    def split_head(x):  # nncp.c:554-565
        d = nc.dims(x)
        x = nc.nc_reshape_4d(x, d[0] // H, H, d[1], d[2])
        return nc.nc_permute_4d(x, 0, 3, 1, 2)

    key = nc.nc_slice(nc.dup(kv), 0, 0, HDk)
    value = nc.nc_slice(kv, 0, HDk, HDk + HDv)
    key0 = nc.nc_slice(nc.dup(kvm), 0, 0, HDk)
    value0 = nc.nc_slice(kvm, 0, HDk, HDk + HDv)
    key = nc.nc_concat(_arr(nc, [key0, key]), 2, 2)
    value = nc.nc_concat(_arr(nc, [value0, value]), 2, 2)
    key, query, value = split_head(key), split_head(q), split_head(value)
    tmp_w_r = nc.nc_repeat_1d(w_r, B)
    b = nc.nc_mul(b_r, nc.nc_new_f32(nc.dev, float(b_r_scale)))
    b = nc.nc_repeat_2d(b, T, B)
    tmp_b_r = nc.nc_permute_4d(b, 0, 2, 1, 3)
    t0 = nc.nc_matmul_add(key, nc.dup(query), None, 1, 0, 1.0)
    rd = nc.nc_matmul_add(tmp_w_r, query, None, 1, 0, 1.0)
    rd = nc.nc_pad(rd, K - d_pos, 1, 0, 0)
    rd = nc.nc_add(rd, tmp_b_r)
    rd = nc.nc_rel_shift(rd, -(T - 1), 1)
    t0 = nc.nc_add(rd, t0)
    t0 = nc.nc_mul(t0, nc.nc_new_f32(nc.dev, float(np.float32(1.0) / np.sqrt(np.float32(dk)))))
    mask = np.zeros((T, K), dtype=np.int8)
    for i in range(T):
        for j in range(K):
            pos = i + M - j
            mask[i, j] = not (0 <= pos < attn_len)
    t0 = nc.nc_masked_fill(t0, nc.tensor(mask), -np.inf, 0)
    t0 = nc.nc_soft_max(t0)
    t0 = nc.nc_matmul(value, t0)
    t0 = nc.nc_permute_4d(t0, 0, 2, 3, 1)  # concat_head, nncp.c:569-579
    return nc.nc_reshape_3d(t0, dv * H, B, T)


def _attn_unfused(H, dk, attn_len):
    def build(nc, q, kv, kvm, w_r, b_r):
        return unfused_attention(nc, q, kv, kvm, w_r, b_r, H, dk, attn_len, 3.0)
    return build


CASES = []


def _add(*a, **k):
    CASES.append(Case(*a, **k))


for _ta in (0, 1):
    for _tb in (0, 1):
        _b, _r = _mm(_ta, _tb)
        _add("matmul_%d%d" % (_ta, _tb), _mm_shapes(_ta, _tb, 7, 5, 3), _b, _r)
        _add("matmul_batched_%d%d" % (_ta, _tb), _mm_shapes(_ta, _tb, 4, 6, 5, (2, 3)), _b, _r)
_add("matmul_2d_nd", [(5, 7), (2, 3, 5)], lambda nc, a, b: nc.nc_matmul(a, b),
     lambda a, b: b @ a)
_add("add_same", [(3, 4), (3, 4)], lambda nc, a, b: nc.nc_add(a, b), lambda a, b: a + b)
_add("add_vec", [(3, 4), (4,)], lambda nc, a, b: nc.nc_add(a, b), lambda a, b: a + b)
_add("mul_vec", [(3, 4), (4,)], lambda nc, a, b: nc.nc_mul(a, b), lambda a, b: a * b)
_add("mul_scalar", [(3, 4), ()], lambda nc, a, b: nc.nc_mul(a, b), lambda a, b: a * b)
_add("add_bcast_mid", [(2, 3, 4, 5), (2, 3, 1, 5)], lambda nc, a, b: nc.nc_add(a, b),
     lambda a, b: a + b)
_add("mul_bcast_mid", [(2, 3, 4, 5), (2, 3, 1, 5)], lambda nc, a, b: nc.nc_mul(a, b),
     lambda a, b: a * b)
_add("masked_fill", [(2, 3, 4, 6)],
     lambda nc, x: nc.nc_masked_fill(x, nc.tensor(_MASK), -7.0, 0),
     lambda x: np.where(_MASK != 0, -7.0, x))
_add("masked_fill_inv", [(2, 3, 4, 6)],
     lambda nc, x: nc.nc_masked_fill(x, nc.tensor(_MASK), 2.0, 1),
     lambda x: np.where(_MASK == 0, 2.0, x))
_add("sigmoid", [(3, 5)], lambda nc, x: nc.nc_sigmoid(x), lambda x: 1 / (1 + np.exp(-x)))
_add("tanh", [(3, 5)], lambda nc, x: nc.nc_tanh(x), np.tanh)
_add("relu", [(3, 5)], lambda nc, x: nc.nc_relu(x), lambda x: np.maximum(x, 0))
_add("gelu", [(3, 5)], lambda nc, x: nc.nc_gelu(x), U.gelu, scale=2.0)
_add("gated_swish", [(3, 5), (3, 5)], lambda nc, g, x: nc.nc_gated_swish(g, x, 1.0),
     lambda g, x: g * x / (1 + np.exp(-x)))
_add("lerp", [(3, 5), (3, 5), (3, 5)], lambda nc, a, b, t: nc.nc_lerp(a, b, t),
     lambda a, b, t: a * (1 - t) + b * t)
_add("lstm_clamped", [(3, 5)] * 4, lambda nc, c, i, f, g: nc.nc_lstm_clamped(c, i, f, g),
     lambda c, i, f, g: c * f + np.minimum(1 - f, g) * i)
_add("reshape", [(4, 6)], lambda nc, x: nc.nc_reshape_3d(x, 2, 3, 4),
     lambda x: x.reshape(4, 3, 2))
_add("repeat_1d", [(2, 3)], lambda nc, x: nc.nc_repeat_1d(x, 4),
     lambda x: np.broadcast_to(x, (4, 2, 3)))
_add("repeat_2d", [(2, 3)], lambda nc, x: nc.nc_repeat_2d(x, 4, 5),
     lambda x: np.broadcast_to(x, (5, 4, 2, 3)))
_add("reduce_sum", [(3, 4), (5, 2, 3, 4)], _reduce_build,
     lambda y0, x: y0 + x.sum(axis=(0, 1)))
_add("sum", [(3, 4)], lambda nc, x: nc.nc_sum(x), lambda x: x.sum())
_add("slice_axis0", [(3, 8)], lambda nc, x: nc.nc_slice(x, 0, 2, 7), lambda x: x[:, 2:7])
_add("slice_axis2", [(5, 3, 4)], lambda nc, x: nc.nc_slice(x, 2, 1, 4), lambda x: x[1:4])
_add("concat_axis2", [(2, 3, 4), (5, 3, 4)], _concat_build,
     lambda a, b: np.concatenate([a, b], axis=0))
_add("split_geglu", [(3, 8)], _split_build, lambda x: U.gelu(x[:, :4]) * x[:, 4:])
_add("pad_dup_left", [(2, 3, 4)], lambda nc, x: nc.nc_pad(x, 3, 1, 0, 0), _pad_ref(3, 1, 0, 0))
_add("pad_zero_both", [(2, 3, 4)], lambda nc, x: nc.nc_pad(x, 2, 0, 1, 0), _pad_ref(2, 0, 1, 0))
_add("pad_dup_right", [(2, 3, 4)], lambda nc, x: nc.nc_pad(x, 0, 0, 2, 1), _pad_ref(0, 0, 2, 1))
_add("trim_sum_left", [(2, 3, 6)], lambda nc, x: nc.nc_pad(x, -2, 1, 0, 0), _pad_ref(-2, 1, 0, 0))
_add("trim_normal", [(2, 3, 6)], lambda nc, x: nc.nc_pad(x, -2, 0, -1, 0), _pad_ref(-2, 0, -1, 0))
_add("permute_0312", [(2, 3, 4, 5)], _perm_build, _perm_ref)
_add("permute_0231", [(2, 3, 4, 5)], lambda nc, x: nc.nc_permute_4d(x, 0, 2, 3, 1),
     lambda x: np.transpose(x, [3 - [0, 2, 3, 1][3 - j] for j in range(4)]))
_add("rel_shift_neg", [(2, 4, 6)], lambda nc, x: nc.nc_rel_shift(x, -3, 1), _rel_shift_ref(-3, 1))
_add("rel_shift_pos", [(2, 4, 6)], lambda nc, x: nc.nc_rel_shift(x, 1, -1), _rel_shift_ref(1, -1))
_add("get_col", [(6, 4)], lambda nc, w: nc.nc_get_col(w, _i32(nc, _IDX)), lambda w: w[_IDX])
_add("soft_max", [(2, 3, 7)], lambda nc, x: nc.nc_soft_max(x), U.softmax, scale=2.0)
_add("nll_fused", [(2, 3, 5)], _nll_build, _nll_ref)
_add("nll_unfused", [(2, 3, 5)], _nll_unfused_build, _nll_ref)
_add("layer_norm", [(3, 16)], lambda nc, x: nc.nc_layer_norm(x, 1e-5), U.layer_norm)
_add("rms_norm", [(3, 16)], lambda nc, x: nc.nc_rms_norm(x, 1e-5),
     lambda x: U.layer_norm(x, 1e-5, False))
for _avg in (1, 0):
    _b, _r = _ln_affine(_avg)
    _add("fused_ln_avg%d" % _avg, [(3, 16), (16,), (16,)], _b, _r)
_add("ln_unfused_affine", [(3, 16), (16,), (16,)], _ln_unfused_build, _ln_affine(1)[1])
_add("linear_gelu", [(5, 7), (3, 5), (7,)],
     lambda nc, w, x, b: nc.nc_linear(w, x, b, 1), lambda w, x, b: U.gelu(x @ w + b))
_add("linear_nobias", [(5, 7), (3, 5)],
     lambda nc, w, x: nc.nc_linear(w, x, None, 0), lambda w, x: x @ w)
_add("linear_add_gelu", [(5, 7), (3, 5), (7,), (3, 7)],
     lambda nc, w, x, b, r: nc.nc_linear_add(w, x, b, 1, r), lambda w, x, b, r: U.gelu(x @ w + b) + r)
_add("linear_add_nobias", [(5, 7), (3, 5), (3, 7)],
     lambda nc, w, x, r: nc.nc_linear_add(w, x, None, 0, r), lambda w, x, r: x @ w + r)
_add("matmul_add_residual", [(5, 7), (3, 5), (3, 7)],
     lambda nc, w, x, r: nc.nc_matmul_add(w, x, r, 0, 0, 0.5), lambda w, x, r: 0.5 * (x @ w) + r)
_add("mlp_gelu_linear", [(5, 7), (3, 5), (7,), (7, 4), (4,)],
     lambda nc, w1, x, b1, w2, b2: nc.nc_linear(w2, nc.nc_linear(w1, x, b1, 1), b2, 0),
     lambda w1, x, b1, w2, b2: U.gelu(x @ w1 + b1) @ w2 + b2)
_add("mlp_relu_linear_add", [(5, 7), (3, 5), (7, 4), (3, 4)],
     lambda nc, w1, x, w2, r: nc.nc_linear_add(w2, nc.nc_linear(w1, x, None, 2), None, 0, r),
     lambda w1, x, w2, r: np.maximum(x @ w1, 0) @ w2 + r)
_add("linear_relu", [(5, 7), (3, 5), (7,)],
     lambda nc, w, x, b: nc.nc_linear(w, x, b, 2), lambda w, x, b: np.maximum(x @ w + b, 0))

# attention: H=2, dk=4, dv=3, B=2, T=5, M=3, d_pos=6, K=8
_ATT = dict(H=2, dk=4, dv=3, B=2, T=5, M=3, d_pos=6)
_b, _r = _attn(2, 4, 8, True, True, True)
_add("attn_full", _attn_shapes(**_ATT), _b, _r, scale=0.7)
_b, _r = _attn(2, 4, 4, True, True, True)
_add("attn_window4", _attn_shapes(**_ATT), _b, _r, scale=0.7)
_b, _r = _attn(2, 4, 8, False, False, True)
_add("attn_plain", _attn_shapes(**_ATT), _b, _r, scale=0.7)
_b, _r = _attn(2, 4, 5, True, True, False)
_add("attn_nomem", _attn_shapes(**dict(_ATT, d_pos=4), use_mem=False), _b, _r, scale=0.7)
_add("attn_unfused_seq", _attn_shapes(**_ATT), _attn_unfused(2, 4, 8),
     _attn(2, 4, 8, True, True, True)[1], scale=0.7)
_add("attn_unfused_window", _attn_shapes(**_ATT), _attn_unfused(2, 4, 4),
     _attn(2, 4, 4, True, True, True)[1], scale=0.7)

BY_NAME = {c.name: c for c in CASES}
