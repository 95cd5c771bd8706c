"""Test infrastructure: every op family of the tensor ABI at seeded random shapes (sizes drawn
around the kernels' block, wavefront and vector-width boundaries, broadcast forms of every
kind), forward and backward, through the CPU build of the product kernels (each device buffer
ends at a guard page) against the CPU checker and, forward, against numpy.
Usage: fuzz_ops.py <seed> <cases>, library path in NNCP_TEST_HIP_LIB."""
import ctypes as C, os, sys, time, faulthandler
import numpy as np
faulthandler.enable()
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), '..'))
from conftest import load_pkg, REF_LIB
import cases as K
import nputil as U

B = load_pkg().binding
ref = B.NC(REF_LIB, use_device=False)
emu = B.NC(os.environ['NNCP_TEST_HIP_LIB'], use_device=True)
_P = C.c_void_p
SIZES = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 255, 257]
SMALL = [1, 2, 3, 4, 5, 7, 8, 9]
MAX_ELEMS = 12000


def shape(rng, nd, cap=MAX_ELEMS):
    """nd dims; the last numpy axis (libnc axis 0) may be large, the product stays under cap."""
    while True:
        s = [int(rng.choice(SMALL)) for _ in range(nd - 1)] + [int(rng.choice(SIZES))]
        if rng.integers(4) == 0 and nd > 1:
            s[int(rng.integers(nd - 1))] = int(rng.choice(SIZES))
        if int(np.prod(s)) <= cap:
            return tuple(s)


def np_axes(ax):
    """libnc permutation (result axis i = source axis ax[i]) as a numpy transpose."""
    nd = len(ax)
    return [nd - 1 - ax[nd - 1 - j] for j in range(nd)]


def g_binary(rng):
    nd = int(rng.integers(1, 5))
    a = shape(rng, nd)
    mode = int(rng.integers(6))
    if mode == 0:
        b = a
    elif mode == 1:                      # b covers the leading libnc axes
        b = a[nd - int(rng.integers(1, nd + 1)):]
    elif mode == 2:
        b = ()
    elif mode == 3:                      # 1s anywhere in b
        b = tuple(1 if rng.integers(2) else d for d in a)
    elif mode == 4:                      # 1s on both sides
        full = a
        a = tuple(1 if rng.integers(3) == 0 else d for d in full)
        b = tuple(d if x == 1 or rng.integers(2) else 1 for d, x in zip(full, a))
    else:                                # b with more axes than a
        b = a
        a = a[int(rng.integers(0, nd)):]
    if rng.integers(2):
        a, b = b, a
    if rng.integers(2):
        return "add", [a, b], lambda nc, x, y: nc.nc_add(x, y), lambda x, y: x + y, {}
    return "mul", [a, b], lambda nc, x, y: nc.nc_mul(x, y), lambda x, y: x * y, {}


def g_unary(rng):
    s = shape(rng, int(rng.integers(1, 4)))
    name, ref_fn = [("sigmoid", lambda x: 1 / (1 + np.exp(-x))), ("tanh", np.tanh),
                    ("relu", lambda x: np.maximum(x, 0)), ("gelu", U.gelu)][int(rng.integers(4))]
    return name, [s], lambda nc, x: getattr(nc, "nc_" + name)(x), ref_fn, dict(scale=2.0)


def g_ternary(rng):
    s = shape(rng, int(rng.integers(1, 4)))
    k = int(rng.integers(3))
    if k == 0:
        beta = float(rng.choice([1.0, 0.5, 1.702]))
        return ("gated_swish", [s, s], lambda nc, g, x: nc.nc_gated_swish(g, x, beta),
                lambda g, x: g * x / (1 + np.exp(-beta * x)), {})
    if k == 1:
        return ("lerp", [s, s, s], lambda nc, a, b, t: nc.nc_lerp(a, b, t),
                lambda a, b, t: a * (1 - t) + b * t, {})
    return ("lstm_clamped", [s] * 4, lambda nc, c, i, f, g: nc.nc_lstm_clamped(c, i, f, g),
            lambda c, i, f, g: c * f + np.minimum(1 - f, g) * i, {})


def g_reduce(rng):
    if rng.integers(3) == 0:
        s = shape(rng, int(rng.integers(1, 4)), 60000 if rng.integers(3) == 0 else MAX_ELEMS)
        return "sum", [s], lambda nc, x: nc.nc_sum(x), lambda x: x.sum(), {}
    keep = int(rng.integers(1, 3))
    extra = int(rng.integers(1, 3))
    xs = shape(rng, keep + extra)
    if rng.integers(3) == 0:             # many rows summed into a short vector
        xs = (int(rng.choice([300, 1000, 2500])),) + (1,) * (extra - 1) + tuple(min(d, 33) for d in xs[extra:])
    red = tuple(range(extra))
    return ("reduce_sum", [xs[extra:], xs], lambda nc, y0, x: nc.nc_reduce_sum(y0, x, keep),
            lambda y0, x: y0 + x.sum(axis=red), {})


def g_reshape_repeat(rng):
    k = int(rng.integers(3))
    if k == 0:
        s = shape(rng, 3)
        return ("reshape", [s], lambda nc, x: nc.nc_reshape_2d(x, s[2] * s[1], s[0]),
                lambda x: x.reshape(s[0], s[1] * s[2]), {})
    s = shape(rng, int(rng.integers(1, 3)), 2000)
    n0, n1 = int(rng.choice(SMALL)), int(rng.choice(SMALL))
    if k == 1:
        return ("repeat_1d", [s], lambda nc, x: nc.nc_repeat_1d(x, n0),
                lambda x: np.broadcast_to(x, (n0,) + s), {})
    return ("repeat_2d", [s], lambda nc, x: nc.nc_repeat_2d(x, n0, n1),
            lambda x: np.broadcast_to(x, (n1, n0) + s), {})


def g_slice_concat_split(rng):
    nd = int(rng.integers(1, 5))
    s = shape(rng, nd)
    axis = int(rng.integers(nd))         # libnc axis
    npax = nd - 1 - axis
    n = s[npax]
    k = int(rng.integers(3))
    if k == 0:
        a = int(rng.integers(0, n))
        b = int(rng.integers(a + 1, n + 1))
        return ("slice", [s], lambda nc, x: nc.nc_slice(x, axis, a, b),
                lambda x: np.take(x, range(a, b), axis=npax), {})
    if k == 1:
        cnt = int(rng.integers(2, 4))
        shapes = [s[:npax] + (int(rng.choice(SMALL)),) + s[npax + 1:] for _ in range(cnt)]
        return ("concat", shapes, lambda nc, *xs: nc.nc_concat(K._arr(nc, list(xs)), cnt, axis),
                lambda *xs: np.concatenate(xs, axis=npax), {})
    # split, then the parts concatenated back in reverse order
    cnt = int(rng.integers(2, 4))
    equal = bool(rng.integers(2))
    if equal:
        part = max(1, n // cnt)
        sizes = [part] * cnt
    else:
        sizes = [int(rng.integers(1, 6)) for _ in range(cnt)]
    s = s[:npax] + (sum(sizes),) + s[npax + 1:]
    cuts = np.cumsum(sizes)[:-1]

    def build(nc, x):
        tab = (_P * cnt)()
        nc.nc_split(tab, x, cnt, None if equal else (C.c_size_t * cnt)(*sizes), axis)
        return nc.nc_concat(K._arr(nc, [tab[i] for i in reversed(range(cnt))]), cnt, axis)
    return ("split", [s], build,
            lambda x: np.concatenate(np.split(x, cuts, axis=npax)[::-1], axis=npax), {})


def g_pad(rng):
    s = shape(rng, int(rng.integers(1, 4)))
    n = s[-1]
    while True:
        left = int(rng.integers(-min(n - 1, 4), 6))
        right = int(rng.integers(-min(n - 1, 4), 6))
        if n + min(left, 0) + min(right, 0) >= 1:
            break
    lop, rop = int(rng.integers(2)), int(rng.integers(2))
    return ("pad", [s], lambda nc, x: nc.nc_pad(x, left, lop, right, rop),
            K._pad_ref(left, lop, right, rop), {})


def g_permute(rng):
    nd = int(rng.integers(2, 5))
    s = shape(rng, nd)
    if rng.integers(2):                  # both a long row and a long column: the tiled transpose
        s = tuple(int(rng.choice([33, 64, 70])) if i in (0, nd - 1) else min(d, 3) for i, d in enumerate(s))
    ax = [int(v) for v in rng.permutation(nd)]
    return ("permute", [s], lambda nc, x: nc.nc_permute(x, nd, (C.c_int * nd)(*ax)),
            lambda x: np.transpose(x, np_axes(ax)), {})


def g_rel_shift(rng):
    s = shape(rng, int(rng.integers(2, 5)))
    pos = int(rng.integers(-s[-1] - 1, s[-1] + 2))
    mult = int(rng.choice([-1, 0, 1, 1, 2]))
    return ("rel_shift", [s], lambda nc, x: nc.nc_rel_shift(x, pos, mult), K._rel_shift_ref(pos, mult), {})


def g_get_col(rng):
    V, D = int(rng.choice(SIZES)), int(rng.choice(SIZES))
    if V * D > MAX_ELEMS:
        V = max(1, MAX_ELEMS // D)
    idx = rng.integers(0, V, size=int(rng.choice(SIZES[:14]))).astype(np.int32)
    if rng.integers(2):
        idx[:] = idx[0]                  # every column collides in the backward scatter
    return ("get_col", [(V, D)], lambda nc, w: nc.nc_get_col(w, K._i32(nc, idx)), lambda w: w[idx], {})


def g_masked_fill(rng):
    nd = int(rng.integers(2, 5))
    s = shape(rng, nd)
    mask = (rng.integers(0, 3, size=s[-2:]) == 0).astype(np.int8)
    inv = int(rng.integers(2))
    c = float(rng.choice([-7.0, 0.0, 2.5]))
    return ("masked_fill", [s], lambda nc, x: nc.nc_masked_fill(x, nc.tensor(mask), c, inv),
            lambda x: np.where((mask != 0) != bool(inv), c, x), {})


def g_rows(rng):
    """softmax, the norms and the log-likelihood: rows of any length, a few of them long."""
    n = int(rng.choice(SIZES[1:] + [300, 1024, 1500, 4097]))
    lead = shape(rng, int(rng.integers(1, 3)), max(1, min(40, MAX_ELEMS // n)))
    s = lead + (n,)
    k = int(rng.integers(6))
    if k in (1, 3) and n < 4:            # two or three values minus their mean: the gradient is all cancellation
        k = 2
    if k == 0:
        return "soft_max", [s], lambda nc, x: nc.nc_soft_max(x), U.softmax, dict(scale=2.0)
    if k == 1:
        return "layer_norm", [s], lambda nc, x: nc.nc_layer_norm(x, 1e-5), U.layer_norm, {}
    if k == 2:
        return ("rms_norm", [s], lambda nc, x: nc.nc_rms_norm(x, 1e-5),
                lambda x: U.layer_norm(x, 1e-5, False), {})
    if k == 3:
        avg = int(rng.integers(2))
        b, r = K._ln_affine(avg)
        return "fused_ln", [s, (n,), (n,)], b, r, {}
    tgt = rng.integers(0, n, size=lead).astype(np.int32)

    def nll_ref(x):
        p = U.softmax(x)
        return np.log(np.take_along_axis(p, tgt[..., None].astype(np.int64), axis=-1)[..., 0])
    if k == 4:
        return ("nll_fused", [s], lambda nc, x: nc.nc_indexed_log(nc.nc_soft_max(x), K._i32(nc, tgt)),
                nll_ref, dict(scale=2.0))

    def unfused(nc, x):                  # the softmax output is also kept: no fused gradient
        p = nc.nc_soft_max(x)
        q = nc.nc_mul(nc.dup(p), nc.nc_new_f32(nc.dev, 1.0))
        l = nc.nc_indexed_log(p, K._i32(nc, tgt))
        return nc.nc_add(l, nc.nc_mul(nc.nc_sum(q), nc.nc_new_f32(nc.dev, 0.0)))
    return "nll_unfused", [s], unfused, nll_ref, dict(scale=2.0)


def g_matmul(rng):
    m, n, k = (int(rng.choice(SIZES)) for _ in range(3))
    while m * n * k > 400000:
        m, n, k = max(1, m // 2), max(1, n // 2), k
        if m * n <= 4:
            k //= 2
    batch = tuple(int(v) for v in rng.choice([2, 3], size=int(rng.integers(0, 3)))) if m * n * k < 60000 else ()
    kind = int(rng.integers(4))
    if kind == 0:
        ta, tb = int(rng.integers(2)), int(rng.integers(2))
        b, r = K._mm(ta, tb)
        return "matmul_%d%d" % (ta, tb), K._mm_shapes(ta, tb, m, k, n, batch), b, r, {}
    if kind == 1:                        # residual operand, alpha
        return ("matmul_add", [(k, m), (n, k), (n, m)], lambda nc, w, x, c: nc.nc_matmul_add(w, x, c, 0, 0, 0.5),
                lambda w, x, c: 0.5 * (x @ w) + c, {})
    act = int(rng.integers(3))
    bias = bool(rng.integers(2))
    f = [lambda v: v, U.gelu, lambda v: np.maximum(v, 0)][act]
    xs = (n, k) if rng.integers(2) else (int(rng.choice([2, 3])), max(1, n // 2), k)
    shapes = [(k, m), xs] + ([(m,)] if bias else [])
    if kind == 2:
        return ("linear", shapes, lambda nc, w, x, *b: nc.nc_linear(w, x, b[0] if bias else None, act),
                lambda w, x, *b: f(x @ w + (b[0] if bias else 0)), dict(gtol=2e-4))
    shapes.append(xs[:-1] + (m,))
    return ("linear_add", shapes,
            lambda nc, w, x, *r: nc.nc_linear_add(w, x, r[0] if bias else None, act, r[-1]),
            lambda w, x, *r: f(x @ w + (r[0] if bias else 0)) + r[-1], dict(gtol=2e-4))


GENS = [g_binary, g_binary, g_unary, g_ternary, g_reduce, g_reshape_repeat, g_slice_concat_split,
        g_slice_concat_split, g_pad, g_permute, g_rel_shift, g_get_col, g_masked_fill, g_rows, g_rows, g_matmul,
        g_matmul]


def optimiser_case(rng, tag):
    """A few steps of each update rule on one parameter of random size, tied uses accumulated."""
    w0 = rng.standard_normal(shape(rng, int(rng.integers(1, 3)))).astype(np.float32)
    algo = int(rng.choice([16, 1, 0]))
    clip = float(rng.choice([0.0, 0.1]))
    steps = [rng.standard_normal((2,) + w0.shape).astype(np.float32) for _ in range(3)]
    res = []
    for lib, on_device in ((os.environ['NNCP_TEST_HIP_LIB'], True), (REF_LIB, False)):
        nc = B.NC(lib, use_device=on_device)         # a context of its own: its parameter list ends with it
        h, p = nc.param(w0, "w")
        sp = B.SGDOptParams(algo=algo, beta1=0.0, beta2=0.99, eps=1e-8, gradient_clip=clip, lr=3e-3)
        opt = nc.nc_sgd_opt_init(nc.ctx, C.byref(sp))
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), opt)
        for g in steps:
            nc.sgd_opt_update_var(p, nc.tensor(g[0]), None)
            nc.sgd_opt_update_var(p, nc.tensor(g[1]), None)
            nc.nc_sgd_opt_update(opt)
        res.append(nc.numpy(h.value))
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), None)
        nc.nc_sgd_opt_end(opt)
        nc.close()
    assert abserr(res[0], res[1]) <= 1e-6 * float(np.abs(res[1]).max()) + 1e-7, (tag, algo, w0.shape)


def view_case(rng, tag):
    """Writes through an alias of a slice, an overlapping shift along the last axis and a
    fill, bit-exact against numpy."""
    nd = int(rng.integers(1, 4))
    s = shape(rng, nd, 4000)
    x = rng.standard_normal(s).astype(np.float32)
    for nc in (emu, ref):
        t = nc.tensor(x)
        want = x.copy()
        n = s[0]                                     # numpy axis 0 = the last libnc axis
        a = int(rng.integers(0, n)); b = int(rng.integers(a + 1, n + 1))
        src = rng.standard_normal((b - a,) + s[1:]).astype(np.float32)
        al = nc.nc_slice_alias(t, nd - 1, a, b)
        st = nc.tensor(src)
        nc.nc_tensor_copy(al, st)
        nc.free(al, st)
        want[a:b] = src
        assert np.array_equal(nc.numpy(t), want), (tag, "alias write", s, a, b)
        if n > 1:
            ln = int(rng.integers(1, n)); d0 = int(rng.integers(0, n - ln + 1)); s0 = int(rng.integers(0, n - ln + 1))
            nc.nc_tensor_copy_slice(t, t, nd - 1, d0, d0 + ln, s0)
            want[d0:d0 + ln] = want[s0:s0 + ln].copy()
            assert np.array_equal(nc.numpy(t), want), (tag, "shift", s, d0, ln, s0)
        nc.nc_tensor_set_f32(t, 1.5)
        assert (nc.numpy(t) == 1.5).all()
        nc.free(t)


def abserr(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max()) if np.size(a) else 0.0


rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 0)
n_cases = int(sys.argv[2]) if len(sys.argv) > 2 else 100
t0 = time.time()
seen = {}
for it in range(n_cases):
    if it % 12 == 11:
        kind = [optimiser_case, view_case][int(rng.integers(2))]
        kind(rng, it)
        seen[kind.__name__] = seen.get(kind.__name__, 0) + 1
        continue
    name, shapes, build, ref_fn, kw = GENS[int(rng.integers(len(GENS)))](rng)
    gtol = kw.pop("gtol", 5e-5)           # an activation's slope amplifies the rounding of a long dot product
    case = K.Case(name, shapes, build, ref_fn, **kw)
    arrays = case.inputs(rng)
    tag = (it, name, shapes)
    expect = ref_fn(*[a.astype(np.float64) for a in arrays])
    weight = rng.standard_normal(np.shape(expect))
    out_r, grads_r = case.run(ref, arrays, weight)
    out_e, grads_e = case.run(emu, arrays, weight)
    assert out_r.shape == np.shape(expect) == out_e.shape, (tag, out_r.shape, out_e.shape, np.shape(expect))
    # a sum of n terms of order one carries their rounding, however small it comes out
    ffloor = 3e-7 * max(1.0, max(a.size for a in arrays) / max(out_r.size, 1))
    amax = float(np.abs(expect).max()) if out_r.size else 0.0
    assert abserr(out_r, expect) <= 2e-5 * amax + ffloor, (tag, "checker vs numpy", abserr(out_r, expect), amax)
    assert abserr(out_e, out_r) <= 1e-5 * amax + ffloor, (tag, "forward", abserr(out_e, out_r), amax)
    for i, (ge, gr) in enumerate(zip(grads_e, grads_r)):
        assert ge.shape == gr.shape, (tag, i)
        floor = 3e-7 * max(1.0, weight.size / max(ge.size, 1))
        err = abserr(ge, gr)
        assert err <= gtol * float(np.abs(gr).max()) + floor, (tag, "grad %d" % i, err, float(np.abs(gr).max()))
    seen[name] = seen.get(name, 0) + 1
print("ok: %d cases in %.1fs (%s)" % (n_cases, time.time() - t0,
                                      ", ".join("%s %d" % kv for kv in sorted(seen.items()))))
