"""Pins the CPU checker (oracle/libnc_ref.so): every op the Transformer path
uses is compared with an independent float64 numpy restatement (forward) and
with central finite differences of that restatement (backward)."""
import numpy as np
import pytest

import cases
import nputil as U


@pytest.mark.parametrize("name", [c.name for c in cases.CASES])
def test_op_forward_backward(ref, rng, name):
    case = cases.BY_NAME[name]
    arrays = case.inputs(rng)
    expect = case.ref(*[a.astype(np.float64) for a in arrays])
    weight = rng.standard_normal(np.shape(expect))
    out, grads = case.run(ref, arrays, weight)
    assert out.shape == np.shape(expect)
    np.testing.assert_allclose(out, expect, rtol=2e-5, atol=2e-6)
    fd = U.fd_grad(lambda *xs: float((case.ref(*xs) * weight).sum()), arrays)
    for g, f in zip(grads, fd):
        assert g.shape == f.shape
        np.testing.assert_allclose(g, f, rtol=3e-3, atol=3e-4)


def test_softmax_closed_forms(ref, rng):
    x = rng.standard_normal((4, 9)).astype(np.float32) * 3
    p = ref.numpy(ref.nc_soft_max(ref.tensor(x)), free=True)
    np.testing.assert_allclose(p.sum(axis=-1), 1.0, rtol=1e-6)
    p2 = ref.numpy(ref.nc_soft_max(ref.tensor(x + 5.0)), free=True)
    np.testing.assert_allclose(p, p2, rtol=1e-5)
    big = np.array([[1000.0, 0.0, -1000.0]], dtype=np.float32)
    p3 = ref.numpy(ref.nc_soft_max(ref.tensor(big)), free=True)
    np.testing.assert_array_equal(p3, [[1.0, 0.0, 0.0]])


def test_layer_norm_closed_forms(ref, rng):
    x = rng.standard_normal((5, 64)).astype(np.float32) * 4 + 2
    y = ref.numpy(ref.nc_layer_norm(ref.tensor(x), 1e-5), free=True)
    np.testing.assert_allclose(y.mean(axis=-1), 0, atol=1e-6)
    np.testing.assert_allclose(y.var(axis=-1), 1, rtol=1e-4)
    y2 = ref.numpy(ref.nc_layer_norm(ref.tensor(3 * x + 7), 1e-5), free=True)
    np.testing.assert_allclose(y, y2, atol=1e-5)
    r = ref.numpy(ref.nc_rms_norm(ref.tensor(x), 1e-5), free=True)
    np.testing.assert_allclose((r ** 2).mean(axis=-1), 1, rtol=1e-4)


def test_attention_special_cases(ref, rng):
    """w_r = b_r = 0 reduces to textbook causal attention with memory;
    q = 0 reduces to the softmax of the bias profile."""
    H, dk, dv, B, T, M = 2, 4, 4, 2, 6, 4
    K = M + T
    q = rng.standard_normal((T, B, H * dk)).astype(np.float32)
    kv = rng.standard_normal((T, B, H * (dk + dv))).astype(np.float32)
    kvm = rng.standard_normal((M, B, H * (dk + dv))).astype(np.float32)
    y = ref.numpy(ref.nc_relpos_attention(ref.tensor(q), ref.tensor(kv), ref.tensor(kvm),
                                          None, None, H, dk, K, 1.0), free=True)
    allkv = np.concatenate([kvm, kv], 0).astype(np.float64)
    for b in range(B):
        for h in range(H):
            k = allkv[:, b, h * dk:(h + 1) * dk]
            v = allkv[:, b, H * dk + h * dv:H * dk + (h + 1) * dv]
            s = q[:, b, h * dk:(h + 1) * dk].astype(np.float64) @ k.T / np.sqrt(dk)
            causal = np.arange(K)[None, :] <= np.arange(T)[:, None] + M
            s = np.where(causal, s, -np.inf)
            np.testing.assert_allclose(y[:, b, h * dv:(h + 1) * dv], U.softmax(s) @ v,
                                       rtol=1e-5, atol=1e-6)
    b_r = rng.standard_normal((H, K)).astype(np.float32)
    y0 = ref.numpy(ref.nc_relpos_attention(ref.tensor(np.zeros_like(q)), ref.tensor(kv),
                                           ref.tensor(kvm), None, ref.tensor(b_r), H, dk, K, 2.0),
                   free=True)
    for h in range(H):
        for i in range(T):
            # key j sees bias row K-1-(i+M-j)
            prof = np.array([2.0 * b_r[h, K - 1 - (i + M - j)] / np.sqrt(dk) if j <= i + M
                             else -np.inf for j in range(K)])
            a = U.softmax(prof[None])[0]
            v = allkv[:, 0, H * dk + h * dv:H * dk + (h + 1) * dv]
            np.testing.assert_allclose(y0[i, 0, h * dv:(h + 1) * dv], a @ v, rtol=1e-5, atol=1e-6)


def test_rel_shift_places_distance_zero_on_last_row(ref):
    """nncp.c:784 with the mask of nncp.c:355-363: after the shift, row j of
    query column i must hold the entry of distance (i+M)-j, i.e. source row
    j+T-1-i; distance 0 (source row K-1) lands on key j = i+M."""
    T, M = 4, 3
    K = T + M
    rd = np.arange(K, dtype=np.float32)[None, :].repeat(T, 0)  # value = source row p
    y = ref.numpy(ref.nc_rel_shift(ref.tensor(rd), -(T - 1), 1), free=True)
    for i in range(T):
        for j in range(K):
            p = j + T - 1 - i
            assert y[i, j] == (p if p < K else 0)
        assert y[i, i + M] == K - 1


def test_backward_sums_tied_parameter(ref, rng):
    """A tensor used twice (tied w_r/b_r, nncp.c:742-760) is reported once with
    the summed gradient."""
    w = rng.standard_normal((3, 3)).astype(np.float32)
    x = rng.standard_normal((2, 3)).astype(np.float32)
    h, p = ref.param(w)
    y = ref.nc_matmul(ref.dup(h.value), ref.nc_matmul(ref.dup(h.value), ref.tensor(x)))
    loss = ref.nc_sum(y)
    g = ref.backward(loss)[p]
    fd = U.fd_grad(lambda w_: float((x @ w_ @ w_).sum()), [w])[0]
    np.testing.assert_allclose(g, fd, rtol=2e-3, atol=1e-4)


def test_views_and_copies(ref, rng):
    """nc_slice_alias shares storage; nc_tensor_copy through it mutates the
    parent (nncp.c:650-657); nc_tensor_copy_slice shifts memory (nncp.c:1212)."""
    x = rng.standard_normal((6, 2, 3)).astype(np.float32)  # libnc (3,2,6)
    t = ref.tensor(x)
    src = rng.standard_normal((1, 2, 3)).astype(np.float32)
    a = ref.nc_slice_alias(t, 2, 4, 5)
    s = ref.tensor(src)
    ref.nc_tensor_copy(a, s)
    ref.free(a, s)
    x[4:5] = src
    np.testing.assert_array_equal(ref.numpy(t), x)
    ref.nc_tensor_copy_slice(t, t, 2, 0, 4, 2)  # overlapping shift left by 2
    x[0:4] = x[2:6].copy()
    np.testing.assert_array_equal(ref.numpy(t), x)
    ref.nc_tensor_set_zero(t)
    assert not ref.numpy(t).any()
    ref.free(t)


def test_optimisers_closed_form(ref, pkg):
    """One scalar parameter, known gradients: RMSProp as BASELINE states it
    and Adam(beta1=0) with bias correction."""
    B = pkg.binding
    import ctypes as C
    for algo in (B.SGD_OPT_RMSPROP, B.SGD_OPT_ADAM, B.SGD_OPT_BASIC):
        nc = B.NC(ref.lib._name, use_device=False)
        h, p = nc.param(np.array([1.0, -2.0], dtype=np.float32))
        sp = B.SGDOptParams(algo=algo, beta1=0.0, beta2=0.99, eps=1e-8, gradient_clip=0.0, lr=3e-4)
        opt = nc.nc_sgd_opt_init(nc.ctx, C.byref(sp))
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), opt)
        w = np.array([1.0, -2.0])
        v = np.zeros(2)
        for t in range(1, 4):
            g = np.array([0.5 * t, -0.25])
            nc.sgd_opt_update_var(p, nc.tensor(g.astype(np.float32)), None)
            nc.nc_sgd_opt_set_lr(opt, 3e-4)
            nc.nc_sgd_opt_update(opt)
            if algo == B.SGD_OPT_RMSPROP:
                v = 0.99 * v + 0.01 * g * g
                w = w - 3e-4 * g / (np.sqrt(v) + 1e-8)
            elif algo == B.SGD_OPT_ADAM:
                v = 0.99 * v + 0.01 * g * g
                w = w - 3e-4 * g / (np.sqrt(v / (1 - 0.99 ** t)) + 1e-8)
            else:
                w = w - 3e-4 * g
            np.testing.assert_allclose(nc.numpy(h.value), w, rtol=1e-6)
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), None)
        nc.nc_sgd_opt_end(opt)
        nc.close()


def test_optimisers_against_library_routines(ref, pkg):
    """RMSProp and Adam of the checker against torch.optim (CPU, float64) on a random
    tensor over several steps with beta1 != 0: a library's statement of the two
    updates rather than a retyped formula.  torch's Adam divides sqrt(v) by
    sqrt(1 - beta2^t) before eps is added, as the checker does."""
    import ctypes as C
    import torch
    B = pkg.binding
    rng = np.random.default_rng(77)
    w0 = rng.normal(0, 0.5, 257).astype(np.float32)
    grads = [(rng.normal(0, 1.0, 257) * 10.0 ** rng.integers(-3, 1)).astype(np.float32) for _ in range(6)]
    for algo, b1 in ((B.SGD_OPT_RMSPROP, 0.0), (B.SGD_OPT_ADAM, 0.9), (B.SGD_OPT_ADAM, 0.0)):
        nc = B.NC(ref.lib._name, use_device=False)
        h, p = nc.param(w0.copy())
        sp = B.SGDOptParams(algo=algo, beta1=b1, beta2=0.99, eps=1e-8, gradient_clip=0.0, lr=3e-3)
        opt = nc.nc_sgd_opt_init(nc.ctx, C.byref(sp))
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), opt)
        tw = torch.tensor(w0.astype(np.float64), requires_grad=True)
        if algo == B.SGD_OPT_RMSPROP:
            topt = torch.optim.RMSprop([tw], lr=3e-3, alpha=0.99, eps=1e-8)
        else:
            topt = torch.optim.Adam([tw], lr=3e-3, betas=(b1, 0.99), eps=1e-8)
        for g in grads:
            nc.sgd_opt_update_var(p, nc.tensor(g), None)
            nc.nc_sgd_opt_set_lr(opt, 3e-3)
            nc.nc_sgd_opt_update(opt)
            tw.grad = torch.tensor(g.astype(np.float64))
            topt.step()
            np.testing.assert_allclose(nc.numpy(h.value), tw.detach().numpy(), rtol=2e-5, atol=2e-7)
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), None)
        nc.nc_sgd_opt_end(opt)
        nc.close()


def test_bf16_operand_rounding_is_round_to_nearest_even(ref):
    """The operand rounding of the bf16 variant, read off as A * I with the switch on
    (products with 1 and sums with 0 are exact), against torch's float32 -> bfloat16
    conversion bit for bit: random values over many binades, exact ties to either side,
    values one unit off a tie, subnormals, signed zeros, the largest finite value."""
    import torch
    rng = np.random.default_rng(12)
    vals = (rng.standard_normal(4000) * 10.0 ** rng.integers(-30, 30, 4000)).astype(np.float32)
    bits = rng.integers(0, 1 << 31, 3000, dtype=np.int64).astype(np.uint32)
    ties = (bits & np.uint32(0xFFFF0000)) | np.uint32(0x8000)               # exactly halfway
    near = np.concatenate([ties - np.uint32(1), ties + np.uint32(1)])
    special = np.array([0x00000001, 0x00008000, 0x00018000, 0x007FFFFF, 0x80000000, 0x7F7F0000, 0x7F7F7FFF],
                       dtype=np.uint32)
    allbits = np.concatenate([vals.view(np.uint32), ties, near, special, ties | np.uint32(0x80000000)])
    a = allbits.view(np.float32)
    a = a[np.isfinite(a)]
    a = a[: a.size // 8 * 8].reshape(-1, 8)                                 # libnc (8, n): 8 rows
    eye = np.eye(8, dtype=np.float32)
    ref.nc_set_matmul_bf16(ref.ctx, 1)
    got = ref.numpy(ref.nc_matmul(ref.tensor(eye), ref.tensor(a)), free=True)
    ref.nc_set_matmul_bf16(ref.ctx, 0)
    want = torch.from_numpy(a.copy()).to(torch.bfloat16).to(torch.float32).numpy()
    finite = np.isfinite(want)                                              # a rounding that overflows: not a GEMM input
    assert finite.mean() > 0.99
    nz = finite & (want != 0)                                               # -0 * 1 + 0 * 0 ... sums to +0
    assert np.array_equal(got[nz].view(np.uint32), want[nz].view(np.uint32))
    assert not got[finite & (want == 0)].any()


# ---- coder-side probability path: what the mathematics fixes ---------------------
def _zipf_logits(rng, n, V):
    bias = -np.log(rng.permutation(V) + 1.0)
    return (rng.normal(0, 3, (n, V)) + bias).astype(np.float32)


@pytest.mark.parametrize("V,n", [(256, 6), (16384, 2), (1, 3), (3, 5), (1000, 4)])
@pytest.mark.parametrize("mult", [65536.0, 1000.5, 2.0 ** 31, 1.0])
def test_soft_max_int_against_float64_softmax(ref, rng, V, n, mult):
    """nc_soft_max_int (libnc.h:383-384), "max(soft_max[i] * mult, 1) converted to int32", pinned
    by what it must be: int32, never below 1, ordered like the logits, and the float64 softmax
    times mult to within one unit plus the accuracy of the exponentials it is built from
    (24-bit fixed point relative to the column's largest, each rounded down: 2^-23 of the
    largest entry absolute, 2^-20 relative, and V * 2^-24 relative from the V floors in the sum)."""
    x = _zipf_logits(rng, n, V)
    y = ref.numpy(ref.nc_soft_max_int(ref.tensor(x), mult), free=True)
    assert y.dtype == np.int32 and y.shape == x.shape and (y >= 1).all()
    p = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    want = np.maximum(p * mult, 1.0)
    assert (np.abs(y - want) <= 1.0 + want * (2.0 ** -20 + V * 2.0 ** -24)
            + mult * p.max(axis=1, keepdims=True) * 2.0 ** -23).all()
    order = np.argsort(x, axis=1, kind="stable")
    assert (np.diff(np.take_along_axis(y, order, axis=1), axis=1) >= 0).all()


@pytest.mark.parametrize("V,n", [(256, 8), (16384, 3), (2, 4), (1000, 5), (65535, 2)])
def test_cdf16_invariants_and_accuracy(ref, rng, V, n):
    """The integer CDF is pinned by what it must be, not by its own formula:
    starts at 0, every frequency >= 1, total exactly 2^16, and each frequency
    is 1 + (65536 - V) * softmax within the rounding the construction allows
    (one floor of a 24-bit quantised exponential per symbol, one floor of the
    scaled prefix per boundary)."""
    x = _zipf_logits(rng, n, V)
    x[0] = 0.0                                  # uniform: every frequency equal up to the floor
    cdf = ref.numpy(ref.nc_soft_max_cdf16(ref.tensor(x)), free=True).astype(np.int64)
    assert (cdf[:, 0] == 0).all()
    freq = np.diff(np.concatenate([cdf, np.full((n, 1), 65536)], axis=1), axis=1)
    assert (freq >= 1).all() and (freq.sum(axis=1) == 65536).all()
    x64 = x.astype(np.float64)
    p = np.exp(np.maximum(x64 - x64.max(axis=1, keepdims=True), -30.0))
    p /= p.sum(axis=1, keepdims=True)
    want = 1.0 + (65536 - V) * p
    # quantising exp to 2^-24 moves a share by < V * 2^-24 relative to the total (the
    # largest term is 1), each boundary floors once: 2 for the floors + the quantisation
    slack = 2.0 + (65536 - V) * (V * 2.0 ** -24 + 3e-7)
    assert np.abs(freq - want).max() <= slack
    u = freq[0]
    assert u.max() - u.min() <= 1


def test_cdf_lookup_is_the_inverse_of_the_cdf(ref, rng):
    """searchsorted is an independent statement of 'the symbol whose interval
    holds the target'."""
    V, n, m = 4099, 3, 20000
    cdf_t = ref.nc_soft_max_cdf16(ref.tensor(_zipf_logits(rng, n, V)))
    cdf = ref.numpy(cdf_t).astype(np.int64)
    t = rng.integers(0, 65536, size=(n, m)).astype(np.uint16)
    t[:, :2] = [0, 65535]
    sym = ref.numpy(ref.nc_cdf_lookup(cdf_t, ref.tensor(t)), free=True).astype(np.int64)
    for r in range(n):
        assert np.array_equal(sym[r], np.searchsorted(cdf[r], t[r].astype(np.int64), side="right") - 1)


# ---- against the reference tree's own scalar restatement ------------------------------
# src/neural/compatibility/cuda_math_compat.c, compiled where it lies into
# oracle/_ref/libmath_compat_ref.so (softmax :287-332, ReLU :334-348, GELU :350-369,
# matmul :259-284).  Its tensors are row-major with plain shapes.
def _compat():
    import ctypes as C
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "oracle", "_ref", "libmath_compat_ref.so")
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/libmath_compat_ref.so is not built (no reference tree)")
    lib = C.CDLL(path)

    class T(C.Structure):
        _fields_ = [("data", C.POINTER(C.c_float)), ("shape", C.POINTER(C.c_size_t)), ("ndim", C.c_size_t),
                    ("total_size", C.c_size_t), ("requires_grad", C.c_bool), ("is_metal_backed", C.c_bool),
                    ("metal_buffer", C.c_void_p)]
    PT = C.POINTER(T)
    lib.cuda_compat_tensor_create.restype = PT
    lib.cuda_compat_tensor_create.argtypes = [C.POINTER(C.c_size_t), C.c_size_t, C.c_void_p]
    lib.cuda_compat_tensor_free.argtypes = [PT]
    for name, args in (("softmax", [PT, C.c_int, C.c_void_p]), ("relu", [PT, C.c_void_p]),
                       ("gelu", [PT, C.c_void_p]), ("matmul", [PT, PT, C.c_void_p])):
        f = getattr(lib, "cuda_compat_" + name)
        f.restype, f.argtypes = PT, args

    def to(a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        t = lib.cuda_compat_tensor_create((C.c_size_t * a.ndim)(*a.shape), a.ndim, None)
        C.memmove(t.contents.data, a.ctypes.data, a.nbytes)
        return t

    def back(t):
        shape = [t.contents.shape[i] for i in range(t.contents.ndim)]
        out = np.ctypeslib.as_array(t.contents.data, shape=(int(np.prod(shape)),)).reshape(shape).copy()
        lib.cuda_compat_tensor_free(t)
        return out

    def call(name, *arrays, extra=()):
        ts = [to(a) for a in arrays]
        res = getattr(lib, "cuda_compat_" + name)(*ts, *extra, None)
        assert res, name
        for t in ts:
            lib.cuda_compat_tensor_free(t)
        return back(res)
    return call


def test_softmax_matches_the_reference_restatement(ref, rng):
    """Same order of operations (row maximum, expf of the difference, left-to-right
    sum); the checker multiplies by the reciprocal of the sum where the restatement
    divides, so results agree to the last bit or the one before it, also for long
    rows and large magnitudes."""
    call = _compat()
    for shape, scale in (((7, 256), 3.0), ((3, 16384), 2.0), ((5, 1), 1.0), ((4, 33), 40.0)):
        x = (rng.standard_normal(shape) * scale).astype(np.float32)
        want = call("softmax", x, extra=(1,))
        got = ref.numpy(ref.nc_soft_max(ref.tensor(x)), free=True)
        assert np.array_equal(got == 0, want == 0), shape
        nz = want != 0
        assert (np.abs(got[nz] - want[nz]) <= 2.5e-7 * want[nz]).all(), shape


def test_activations_match_the_reference_restatement(ref, rng):
    """The tanh form of GELU with the constants 0.7978845608 and 0.044715, and ReLU."""
    call = _compat()
    x = np.concatenate([rng.standard_normal(4000) * 3, [0.0, -0.0, 1e-20, -30.0, 30.0]]).astype(np.float32)
    g_want = call("gelu", x)
    g_got = ref.numpy(ref.nc_gelu(ref.tensor(x)), free=True)
    assert np.abs(g_got - g_want).max() <= 1e-6 * max(1.0, np.abs(g_want).max())
    assert np.array_equal(ref.numpy(ref.nc_relu(ref.tensor(x)), free=True), call("relu", x))


def test_matmul_matches_the_reference_restatement(ref, rng):
    """Its row-major (m,k)x(k,n) product against nc_matmul on the same memory read
    column-major: numpy (n,k) @ numpy (k,m) in the checker's layout."""
    call = _compat()
    for m, k, n in ((5, 7, 3), (33, 129, 17), (1, 300, 1)):
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        want = call("matmul", a, b)                        # row-major (m, n)
        # row-major a (m,k) is the column-major (k,m) matrix a^T; w = b^T (n rows... k cols) likewise
        got = ref.numpy(ref.nc_matmul(ref.tensor(b), ref.tensor(a)), free=True)
        assert got.shape == want.shape
        assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max() * np.sqrt(k)


def _xorwow_stream(seed, n):
    """Marsaglia's xorwow ("Xorshift RNGs", 2003, section 3.1) from the paper's own starting state,
    the seed folded into x and d, 16 outputs discarded: the stream the build defines for libnc's
    RNDState (libnc.h:584-589 names exactly these six words)."""
    mask = 0xFFFFFFFF
    x, y, z, w, v = (123456789 ^ seed) & mask, 362436069, 521288629, 88675123, 5783321
    d = (6615241 + seed * 2654435761) & mask
    out = []
    for i in range(n + 16):
        t = x ^ (x >> 2)
        x, y, z, w = y, z, w, v
        v = ((v ^ (v << 4)) ^ (t ^ (t << 1))) & mask
        d = (d + 362437) & mask
        if i >= 16:
            out.append((d + v) & mask)
    return np.array(out, dtype=np.uint64)


def test_rnd_unif_is_the_xorwow_stream_and_uniform(ref):
    """nc_tensor_set_rnd_unif (libnc.h:195-200): the stream against an independent statement of
    the published generator, value for value; range [avg - range, avg + range) and moments of the
    uniform law; a Kolmogorov-Smirnov test; equal seeds give equal tensors, other seeds do not; a
    second call continues the stream."""
    from scipy import stats
    n = 200000

    def draw(seed, avg, rng_, count=n, calls=1):
        rs = ref.lib.nc_rnd_init(None, seed)
        outs = []
        for _ in range(calls):
            t = ref.tensor(np.zeros(count, np.float32))
            ref.lib.nc_tensor_set_rnd_unif(t, avg, rng_, rs)
            outs.append(ref.numpy(t, free=True))
        ref.lib.nc_rnd_end(rs)
        return outs if calls > 1 else outs[0]

    for seed in (0, 123, 0xDEADBEEF):
        u = (_xorwow_stream(seed, 1000) >> np.uint64(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)
        expect = np.float32(0.25) + np.float32(0.5) * (np.float32(2.0) * u - np.float32(1.0))
        assert np.array_equal(draw(seed, 0.25, 0.5, 1000), expect), seed
    a = draw(123, 1.5, 0.25)
    assert a.min() >= 1.25 and a.max() < 1.75
    assert abs(a.mean() - 1.5) < 4 * 0.25 / np.sqrt(3 * n)                 # 4 sigma of the sample mean
    assert abs(a.var() - 0.25 ** 2 / 3) < 0.01 * 0.25 ** 2 / 3
    assert stats.kstest((a - 1.25) / 0.5, "uniform").pvalue > 1e-3
    assert abs(np.corrcoef(a[:-1], a[1:])[0, 1]) < 0.01                  # no lag-1 correlation
    assert np.array_equal(a, draw(123, 1.5, 0.25))
    assert not np.array_equal(a, draw(124, 1.5, 0.25))
    first, second = draw(9, 0.0, 1.0, 500, calls=2)
    assert np.array_equal(np.concatenate([first, second]), draw(9, 0.0, 1.0, 1000))
