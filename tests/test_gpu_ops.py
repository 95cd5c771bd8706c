"""GPU parity: every op of the libnc ABI on the MI355X (libnc_hip.so) against
the CPU checker on the same seeded inputs, forward and backward.  Float
results must agree within 1e-5 of the largest reference magnitude (the fp32
bar); integer results bit-exactly."""
import ctypes as C

import numpy as np
import pytest

import cases

pytestmark = pytest.mark.gpu

TOL = 1e-5


def relerr(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / (np.abs(b).max() + 1e-30))


@pytest.mark.parametrize("name", [c.name for c in cases.CASES])
def test_op_matches_checker(hip, ref, rng, name):
    case = cases.BY_NAME[name]
    arrays = case.inputs(rng)
    expect = case.ref(*[a.astype(np.float64) for a in arrays])
    weight = rng.standard_normal(np.shape(expect))
    out_r, grads_r = case.run(ref, arrays, weight)
    out_h, grads_h = case.run(hip, arrays, weight)
    assert out_h.shape == out_r.shape
    assert relerr(out_h, out_r) <= TOL, name
    for gh, gr in zip(grads_h, grads_r):
        assert gh.shape == gr.shape
        assert relerr(gh, gr) <= 5 * TOL, name


GEMM_SHAPES = [(130, 70, 33, 1), (128, 128, 64, 1), (64, 64, 4096, 1), (512, 384, 512, 1),
               (96, 40, 72, 5), (1, 1, 1, 1), (257, 129, 1030, 1), (256, 2048, 128, 1)]


@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
@pytest.mark.parametrize("shape", GEMM_SHAPES)
def test_gemm_vs_checker(hip, ref, rng, ta, tb, shape):
    m, n, k, batch = shape
    bsh = (batch,) if batch > 1 else ()
    a = rng.standard_normal(bsh + ((m, k) if ta else (k, m))).astype(np.float32)
    b = rng.standard_normal(bsh + ((k, n) if tb else (n, k))).astype(np.float32)
    outs = []
    for nc in (hip, ref):
        y = nc.nc_matmul_add(nc.tensor(a), nc.tensor(b), None, ta, tb, 1.0)
        outs.append(nc.numpy(y, free=True))
    assert relerr(outs[0], outs[1]) <= TOL


def test_gemm_columns_do_not_depend_on_batch_width(hip, rng):
    """A column computed alone is bit-identical to the same column computed in
    a wide matrix (what lets a decoder replay an encoder's step)."""
    w = rng.standard_normal((512, 512)).astype(np.float32)
    x = rng.standard_normal((2048, 512)).astype(np.float32)
    full = hip.numpy(hip.nc_matmul(hip.tensor(w), hip.tensor(x)), free=True)
    part = hip.numpy(hip.nc_matmul(hip.tensor(w), hip.tensor(x[64:96])), free=True)
    assert np.array_equal(full[64:96], part)
    again = hip.numpy(hip.nc_matmul(hip.tensor(w), hip.tensor(x)), free=True)
    assert np.array_equal(full, again)


@pytest.mark.parametrize("m,k,n", [(512, 512, 32), (2048, 512, 32), (512, 2048, 32), (256, 512, 32), (100, 70, 7),
                                   (64, 33, 33), (130, 1, 64), (1024, 96, 40), (512, 1024, 32), (96, 4096, 16),
                                   (64, 288, 9), (32, 32, 1), (32, 2304, 64)])
def test_few_column_products_are_the_wide_products_columns(hip, rng, m, k, n):
    """Width-invariant mode: a product with a few token columns (the decoder's per-timestep
    shape, which takes the 16x16x4 MFMA few-column kernel) equals, bit for bit, the same
    product through the vector-ALU kernel (chains of fused multiply-adds in the order an fp32
    MFMA accumulates), through the 32x32x2 MFMA few-column kernel, through the tile kernel, and
    the matching columns of a wide product, with every epilogue option the forward pass uses
    (bias, GELU, residual addend)."""
    lib = C.CDLL(hip.lib._name)
    w = rng.standard_normal((k, m)).astype(np.float32)
    wide = rng.standard_normal((200 + n, k)).astype(np.float32)
    bias = rng.standard_normal(m).astype(np.float32)
    res = rng.standard_normal((200 + n, m)).astype(np.float32)
    NC_ACT_NONE, NC_ACT_GELU = 0, 1

    def products(x, r):
        outs = [hip.numpy(hip.nc_matmul(hip.tensor(w), hip.tensor(x)), free=True),
                hip.numpy(hip.nc_linear(hip.tensor(w), hip.tensor(x), hip.tensor(bias), NC_ACT_GELU), free=True),
                hip.numpy(hip.nc_linear_add(hip.tensor(w), hip.tensor(x), hip.tensor(bias), NC_ACT_NONE, hip.tensor(r)), free=True),
                hip.numpy(hip.nc_matmul_add(hip.tensor(w), hip.tensor(x), hip.tensor(r), 0, 0, 1.0), free=True)]
        return outs
    hip.nc_set_matmul_width_invariant(hip.ctx, 1)
    try:
        whole = products(wide, res)
        few = products(wide[150:150 + n], res[150:150 + n])
        others = []
        for kernel in (2, 1, 0):
            lib.nchip_gemm_few_columns_kernel(kernel)
            others.append(products(wide[150:150 + n], res[150:150 + n]))
    finally:
        lib.nchip_gemm_few_columns_kernel(3)
        hip.nc_set_matmul_width_invariant(hip.ctx, 0)
    for i, (a, b) in enumerate(zip(whole, few)):
        assert np.array_equal(a[150:150 + n], b)
        for other in others:
            assert np.array_equal(b, other[i])
    ref64 = wide[150:150 + n].astype(np.float64) @ w.astype(np.float64)
    assert relerr(few[0], ref64) <= TOL


@pytest.mark.parametrize("m0,m1,k,n,T", [(512, 1024, 512, 32, 4), (64, 96, 64, 5, 3), (40, 24, 19, 3, 2)])
def test_projection_pair_of_a_timestep(hip, ref, rng, m0, m1, k, n, T):
    """nc_linear_pair_into: the query projection and the key / value projection of one decoder
    timestep in one launch, the second written into its cache slot.  In width-invariant mode
    the values are the bits of nc_linear and nc_matmul; in every mode they match the checker,
    and the other slots of the cache are left alone."""
    w0 = rng.standard_normal((k, m0)).astype(np.float32)
    w1 = rng.standard_normal((k, m1)).astype(np.float32)
    b0 = rng.standard_normal(m0).astype(np.float32)
    x = rng.standard_normal((n, k)).astype(np.float32)
    cache = rng.standard_normal((T, n, m1)).astype(np.float32)
    outs = {}
    for name, nc, inv in (("inv", hip, 1), ("plain", hip, 0), ("ref", ref, 0)):
        if nc is hip:
            nc.nc_set_matmul_width_invariant(nc.ctx, inv)
        dst = nc.tensor(cache)
        q = nc.nc_linear_pair_into(nc.tensor(w0), nc.tensor(b0), nc.tensor(w1), nc.tensor(x), dst, T - 1)
        outs[name] = (nc.numpy(q, free=True), nc.numpy(dst, free=True))
        if nc is hip and inv:
            outs["two"] = (nc.numpy(nc.nc_linear(nc.tensor(w0), nc.tensor(x), nc.tensor(b0), 0), free=True),
                           nc.numpy(nc.nc_matmul(nc.tensor(w1), nc.tensor(x)), free=True))
        if nc is hip:
            nc.nc_set_matmul_width_invariant(nc.ctx, 0)
    assert np.array_equal(outs["inv"][0], outs["two"][0])
    assert np.array_equal(outs["inv"][1][T - 1], outs["two"][1])
    for name in ("inv", "plain"):
        assert relerr(outs[name][0], outs["ref"][0]) <= TOL
        assert relerr(outs[name][1][T - 1], outs["ref"][1][T - 1]) <= TOL
        assert np.array_equal(outs[name][1][:T - 1], cache[:T - 1])


def test_gemm_bf16_variant(hip, ref, rng):
    w = rng.standard_normal((256, 320)).astype(np.float32)
    x = rng.standard_normal((200, 256)).astype(np.float32)
    outs = []
    for nc in (hip, ref):
        nc.nc_set_matmul_bf16(nc.ctx, 1)
        outs.append(nc.numpy(nc.nc_matmul(nc.tensor(w), nc.tensor(x)), free=True))
        nc.nc_set_matmul_bf16(nc.ctx, 0)
    # same rounded operands, fp32 accumulation in a different order
    assert relerr(outs[0], outs[1]) <= 1e-5
    exact = x.astype(np.float64) @ w.astype(np.float64)
    assert relerr(outs[0], exact) <= 2e-2


# bf16 products through bf16 copies of the operands (mode 2 forces that route
# for any unbatched shape): the rounded values and the accumulation order are
# those of the 128x128x32 tile kernel rounding inside its loader (config 7),
# so the two must agree bit for bit; the CPU checker rounds the same way and
# accumulates in another order.
@pytest.mark.parametrize("m,n,k", [(256, 384, 512), (130, 70, 100), (1000, 333, 257), (8, 5, 32), (129, 257, 1031)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_gemm_bf16_from_rounded_copies(hip, ref, rng, m, n, k, ta, tb):
    a = rng.standard_normal((m, k) if ta else (k, m)).astype(np.float32)  # numpy order: (columns, rows)
    b = rng.standard_normal((k, n) if tb else (n, k)).astype(np.float32)
    lib = C.CDLL(hip.lib._name)
    outs = {}
    for nc, mode in ((hip, 2), (hip, 0), (ref, None)):
        nc.nc_set_matmul_bf16(nc.ctx, 1)
        if mode is not None:
            lib.nchip_gemm_bf16_source(mode)
            lib.nchip_gemm_force_config(7)
        x, y = nc.tensor(a), nc.tensor(b)
        outs[(nc is hip, mode)] = nc.numpy(nc.nc_matmul_add(x, y, None, ta, tb, 1.0), free=True)
        nc.nc_set_matmul_bf16(nc.ctx, 0)
    lib.nchip_gemm_bf16_source(1)
    lib.nchip_gemm_force_config(0)
    assert np.array_equal(outs[(True, 2)], outs[(True, 0)])
    assert relerr(outs[(True, 2)], outs[(False, None)]) <= 1e-5


@pytest.mark.parametrize("cfg", [dict(H=2, dk=64, dv=64, B=2, T=64, M=64, d_pos=128, attn_len=128),
                                 dict(H=4, dk=32, dv=32, B=3, T=20, M=20, d_pos=40, attn_len=40),
                                 dict(H=2, dk=32, dv=32, B=2, T=32, M=32, d_pos=32, attn_len=48),
                                 dict(H=2, dk=64, dv=64, B=2, T=33, M=17, d_pos=29, attn_len=25),
                                 dict(H=3, dk=32, dv=32, B=2, T=7, M=50, d_pos=57, attn_len=57),
                                 dict(H=2, dk=64, dv=64, B=1, T=64, M=64, d_pos=64, attn_len=100),
                                 dict(H=2, dk=64, dv=64, B=2, T=48, M=80, d_pos=128, attn_len=128),
                                 dict(H=2, dk=64, dv=64, B=2, T=64, M=96, d_pos=160, attn_len=160),
                                 dict(H=2, dk=64, dv=64, B=19, T=64, M=192, d_pos=256, attn_len=256),
                                 # more than 128 keys: the key-chunked single-kernel path (12, 16, 20 key tiles)
                                 dict(H=2, dk=64, dv=64, B=3, T=64, M=256, d_pos=320, attn_len=320),
                                 dict(H=1, dk=64, dv=64, B=2, T=40, M=160, d_pos=40, attn_len=90),
                                 dict(H=2, dk=64, dv=64, B=2, T=64, M=140, d_pos=204, attn_len=204),
                                 dict(H=2, dk=64, dv=64, B=2, T=17, M=283, d_pos=300, attn_len=150),
                                 # heads of 128 features (the enwik profile: 8 x 128, 64 + 256 keys): the
                                 # chunked kernels with the feature axis in halves; 8, 12, 16, 20 key tiles
                                 dict(H=2, dk=128, dv=128, B=3, T=64, M=256, d_pos=320, attn_len=320),
                                 dict(H=2, dk=128, dv=128, B=2, T=64, M=64, d_pos=128, attn_len=128),
                                 dict(H=2, dk=128, dv=128, B=2, T=32, M=20, d_pos=29, attn_len=25),
                                 dict(H=1, dk=128, dv=128, B=2, T=40, M=160, d_pos=40, attn_len=90),
                                 dict(H=2, dk=128, dv=128, B=2, T=48, M=116, d_pos=164, attn_len=100),
                                 dict(H=3, dk=128, dv=128, B=1, T=7, M=49, d_pos=56, attn_len=56)])
def test_relpos_attention_model_shapes(hip, ref, rng, cfg):
    H, dk, dv, B, T, M, d_pos = (cfg[k] for k in ("H", "dk", "dv", "B", "T", "M", "d_pos"))
    K = M + T
    shapes = [(T, B, H * dk), (T, B, H * (dk + dv)), (M, B, H * (dk + dv)), (H, d_pos, dk), (H, K)]
    arrays = [(rng.standard_normal(s) * 0.5).astype(np.float32) for s in shapes]
    weight = rng.standard_normal((T, B, H * dv)).astype(np.float32)
    res = []
    lib = C.CDLL(hip.lib._name)
    # heads of 128 beyond 128 keys: by default one kernel forward and the batched products
    # backward; the single-kernel backward is switched on for a second pass
    passes = [(hip, 0), (ref, 0)] + ([(hip, 1)] if dk == 128 and K > 128 else [])
    for nc, wide_bwd in passes:
        lib.nchip_relpos_attn_wide_backward(wide_bwd)
        hs = [nc.param(a, "p%d" % i) for i, a in enumerate(arrays)]
        y = nc.nc_relpos_attention(*[nc.dup(h.value) for h, _ in hs], H, dk, cfg["attn_len"], 2.5)
        if nc is hip and dk in (64, 128) and K % 4 == 0 and K <= 320:
            assert lib.nchip_relpos_attn_last_launches() == 1
        out = nc.numpy(y)
        loss = nc.nc_sum(nc.nc_mul(y, nc.tensor(weight)))
        g = nc.backward(loss)
        nc.free(loss)
        if nc is hip and K % 4 == 0 and K <= 320 and (dk == 64 or (dk == 128 and (K <= 128 or wide_bwd))):
            # these shapes take one kernel each way (plus the sum of the per-stream partials)
            assert lib.nchip_relpos_attn_last_launches() <= 2
        res.append((out, [g[p] for _, p in hs]))
    lib.nchip_relpos_attn_wide_backward(0)
    for got in [res[0]] + res[2:]:
        assert relerr(got[0], res[1][0]) <= TOL
        for gh, gr in zip(got[1], res[1][1]):
            assert relerr(gh, gr) <= 5 * TOL


def _adversarial_logits(rng, V, n):
    x = rng.standard_normal((n, V)).astype(np.float32) * 3
    x[0] = 0.0                       # all equal
    x[1] = -50.0; x[1, V // 3] = 40  # one dominant symbol
    x[2] = np.linspace(-200, 200, V, dtype=np.float32)
    x[3] *= 1e-3
    x[4] += -np.log(np.arange(1, V + 1, dtype=np.float32))[rng.permutation(V)]
    return x


@pytest.mark.parametrize("V,n", [(256, 64), (16384, 16), (2, 8), (1000, 33), (65535, 6)])
def test_cdf16_bit_exact(hip, ref, rng, V, n):
    x = _adversarial_logits(rng, V, max(n, 5))
    c_h = hip.numpy(hip.nc_soft_max_cdf16(hip.tensor(x)), free=True)
    c_r = ref.numpy(ref.nc_soft_max_cdf16(ref.tensor(x)), free=True)
    assert np.array_equal(c_h, c_r)
    c = c_h.astype(np.int64)
    assert (c[:, 0] == 0).all()
    freq = np.diff(np.concatenate([c, np.full((c.shape[0], 1), 65536)], axis=1), axis=1)
    assert (freq >= 1).all() and (freq.sum(axis=1) == 65536).all()


# m >= 262144 targets per column takes the inverse-table kernel (vector path
# when m is a multiple of 4), fewer the per-target search (CDF in LDS up to
# V 16384, read from memory beyond)
@pytest.mark.parametrize("V,n,m", [(16384, 4, 50000), (16384, 3, 300000), (1000, 2, 262147),
                                   (65535, 2, 40000), (65535, 2, 262144), (2, 3, 1000)])
def test_cdf_lookup_bit_exact(hip, ref, rng, V, n, m):
    x = _adversarial_logits(rng, V, 5)[:n]
    t = rng.integers(0, 65536, size=(n, m)).astype(np.uint16)
    t[:, :4] = [0, 65535, 1, 65534]
    res = []
    for nc in (hip, ref):
        cdf = nc.nc_soft_max_cdf16(nc.tensor(x))
        res.append(nc.numpy(nc.nc_cdf_lookup(cdf, nc.tensor(t)), free=True))
    assert np.array_equal(res[0], res[1])


@pytest.mark.parametrize("V,n", [(256, 2048), (16384, 129), (2, 5), (3, 300), (1000, 257), (65535, 9), (4096, 40), (1, 7),
                                 (255, 33), (4097, 12)])
def test_cdf_path_bit_exact(hip, ref, rng, V, n):
    """The CDF entries an encoder's coder reads for known symbols (symbols outside the alphabet
    included: they read nothing outside their column)."""
    x = _adversarial_logits(rng, V, max(n, 5))
    sym = rng.integers(0, V, size=x.shape[0]).astype(np.int32)
    sym[:5] = [0, V - 1, -7, V, 2 ** 31 - 1]
    res = []
    for nc in (hip, ref):
        res.append(nc.numpy(nc.nc_cdf_path(nc.nc_soft_max_cdf16(nc.tensor(x)), nc.tensor(sym)), free=True))
    assert res[0].shape == (x.shape[0], max(1, int(np.ceil(np.log2(V))))) and np.array_equal(res[0], res[1])
    # and as one op (no table is built)
    for nc in (hip, ref):
        one = nc.numpy(nc.nc_soft_max_cdf16_path(nc.tensor(x), nc.tensor(sym)), free=True)
        assert np.array_equal(one, res[0])
    # the build kernel's own path form through its entry point, for every kernel shape of the build
    lib = C.CDLL(hip.lib._name)
    lib.nchip_softmax_cdf16_path.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int]
    st = C.c_void_p(hip.nc_context_stream(hip.ctx))
    ptr = lambda t: C.c_void_p(hip.lib.nc_tensor_get_ptr(t, None))
    levels = res[0].shape[1]
    tx, ts, tp = hip.tensor(x), hip.tensor(sym), hip.tensor(np.full(res[0].shape, 0xABCD, np.uint16))
    assert lib.nchip_softmax_cdf16_path(st, ptr(tx), ptr(ts), ptr(tp), V, x.shape[0], levels) == 0
    got = hip.numpy(tp)
    hip.free(tx, ts, tp)
    assert np.array_equal(got, res[0])


@pytest.mark.parametrize("algo", [16, 1, 0])
def test_optimiser_step(hip, ref, rng, pkg, algo):
    B = pkg.binding
    w0 = rng.standard_normal((300, 70)).astype(np.float32)
    res = []
    for lib, dev in ((hip.lib._name, True), (ref.lib._name, False)):
        nc = B.NC(lib, use_device=dev)
        h, p = nc.param(w0)
        sp = B.SGDOptParams(algo=algo, beta1=0.0, beta2=0.99, eps=1e-8, gradient_clip=0.1, lr=3e-4)
        opt = nc.nc_sgd_opt_init(nc.ctx, C.byref(sp))
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), opt)
        r2 = np.random.default_rng(7)
        for _ in range(3):
            g = r2.standard_normal(w0.shape).astype(np.float32)
            nc.sgd_opt_update_var(p, nc.tensor(g), None)
            nc.sgd_opt_update_var(p, nc.tensor(0.5 * g), None)  # tied use: accumulates
            nc.nc_sgd_opt_update(opt)
        res.append(nc.numpy(h.value))
        nc.nc_sgd_opt_set_all(C.byref(nc.plist), None)
        nc.nc_sgd_opt_end(opt)
        nc.close()
    assert relerr(res[0], res[1]) <= 1e-6


def test_two_gradients_before_one_update_with_deferred_weight_gradients(hip, rng, pkg):
    """Gradient accumulation (two nc_backward passes, one nc_sgd_opt_update) while the weight
    gradients of a pass are deferred to one grouped launch at its end: the second pass must
    add to a gradient that has been written.  Plain SGD with lr = 1 exposes the sum."""
    B = pkg.binding
    w0 = rng.standard_normal((30, 40)).astype(np.float32)          # (m = 40, k = 30) in libnc order
    x = rng.standard_normal((16, 30)).astype(np.float32)
    up = [rng.standard_normal((16, 40)).astype(np.float32) for _ in range(2)]
    nc = B.NC(hip.lib._name, use_device=True)
    nc.nc_set_deferred_weight_grad(nc.ctx, 1)
    h, p = nc.param(w0)
    sp = B.SGDOptParams(algo=B.SGD_OPT_BASIC, lr=1.0)
    opt = nc.nc_sgd_opt_init(nc.ctx, C.byref(sp))
    nc.nc_sgd_opt_set_all(C.byref(nc.plist), opt)
    forward = C.cast(nc.lib.sgd_opt_update_var, B.PARAM_UPDATE_FUNC)
    for u in up:
        y = nc.nc_matmul(nc.dup(h.value), nc.tensor(x))
        loss = nc.nc_sum(nc.nc_mul(y, nc.tensor(u)))
        nc.lib.nc_backward(loss, nc.nc_new_f32(nc.dev, 1.0), forward, 0)
        nc.free(loss)
    nc.nc_sgd_opt_update(opt)
    w1 = nc.numpy(h.value)
    nc.nc_sgd_opt_set_all(C.byref(nc.plist), None)
    nc.nc_sgd_opt_end(opt)
    nc.close()
    grad = x.astype(np.float64).T @ (up[0].astype(np.float64) + up[1])     # numpy (k, m): dW[m, k] = sum_n dY[m, n] X[k, n]
    assert relerr(w0 - w1, grad) <= 1e-5


def test_random_fills_are_the_checkers_bit_for_bit(hip, ref):
    """nc_tensor_set_rnd_unif and nc_tensor_set_dropout (libnc.h:195-201): same seed, same
    tensors from both libraries, across several calls on one generator state."""
    outs = []
    for nc in (hip, ref):
        rs = nc.lib.nc_rnd_init(nc.dev, 321)
        got = []
        for shape, avg, width in (((64, 48), 0.0, 0.0625), ((1000,), 1.0, 2.0)):
            t = nc.tensor(np.zeros(shape, np.float32))
            nc.lib.nc_tensor_set_rnd_unif(t, avg, width, rs)
            got.append(nc.numpy(t, free=True))
        t = nc.tensor(np.zeros((50, 30), np.float32))
        nc.lib.nc_tensor_set_dropout(t, 0.3, rs)
        got.append(nc.numpy(t, free=True))
        nc.lib.nc_rnd_end(rs)
        outs.append(got)
    for a, b in zip(*outs):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.ptp(outs[0][0]) > 0.1 and set(np.unique(outs[0][2])) == {0.0, np.float32(1 / 0.7)}


def test_views_and_copies_on_device(hip, rng):
    x = rng.standard_normal((6, 2, 3)).astype(np.float32)
    t = hip.tensor(x)
    src = rng.standard_normal((1, 2, 3)).astype(np.float32)
    a = hip.nc_slice_alias(t, 2, 4, 5)
    s = hip.tensor(src)
    hip.nc_tensor_copy(a, s)
    hip.free(a, s)
    x[4:5] = src
    assert np.array_equal(hip.numpy(t), x)
    hip.nc_tensor_copy_slice(t, t, 2, 0, 4, 2)
    x[0:4] = x[2:6].copy()
    assert np.array_equal(hip.numpy(t), x)
    hip.nc_tensor_set_zero(t)
    assert not hip.numpy(t).any()
    hip.free(t)


@pytest.mark.parametrize("axis,n,dst0,dst1,src0", [(2, 7, 0, 6, 1), (2, 7, 0, 2, 5), (2, 9, 1, 7, 3), (1, 8, 0, 5, 3),
                                                    (0, 10, 2, 9, 3), (2, 7, 2, 6, 0), (2, 6, 0, 4, 2)])
def test_copy_slice_within_one_tensor(hip, rng, axis, n, dst0, dst1, src0):
    """nc_tensor_copy_slice of a tensor onto itself (the memory update, nncp.c:1205-1221): shifts
    towards the front go piece by piece without a temporary, whatever the distance and the length;
    a shift towards the back goes through one; both equal numpy's copy of the source first."""
    shape = [4, 5, 6]
    shape[2 - axis] = n                                  # numpy axes are libnc's reversed
    x = rng.standard_normal(shape).astype(np.float32)
    t = hip.tensor(x)
    hip.nc_tensor_copy_slice(t, t, axis, dst0, dst1, src0)
    sl = lambda a, b: tuple(slice(a, b) if i == 2 - axis else slice(None) for i in range(3))
    want = x.copy()
    want[sl(dst0, dst1)] = x[sl(src0, src0 + dst1 - dst0)]
    assert np.array_equal(hip.numpy(t), want)
    hip.free(t)


def _run_graph(nc, arrays, build, weight):
    hs = [nc.param(a, "p%d" % i) for i, a in enumerate(arrays)]
    y = build(nc, *[nc.dup(h.value) for h, _ in hs])
    out = nc.numpy(y)
    loss = nc.nc_sum(nc.nc_mul(y, nc.tensor(weight)))
    g = nc.backward(loss)
    nc.free(loss)
    return out, [g[p] for _, p in hs]


@pytest.mark.parametrize("d,n", [(128, 80), (256, 37), (512, 2048), (512, 100), (1024, 64), (96, 50)])
@pytest.mark.parametrize("avg", [0, 1])
def test_norm_model_shapes(hip, ref, rng, d, n, avg):
    """LayerNorm / RMSNorm with affine at the widths the single-pass backward
    is specialised for (and one it is not), ragged column counts included."""
    arrays = [rng.standard_normal((n, d)).astype(np.float32),
              (1 + 0.1 * rng.standard_normal(d)).astype(np.float32),
              (0.1 * rng.standard_normal(d)).astype(np.float32)]
    weight = rng.standard_normal((n, d)).astype(np.float32)
    build = lambda nc, x, w, b: nc.nc_fused_layer_norm(x, w, b, 1e-5, avg)
    (oh, gh), (orf, gr) = (_run_graph(nc, arrays, build, weight) for nc in (hip, ref))
    assert relerr(oh, orf) <= TOL
    for a, b in zip(gh, gr):
        assert relerr(a, b) <= 5 * TOL


@pytest.mark.parametrize("v,d,n", [(256, 512, 2048), (50, 128, 333), (16, 40, 9000), (16384, 64, 4096),
                                   (3000, 32, 8192), (1000, 100, 4095), (700, 9, 1023)])
def test_embedding_gradient_model_shapes(hip, ref, rng, v, d, n):
    """get_col backward (deterministic scatter-add), including a token count
    beyond the in-LDS index list, a vocabulary of thousands (most symbols without
    a token) and token counts that leave the threads' slices ragged."""
    w = rng.standard_normal((v, d)).astype(np.float32)
    idx = rng.integers(0, v, size=n).astype(np.int32)
    idx[: min(n, 7)] = 3  # repeated symbol
    idx[n // 3: n // 3 + n // 5] = 5  # and a frequent one: a list of hundreds of tokens
    weight = rng.standard_normal((n, d)).astype(np.float32)
    res = []
    for nc in (hip, ref):
        build = lambda nc, w_: nc.nc_get_col(w_, nc.tensor(idx))
        res.append(_run_graph(nc, [w], build, weight))
    assert np.array_equal(res[0][0], res[1][0])
    assert relerr(res[0][1][0], res[1][1][0]) <= 5 * TOL
    # same inputs, same bits
    again = _run_graph(hip, [w], lambda nc, w_: nc.nc_get_col(w_, nc.tensor(idx)), weight)
    assert np.array_equal(again[1][0], res[0][1][0])


@pytest.mark.parametrize("v,n", [(2048, 37), (4096, 5), (5000, 9), (16384, 33), (4098, 6), (20000, 3)])
def test_long_column_softmax_and_log_likelihood(hip, ref, rng, v, n):
    """Vocabularies of thousands: the softmax that holds a column in one workgroup's registers
    (2048..16384 entries in multiples of 4; other lengths take the wave-per-column kernel) and
    the vectorised gradient of the log-likelihood, against float64 and against the checker."""
    x = (3.0 * rng.standard_normal((n, v))).astype(np.float32)
    tgt = rng.integers(0, v, size=n).astype(np.int32)
    tgt[0], tgt[-1] = 0, v - 1
    weight = rng.standard_normal(n).astype(np.float32)
    build = lambda nc, x_: nc.nc_indexed_log(nc.nc_soft_max(x_), nc.tensor(tgt))
    (oh, gh), (orf, gr) = (_run_graph(nc, [x], build, weight) for nc in (hip, ref))
    x64 = x.astype(np.float64)
    lse = np.log(np.exp(x64 - x64.max(axis=1, keepdims=True)).sum(axis=1)) + x64.max(axis=1)
    assert np.abs(oh - (x64[np.arange(n), tgt] - lse)).max() <= 2e-5
    assert relerr(oh, orf) <= TOL
    p64 = np.exp(x64 - lse[:, None])
    want = -p64 * weight[:, None].astype(np.float64)
    want[np.arange(n), tgt] += weight
    assert relerr(gh[0], want) <= 5 * TOL
    assert relerr(gh[0], gr[0]) <= 5 * TOL
    p = hip.numpy(hip.nc_soft_max(hip.tensor(x)), free=True)
    assert relerr(p, p64) <= TOL and np.abs(p.astype(np.float64).sum(axis=1) - 1).max() <= 1e-5


@pytest.mark.parametrize("f,n", [(2048, 2048), (512, 2048), (256, 77), (1000, 513)])
def test_bias_gradient_model_shapes(hip, ref, rng, f, n):
    """Column-sum reductions behind the bias gradients (two-stage, fixed order)."""
    x = rng.standard_normal((n, f)).astype(np.float32)
    b = rng.standard_normal(f).astype(np.float32)
    weight = rng.standard_normal((n, f)).astype(np.float32)
    build = lambda nc, x_, b_: nc.nc_add(x_, b_)
    (oh, gh), (orf, gr) = (_run_graph(nc, [x, b], build, weight) for nc in (hip, ref))
    assert relerr(oh, orf) <= TOL
    exact = weight.astype(np.float64).sum(axis=0)
    assert relerr(gh[1], exact) <= TOL
    assert relerr(gh[1], gr[1]) <= 5 * TOL


def _dev(nc, arr):
    t = nc.tensor(np.ascontiguousarray(arr, dtype=np.float32))
    return t, C.c_void_p(nc.lib.nc_tensor_get_ptr(t, None))


def test_timestep_rows_without_copy_launches(hip, rng):
    """nc_soft_max_cdf16_to_host and nc_get_col_host_indices: the CDF rows the kernel writes
    into host memory are those of nc_soft_max_cdf16, and the gather that reads its indices from
    host memory (times the embedding multiplier) is nc_mul(nc_get_col(...), scale), bit for bit."""
    V, B, D = 256, 32, 512
    logits = (3 * rng.standard_normal((B, V))).astype(np.float32)
    want = hip.numpy(hip.nc_soft_max_cdf16(hip.tensor(logits)), free=True)
    host = hip.nc_soft_max_cdf16_to_host(hip.tensor(logits))
    hip.nc_synchronize(hip.dev)
    got = hip.numpy(host, free=True)
    assert got.dtype == np.uint16 and np.array_equal(got, want)
    w = rng.standard_normal((V, D)).astype(np.float32)
    idx = rng.integers(0, V, B).astype(np.int32)
    scale = float(np.sqrt(D))
    a = hip.nc_mul(hip.nc_get_col(hip.tensor(w), hip.tensor(idx)), hip.nc_new_f32(hip.dev, scale))
    b = hip.nc_get_col_host_indices(hip.tensor(w), hip.tensor(idx, device=hip.cpu), scale)
    a, b = hip.numpy(a, free=True), hip.numpy(b, free=True)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(a, w[idx] * np.float32(scale))


@pytest.mark.parametrize("m,k,n", [(512, 512, 32), (2048, 512, 32), (512, 2048, 32), (256, 512, 5), (64, 96, 64),
                                   (1024, 1024, 33), (32, 4096, 8), (96, 288, 16)])
def test_k_major_weight_copies_change_no_bit(hip, rng, m, k, n):
    """nc_keep_k_major_weight: the few-column products of the width-invariant class read a
    k-major copy of their weight matrix (a quarter of the cache lines) and write the bits they
    write from the matrix itself - plain, with bias and GELU, with a residual, as a pair into a
    cache slot, and behind a norm."""
    w = hip.tensor(rng.standard_normal((k, m)).astype(np.float32))
    w1 = hip.tensor(rng.standard_normal((k, 2 * m)).astype(np.float32))
    x = rng.standard_normal((n, k)).astype(np.float32)
    bias = rng.standard_normal(m).astype(np.float32); res = rng.standard_normal((n, m)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32); b = (0.1 * rng.standard_normal(k)).astype(np.float32)
    cache = rng.standard_normal((2, n, 2 * m)).astype(np.float32)
    d, t = hip.dup, hip.tensor

    def products():
        outs = [hip.numpy(hip.nc_matmul(d(w), t(x)), free=True),
                hip.numpy(hip.nc_linear(d(w), t(x), t(bias), 1), free=True),
                hip.numpy(hip.nc_linear_add(d(w), t(x), t(bias), 0, t(res)), free=True),
                hip.numpy(hip.nc_matmul_add(d(w), t(x), t(res), 0, 0, 1.0), free=True)]
        dst = t(cache)
        outs.append(hip.numpy(hip.nc_linear_pair_into(d(w), t(bias), d(w1), t(x), dst, 1), free=True))
        outs.append(hip.numpy(dst, free=True))
        dst = t(cache)
        pn = C.c_void_p()
        outs.append(hip.numpy(hip.nc_norm_linear_pair_into(t(x), t(g), t(b), 1e-5, 1, d(w), t(bias), 0, d(w1), dst, 0, C.byref(pn)), free=True))
        outs.append(hip.numpy(dst, free=True)); outs.append(hip.numpy(pn, free=True))
        return outs
    hip.nc_set_matmul_width_invariant(hip.ctx, 1)
    try:
        plain = products()
        hip.nc_keep_k_major_weight(w); hip.nc_keep_k_major_weight(w1)
        kept = products()
        hip.nc_forget_k_major_weights(hip.ctx)
        again = products()
    finally:
        hip.nc_forget_k_major_weights(hip.ctx)
        hip.nc_set_matmul_width_invariant(hip.ctx, 0)
        hip.free(w, w1)
    for a, b_, c in zip(plain, kept, again):
        assert np.array_equal(a.view(np.uint32), b_.view(np.uint32))
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32))


@pytest.mark.parametrize("k,m0,m1,n,avg,act", [(512, 512, 1024, 32, 1, 0), (512, 2048, 0, 32, 1, 1), (512, 256, 0, 32, 1, 0),
                                               (256, 64, 96, 5, 0, 0), (128, 96, 0, 64, 0, 2), (512, 64, 0, 17, 1, 1),
                                               (192, 64, 32, 4, 1, 0)])
def test_norm_riding_on_a_product(hip, ref, rng, k, m0, m1, n, avg, act):
    """nc_norm_linear_pair_into: in width-invariant mode the one-launch kernel (k = 128, 256, 512)
    gives the bits of nc_fused_layer_norm followed by nc_linear / nc_linear_pair_into - the
    normalised tensor, the product(s) and the cache slot - and in every mode the values match
    the checker's separate steps."""
    T = 3
    x = rng.standard_normal((n, k)).astype(np.float32) * 2 + 0.3
    g = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32); b = (0.1 * rng.standard_normal(k)).astype(np.float32)
    w0 = rng.standard_normal((k, m0)).astype(np.float32); b0 = rng.standard_normal(m0).astype(np.float32)
    w1 = rng.standard_normal((k, max(m1, 1))).astype(np.float32)
    cache = rng.standard_normal((T, n, max(m1, 1))).astype(np.float32)
    outs = {}
    for name, nc, inv in (("inv", hip, 1), ("plain", hip, 0), ("ref", ref, 0)):
        if nc is hip:
            nc.nc_set_matmul_width_invariant(nc.ctx, inv)
        dst = nc.tensor(cache)
        pn = C.c_void_p()
        y0 = nc.nc_norm_linear_pair_into(nc.tensor(x), nc.tensor(g), nc.tensor(b), 1e-5, avg, nc.tensor(w0), nc.tensor(b0), act,
                                         nc.tensor(w1) if m1 else None, dst if m1 else None, T - 1, C.byref(pn))
        outs[name] = (nc.numpy(y0, free=True), nc.numpy(pn, free=True), nc.numpy(dst, free=True))
        if nc is hip and inv:
            xn = nc.nc_fused_layer_norm(nc.tensor(x), nc.tensor(g), nc.tensor(b), 1e-5, avg)
            xn_np = nc.numpy(xn)
            y = nc.nc_linear(nc.tensor(w0), nc.nc_dup_tensor(xn), nc.tensor(b0), act)
            y1 = nc.nc_matmul(nc.tensor(w1), xn) if m1 else None
            outs["steps"] = (nc.numpy(y, free=True), xn_np, nc.numpy(y1, free=True) if m1 else None)
            if not m1:
                nc.nc_free_tensor(xn)
        if nc is hip:
            nc.nc_set_matmul_width_invariant(nc.ctx, 0)
    assert np.array_equal(outs["inv"][1].view(np.uint32), outs["steps"][1].view(np.uint32))
    assert np.array_equal(outs["inv"][0].view(np.uint32), outs["steps"][0].view(np.uint32))
    if m1:
        assert np.array_equal(outs["inv"][2][T - 1].view(np.uint32), outs["steps"][2].view(np.uint32))
        assert np.array_equal(outs["inv"][2][:T - 1], cache[:T - 1])
    for name in ("inv", "plain"):
        for i in range(3 if m1 else 2):
            assert relerr(outs[name][i], outs["ref"][i]) <= TOL, (name, i)


@pytest.mark.parametrize("H,dk,B,T,M,d_pos,attn_len,has_w,t", [
    (8, 64, 32, 64, 64, 128, 128, 1, 63), (8, 64, 32, 64, 64, 128, 128, 1, 0), (8, 64, 4, 64, 64, 128, 100, 1, 17),
    (2, 32, 3, 9, 7, 13, 11, 1, 5), (2, 32, 3, 9, 7, 13, 16, 1, 8), (3, 64, 2, 20, 0, 20, 20, 1, 19),
    (2, 64, 5, 33, 40, 1, 50, 0, 32), (4, 32, 2, 64, 64, 128, 3, 1, 40)])
def test_one_query_attention_kernels_agree(hip, rng, H, dk, B, T, M, d_pos, attn_len, has_w, t):
    """nchip_relpos_attn_fwd_step: the vector-ALU kernel (fused multiply-add chains in the order
    an fp32 MFMA accumulates) writes the bits of the whole-segment kernel run with every query
    row the one query, and both are the attention of query t in float64 up to rounding."""
    lib = C.CDLL(hip.lib._name)
    st = C.c_void_p(hip.nc_context_stream(hip.ctx))
    K, D = M + T, H * dk
    q = rng.standard_normal((B, D)); kv = rng.standard_normal((T, B, 2 * D)); kvm = rng.standard_normal((max(M, 1), B, 2 * D))
    w_r = rng.standard_normal((H, d_pos, dk)); b_r = rng.standard_normal((H, K))
    b_r_scale = float(np.sqrt(dk * D))
    tens = {k: _dev(hip, v) for k, v in dict(q=q, kv=kv, kvm=kvm, w_r=w_r, b_r=b_r, o0=np.zeros((B, D)), o1=np.ones((B, D))).items()}
    P = {k: v[1] for k, v in tens.items()}
    i64, ci = C.c_int64, C.c_int
    try:
        for mode, out in ((0, "o0"), (1, "o1")):
            lib.nchip_relpos_attn_step_kernel(mode)
            assert lib.nchip_relpos_attn_fwd_step(st, P["q"], i64(D), P["kv"], P["kvm"] if M else None, i64(2 * D),
                                                  P["w_r"] if has_w else None, P["b_r"], P[out], i64(D), ci(H), ci(dk), ci(dk),
                                                  ci(B), ci(T), ci(M), ci(d_pos), ci(attn_len), C.c_float(b_r_scale), ci(t)) == 0
    finally:
        lib.nchip_relpos_attn_step_kernel(1)
    o0, o1 = hip.numpy(tens["o0"][0]), hip.numpy(tens["o1"][0])
    hip.free(*[v[0] for v in tens.values()])
    assert np.array_equal(o0.view(np.uint32), o1.view(np.uint32))
    f = lambda a: np.asarray(a, np.float32).astype(np.float64)
    keys = np.concatenate([f(kvm)[:M], f(kv)], axis=0)              # (K, B, 2D), memory first
    want = np.zeros((B, D))
    for h in range(H):
        for b in range(B):
            qv = f(q)[b, h * dk:(h + 1) * dk]
            js = [j for j in range(K) if 0 <= t + M - j < attn_len]
            sc = []
            for j in js:
                delta = t + M - j
                s_ = keys[j, b, h * dk:(h + 1) * dk] @ qv + b_r_scale * f(b_r)[h, K - 1 - delta]
                if has_w:
                    s_ += f(w_r)[h, max(d_pos - 1 - delta, 0)] @ qv
                sc.append(s_ / np.sqrt(dk))
            pr = np.exp(np.array(sc) - max(sc)); pr /= pr.sum()
            want[b, h * dk:(h + 1) * dk] = sum(p_ * keys[j, b, D + h * dk:D + (h + 1) * dk] for p_, j in zip(pr, js))
    assert relerr(o1, want) <= TOL


@pytest.mark.parametrize("d,n", [(512, 2048), (128, 80), (1024, 333), (256, 5)])
def test_norm_backward_leaves_the_row_sums_of_dx(hip, rng, d, n):
    """nchip_norm_bwd_rowsum: the partial rows it leaves sum, in row order, to the sum of the dx
    it wrote over the columns (what the bias gradient of the layer before the norm is), and dx
    itself is the bits of the plain call."""
    lib = C.CDLL(hip.lib._name)
    st = C.c_void_p(hip.nc_context_stream(hip.ctx))
    g = rng.standard_normal((n, d)); xhat = rng.standard_normal((n, d)); rstd = 0.5 + rng.random(n)
    w = 1.0 + 0.1 * rng.standard_normal(d); add = rng.standard_normal((n, d))
    rows = lib.nchip_norm_bwd_rows(C.c_int(d), C.c_int64(n))
    t = {k: _dev(hip, v) for k, v in dict(g=g, xhat=xhat, rstd=rstd, w=w, add=add, dx_a=np.zeros((n, d)), dx_b=np.ones((n, d)),
                                          part=np.full((rows, d), 7.0)).items()}
    P = {k: v[1] for k, v in t.items()}
    assert lib.nchip_norm_bwd(st, P["g"], P["xhat"], P["rstd"], P["w"], P["dx_a"], P["add"], None, None, None,
                              C.c_int(d), C.c_int64(n), C.c_int(1)) == 0
    assert lib.nchip_norm_bwd_rowsum(st, P["g"], P["xhat"], P["rstd"], P["w"], P["dx_b"], P["add"], None, None, None,
                                     C.c_int(d), C.c_int64(n), C.c_int(1), P["part"]) == 0
    dx_a, dx_b, part = (hip.numpy(t[k][0]) for k in ("dx_a", "dx_b", "part"))
    hip.free(*[v[0] for v in t.values()])
    assert np.array_equal(dx_a.view(np.uint32), dx_b.view(np.uint32))
    want = dx_b.astype(np.float64).sum(axis=0)
    assert relerr(part.astype(np.float64).sum(axis=0), want) <= 1e-6


@pytest.mark.parametrize("m,n,k", [(2048, 1024, 64), (512, 2048, 128), (300, 70, 96), (128, 4100, 64)])
def test_activation_gradient_product_leaves_its_row_sums(hip, rng, m, n, k):
    """nchip_gemm_dact_rowsum: C = (A^T B) .* gelu'(pre) as nchip_gemm_dact computes it, plus
    partial row sums of C whose total is the sum of C over its columns."""
    lib = C.CDLL(hip.lib._name)
    st = C.c_void_p(hip.nc_context_stream(hip.ctx))
    A = rng.standard_normal((m, k)) * 0.1      # stored (k rows, m columns): op(A) = A^T is m x k
    Bm = rng.standard_normal((n, k)) * 0.1     # (k, n)
    pre = rng.standard_normal((n, m))
    rows_cap = lib.nchip_gemm_rowsum_rows(C.c_int(n))
    t = {key: _dev(hip, v) for key, v in dict(A=A, B=Bm, pre=pre, Ca=np.zeros((n, m)), Cb=np.ones((n, m)),
                                              rs=np.full((rows_cap, m), 3.0)).items()}
    P = {key: v[1] for key, v in t.items()}
    NC_ACT_GELU = 1
    i64, f32, ci = C.c_int64, C.c_float, C.c_int
    assert lib.nchip_gemm_dact(st, ci(1), ci(0), ci(m), ci(n), ci(k), f32(1.0), P["A"], i64(k), P["B"], i64(k),
                               P["Ca"], i64(m), P["pre"], ci(NC_ACT_GELU), ci(0), ci(1), None) == 0
    written = C.c_int(-1)
    assert lib.nchip_gemm_dact_rowsum(st, ci(1), ci(0), ci(m), ci(n), ci(k), f32(1.0), P["A"], i64(k), P["B"], i64(k),
                                      P["Cb"], i64(m), P["pre"], ci(NC_ACT_GELU), ci(0), ci(1), None,
                                      P["rs"], C.byref(written)) == 0
    Ca, Cb, rs = (hip.numpy(t[key][0]) for key in ("Ca", "Cb", "rs"))
    hip.free(*[v[0] for v in t.values()])
    assert np.array_equal(Ca.view(np.uint32), Cb.view(np.uint32))
    assert 0 < written.value <= rows_cap
    want = Cb.astype(np.float64).sum(axis=0)
    got = rs[:written.value].astype(np.float64).sum(axis=0)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(Cb).sum(axis=0).max()
