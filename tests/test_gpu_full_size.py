"""GPU parity against the CPU checker at the sizes the throughput figures are quoted on:
the headline configuration (12 layers, d_model 512, 8 x 64, d_ff 2048, 64 + 64 keys, 32
streams, bytes) in full, and a two-layer model with the layer shape of the large-context
configuration (d_model 1024, 16 x 64, d_ff 4096, 64 + 192 keys, 16384 tokens).  Weights
N(0, 0.02) and data as bench.py draws them (nncp.c:581-1235 driven by host/trf_model.c on
both sides).

Bars.  From identical weights (step 1) probabilities, loss and every gradient tensor: 1e-5
against the checker (2e-2 for the bf16-operand variant).  Over several RMSProp steps two fp32
evaluations drift apart faster than that: the second-moment estimate starts at zero, so the
first updates are lr * g / (0.1 |g| + eps) - sign-like - and the rounding noise of gradients
that are sums of cancelling terms is amplified (zero-initialised vectors consist of nothing
else).  There a float64 evaluation of the same steps is the arbiter: the kernels must be
within the bar of it, or no further from it than 3x the checker's own distance (the same
order of rounding noise); randomly initialised matrices stay within the bar of the checker or
of the float64 evaluation itself, or within 3x the checker's own distance from the latter.  Compressed sizes: within 0.5 %."""
import os

import numpy as np
import pytest

import bench
import modelutil as M

pytestmark = pytest.mark.gpu

THREADS = min(os.cpu_count() or 1, 16)
LR = 3e-4
GRAD_LR = 64.0
C4_LAYER = dict(n_layer=2, d_model=1024, n_head=16, d_inner=4096, d_pos=256, mem_len=192, seg_len=64,
                batch_size=8, n_symbols=16384, seed=123)


@pytest.fixture(scope="module")
def hosts():
    return M.hip_host(), M.ref_host()


def _model(host, cfg, dev, bf16=0, opt=None):
    hp = M.load_pkg().host
    m = hp.Model(host, hp.make_config(**dict(cfg, use_device=dev, nb_threads=THREADS, fused=1,
                                             sgd_opt=opt or M.rmsprop(LR))))
    bench.init_weights(m)
    m.nc.nc_set_matmul_bf16(m.ctx, bf16)        # (the checker's switch is process-wide)
    return m


def _trajectory(m, batches, snapshots, lr=LR):
    """probabilities and loss of every step, all parameter tensors after the steps listed"""
    steps, weights = [], {}
    for step, (tok, tgt) in enumerate(batches, 1):
        steps.append(m.train_step(tok, tgt, lr))
        if step in snapshots:
            weights[step] = m.params()
    m.close()
    return steps, weights


def _matrices(w):
    return [k for k in w if w[k].ndim >= 2 and not k.startswith("b_r")]


def _joint(w, keys):
    return np.concatenate([w[k].ravel() for k in keys])


class Reference:
    """The checker's trajectories (fp32, and with its emulation of the bf16 operand rounding)
    and the float64 evaluation for one configuration; computed once per module."""

    def __init__(self, hosts, cfg, batches):
        last = len(batches)
        first = _model(hosts[1], cfg, 0)
        w0 = first.params()
        self.steps, self.weights = _trajectory(first, batches, (last,))
        self.steps_bf16, self.weights_bf16 = _trajectory(_model(hosts[1], cfg, 0, bf16=1), batches, (last,))
        _model(hosts[1], cfg, 0).close()                                   # switch back off
        self.exact_steps, self.exact_weights = M.float64_trajectory(cfg, w0, batches, (last,), LR, threads=THREADS)
        self.last = last
        # one plain-SGD step exposes the raw gradient as (w0 - w1) / lr; lr = 64 (a power of two,
        # so exact) lifts the update above the rounding of weights of size 0.02
        self.grad_probs, w1 = _trajectory(_model(hosts[1], cfg, 0, opt=M.sgd(GRAD_LR)), batches[:1], (1,), GRAD_LR)
        self.grads = {k: w0[k] - w1[1][k] for k in w0}
        self.w0 = w0


def _check_first_step(hosts, cfg, batches, ref, bf16, tol):
    """identical weights: probabilities, loss and every gradient against the checker"""
    steps, w1 = _trajectory(_model(hosts[0], cfg, 1, bf16=bf16, opt=M.sgd(GRAD_LR)), batches[:1], (1,), GRAD_LR)
    (ph, lh), (pr, lr_) = steps[0], ref.grad_probs[0]
    e = M.relerr(ph, pr)
    assert e <= tol, e
    assert abs(lh - lr_) <= tol * abs(lr_), (lh, lr_)
    for k in ref.grads:
        g = ref.w0[k] - w1[1][k]
        if bf16:
            assert M.rel_l2(g, ref.grads[k]) <= tol, (k, M.rel_l2(g, ref.grads[k]))
        else:
            assert M.tensors_close(g, ref.grads[k], tol), (k, M.rel_l2(g, ref.grads[k]))


def _check_steps(hosts, cfg, batches, ref, bf16, tol):
    """several RMSProp steps, float64 as the arbiter (module docstring)"""
    steps, weights = _trajectory(_model(hosts[0], cfg, 1, bf16=bf16), batches, (ref.last,))
    yard_steps = ref.steps_bf16 if bf16 else ref.steps
    yard_w = (ref.weights_bf16 if bf16 else ref.weights)[ref.last]
    e1 = M.relerr(steps[0][0], ref.steps[0][0])
    assert e1 <= tol, e1                                                 # step 1: directly
    yard = max(M.relerr(y[0], x[0]) for y, x in zip(yard_steps, ref.exact_steps))
    for s, ((ph, lh), (px, lx)) in enumerate(zip(steps, ref.exact_steps), 1):
        e = M.relerr(ph, px)
        assert M.within_or_no_worse(e, yard, tol), (s, e, yard)
        assert abs(lh - lx) <= max(tol, 1e-5) * abs(lx), (s, lh, lx)
    w, r, x = weights[ref.last], ref.weights[ref.last], ref.exact_weights[ref.last]
    mats = _matrices(r)
    vecs = [k for k in r if k not in mats]
    for k in mats:          # within the bar of the fp32 checker, or of the float64 evaluation itself,
        # or within 3x the checker's own distance from it, as for the vectors (embedding rows of
        # symbols seen a few times have gradients near eps / 0.1, where the first RMSProp updates
        # lr g / (0.1 |g| + eps) pass the relative rounding noise of g on undamped)
        e, ex, rx = M.rel_l2(w[k], r[k]), M.rel_l2(w[k], x[k]), M.rel_l2(r[k], x[k])
        assert min(e, ex) <= tol or M.within_or_no_worse(ex, rx, tol), (k, e, ex, rx)
    assert M.rel_l2(_joint(w, list(r)), _joint(r, list(r))) <= tol
    yard_v = max(M.rel_l2(yard_w[k], x[k]) for k in vecs)
    for k in vecs:
        e = M.rel_l2(w[k], x[k])
        assert M.within_or_no_worse(e, yard_v, tol), (k, e, yard_v)


# ---- headline configuration --------------------------------------------------------------

@pytest.fixture(scope="module")
def c3_batches():
    cfg = bench.C3
    syms = bench.markov3_dirichlet(cfg["batch_size"] * cfg["seg_len"] * 4, seed=77)
    return M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], 4)


@pytest.fixture(scope="module")
def c3_ref(hosts, c3_batches):
    return Reference(hosts, bench.C3, c3_batches)


@pytest.mark.parametrize("variant,tol", [("fp32", 1e-5), ("bf16", 2e-2)])
def test_c3_full_size_first_step_matches_checker(hosts, c3_batches, c3_ref, variant, tol):
    _check_first_step(hosts, bench.C3, c3_batches, c3_ref, int(variant == "bf16"), tol)


@pytest.mark.parametrize("variant,tol", [("fp32", 1e-5), ("bf16", 2e-2)])
def test_c3_full_size_four_steps(hosts, c3_batches, c3_ref, variant, tol):
    _check_steps(hosts, bench.C3, c3_batches, c3_ref, int(variant == "bf16"), tol)


def test_c3_full_size_compressed_size_within_half_a_percent(hosts):
    """16 trained segments of the order-3 Markov stream: the GPU's fast stream (whole-segment
    evaluation, 16-bit CDF coder), fp32 and bf16-operand variant, against the checker running
    the reference-faithful float coder; sizes within 0.5 %, summed code length of the fp32
    stream within 1e-4, and both GPU streams decode."""
    hp = M.load_pkg().host
    cfg = bench.C3
    n = cfg["batch_size"] * cfg["seg_len"] * 16
    syms = bench.markov3_dirichlet(n, seed=78)
    ref = _model(hosts[1], cfg, 0)
    data_ref, st_ref = ref.compress(syms, hp.MODE_SEGMENT | hp.CODER_FLOAT)
    ref.close()
    for bf16 in (0, 1):
        enc = _model(hosts[0], cfg, 1, bf16=bf16)
        data, st = enc.compress(syms, hp.MODE_SEGMENT | hp.CODER_CDF16)
        enc.close()
        assert abs(len(data) - len(data_ref)) <= 0.005 * len(data_ref), (bf16, len(data), len(data_ref))
        if not bf16:
            assert abs(st.loss_bits - st_ref.loss_bits) <= 1e-4 * st_ref.loss_bits
        dec = _model(hosts[0], cfg, 1, bf16=bf16)
        back, _ = dec.decompress(data, n, hp.MODE_SEGMENT | hp.CODER_CDF16)
        dec.close()
        assert np.array_equal(back, syms), bf16


# ---- layers of the large-context configuration -------------------------------------------

@pytest.fixture(scope="module")
def c4_batches():
    cfg = C4_LAYER
    syms = bench.bigram_zipf_dirichlet(cfg["batch_size"] * cfg["seg_len"] * 2, n_symbols=cfg["n_symbols"], seed=79)
    return M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], 2)


@pytest.fixture(scope="module")
def c4_ref(hosts, c4_batches):
    return Reference(hosts, C4_LAYER, c4_batches)


@pytest.mark.parametrize("variant,tol", [("fp32", 1e-5), ("bf16", 2e-2)])
def test_c4_layer_shape_first_step_matches_checker(hosts, c4_batches, c4_ref, variant, tol):
    _check_first_step(hosts, C4_LAYER, c4_batches, c4_ref, int(variant == "bf16"), tol)


@pytest.mark.parametrize("variant,tol", [("fp32", 1e-5), ("bf16", 2e-2)])
def test_c4_layer_shape_two_steps(hosts, c4_batches, c4_ref, variant, tol):
    _check_steps(hosts, C4_LAYER, c4_batches, c4_ref, int(variant == "bf16"), tol)


# ---- layers of the enwik profile ----------------------------------------------------------
# nncp.c:2515-2572: d_model 1024, 8 heads of 128, gated GELU feed-forward of 3072, RMSNorm in
# front of every block and after the last, 64 + 256 keys with one position vector per key
# (d_pos = 320), position matrices per layer (tied_w_r = 0), position biases shared.  Two such
# layers, 8 streams; weights and data as above.

ENWIK_LAYER = dict(n_layer=2, d_model=1024, n_head=8, d_inner=3072, ff_act=2, d_pos=320, mem_len=256, seg_len=64,
                   batch_size=8, n_symbols=256, ln_flags=2 | 4 | 16, use_bias=1, use_w_r=1, tied_w_r=0, tied_b_r=1,
                   seed=123)


@pytest.fixture(scope="module")
def enwik_batches():
    cfg = ENWIK_LAYER
    syms = bench.markov3_dirichlet(cfg["batch_size"] * cfg["seg_len"] * 2, seed=80)
    return M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], 2)


@pytest.fixture(scope="module")
def enwik_ref(hosts, enwik_batches):
    return Reference(hosts, ENWIK_LAYER, enwik_batches)


@pytest.mark.parametrize("variant,tol", [("fp32", 1e-5), ("bf16", 2e-2)])
def test_enwik_layer_shape_first_step_matches_checker(hosts, enwik_batches, enwik_ref, variant, tol):
    _check_first_step(hosts, ENWIK_LAYER, enwik_batches, enwik_ref, int(variant == "bf16"), tol)


@pytest.mark.parametrize("variant,tol", [("fp32", 1e-5), ("bf16", 2e-2)])
def test_enwik_layer_shape_two_steps(hosts, enwik_batches, enwik_ref, variant, tol):
    """(the second step attends to the first step's 64 hidden states in the memory)"""
    _check_steps(hosts, ENWIK_LAYER, enwik_batches, enwik_ref, int(variant == "bf16"), tol)
