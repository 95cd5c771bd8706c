"""Strict bars beyond the first step, and the two largest configurations at their full size.

Re-synchronised trajectory.  Over several RMSProp steps two correct fp32 evaluations drift
apart (the second moment starts at zero, so the first updates are sign-like and amplify the
rounding noise of near-zero gradients); comparing free-running trajectories therefore needs
an arbiter (tests/test_gpu_full_size.py).  Here nothing is arbitrated: before EVERY step the
GPU model is put into the checker's state of that moment - parameters, RMSProp second
moments, per-layer memories (nncp.c:1205-1235 carries exactly these from step to step) - so
each step starts from identical inputs and is held to the single-step bars against the
checker directly: probabilities and loss 1e-5 (2e-2 for the bf16-operand variant against the
checker's emulation of the same rounding), every gradient tensor 1e-5 / 2e-2 in relative L2
(plus one unit of the arithmetic's resolution at the size that tensor's gradient had while
it was healthy: see the loop), the second moments after the update likewise, and from the
second step on every parameter matrix after the update.  Gradients are read through a plain-SGD probe:
from the same parameters and memories one step with lr = 2^24 (a power of two: lr g is exact)
gives lr g = w - w' on both sides, the difference taken in float64.  The step is that large so
that w' = fl(w - lr g) keeps the gradient's own digits: with a small step the rounding of w'
to fp32 (2^-24 |w|) swamps gradients that have all but vanished (after three steps some
query-projection gradients are below 1e-7), and the comparison would measure the probe.  The parameters after the RMSProp update are not compared with
the checker's at that bar - where the two gradients disagree in sign, which fp32 summation
order decides for elements that are rounding noise around zero, the sign-like first updates
differ by up to 2 lr / sqrt(1 - beta2), and that is all they may differ by - but with the
RMSProp formula applied, in float64, to the GPU's own gradient and the moments going in.

Full-size configurations[3] (20 layers, d_model 1024, batch 64, 16384 tokens): no CPU
evaluation of that size fits a test, so it is checked through the stream's own properties -
encode two segments, decode them by replay, the decoder returns the input and ends with the
encoder's parameters bit for bit; encoding twice gives the same bytes.  configurations[4]
(64 x 16384 logits, 10^6 lookups per stream): equality with the checker, integer for integer.
"""
import os

import numpy as np
import pytest

import bench
import modelutil as M

pytestmark = pytest.mark.gpu

THREADS = min(os.cpu_count() or 1, 16)
LR, BETA2 = 3e-4, 0.99
GRAD_LR = float(2 ** 24)


def _model(host, cfg, dev, bf16=0, opt=None, weights=True):
    hp = M.load_pkg().host
    m = hp.Model(host, hp.make_config(**dict(cfg, use_device=dev, nb_threads=THREADS, fused=1,
                                             sgd_opt=opt or M.rmsprop(LR))))
    if weights:
        bench.init_weights(m)
    m.nc.nc_set_matmul_bf16(m.ctx, bf16)        # (the checker's switch is process-wide)
    return m


def _resync(cfg, batches, bf16, tol, hosts, every=1):
    """the checker runs freely; the GPU restarts every step from the checker's state"""
    gpu_host, ref_host = hosts
    chk = _model(ref_host, cfg, 0, bf16=bf16)
    chk_sgd = _model(ref_host, cfg, 0, bf16=bf16, opt=M.sgd(GRAD_LR), weights=False)
    gpu = _model(gpu_host, cfg, 1, bf16=bf16, weights=False)
    gpu_sgd = _model(gpu_host, cfg, 1, bf16=bf16, opt=M.sgd(GRAD_LR), weights=False)
    step_max = 2 * LR / np.sqrt(1 - BETA2)
    worst = dict(p=0.0, g=0.0, v=0.0, w=0.0)   # g: as a fraction of its bar
    scale = {}
    try:
        for s, (tok, tgt) in enumerate(batches, 1):
            st = chk.state()
            p_r, l_r = chk.train_step(tok, tgt, LR)
            if (s - 1) % every and s != len(batches):
                continue
            after = chk.state()
            gpu.load_state(st)
            p_g, l_g = gpu.train_step(tok, tgt, LR)
            e = M.relerr(p_g, p_r)
            worst["p"] = max(worst["p"], e)
            assert e <= tol, ("probabilities", s, e)
            assert abs(l_g - l_r) <= max(tol, 1e-5) * abs(l_r), ("loss", s, l_g, l_r)
            # gradients of this very step through the plain-SGD probes (no moments involved)
            probe = dict(w=st["w"], v={}, mem=st["mem"])
            chk_sgd.load_state(probe)
            gpu_sgd.load_state(probe)
            chk_sgd.train_step(tok, tgt, GRAD_LR)
            gpu_sgd.train_step(tok, tgt, GRAD_LR)
            now = gpu.state()
            for k, w in st["w"].items():
                w64_ = w.astype(np.float64)
                g_r, g_g = w64_ - chk_sgd.get_param(k), w64_ - gpu_sgd.get_param(k)
                # The bar: tol of the gradient's norm, plus one unit of fp32 (bf16 for that
                # variant's operands) resolution of the largest norm this tensor's gradient has
                # had so far.  The terms that sum to a gradient keep their size while the sum
                # itself may all but vanish (query projections once the attention saturates:
                # 1e-9 after eight steps against 1e-5 at the first); what is left of such a
                # sum is rounding residue on both sides, further from a float64 evaluation than
                # the two are from each other.
                norm_r = float(np.linalg.norm(g_r))
                scale[k] = max(scale.get(k, 0.0), norm_r)
                eg = float(np.linalg.norm(g_g - g_r))
                bar = tol * norm_r + (2.0 ** -9 if bf16 else 2.0 ** -23) * scale[k]
                worst["g"] = max(worst["g"], eg / bar)
                assert eg <= bar, ("gradient", s, k, eg / (norm_r + 1e-300), norm_r / scale[k])
                if not bf16 and norm_r >= 1e-2 * scale[k]:
                    assert M.tensors_close(g_g, g_r, tol), ("gradient", s, k, M.rel_l2(g_g, g_r))
                # from the second step on the second moments are there, an element's update is
                # no longer sign-like, and the parameters after the update are held to the bar
                # directly (matrices; zero-initialised vectors stay sign-like for longer)
                if s >= 2 and w.ndim >= 2 and not k.startswith("b_r"):
                    ew = M.rel_l2(now["w"][k], after["w"][k])
                    worst["w"] = max(worst["w"], ew)
                    assert ew <= tol, ("parameters after the update", s, k, ew)
                ev = M.rel_l2(now["v"][k], after["v"][k])
                worst["v"] = max(worst["v"], ev)
                assert ev <= 2.5 * tol, ("second moment", s, k, ev)     # v holds g^2: twice the relative error
                d = np.abs(now["w"][k].astype(np.float64) - after["w"][k])
                assert d.max() <= step_max * 1.001, ("update", s, k, d.max())
                # ... and it is the RMSProp update of the GPU's own gradient (nncp's optimiser
                # settings: beta2 0.99, eps 1e-8), evaluated here in float64
                g64, w64 = g_g.astype(np.float64) / GRAD_LR, w.astype(np.float64)
                v_new = BETA2 * st["v"][k].astype(np.float64).reshape(w.shape) + (1 - BETA2) * g64 * g64
                upd = LR * g64 / (np.sqrt(v_new) + 1e-8)
                got = w64 - now["w"][k]
                # (g64 carries the rounding of w' = fl(w - lr g): 2^-24 max(|w|, |lr g|) / lr per element)
                dg = np.maximum(np.abs(w64), np.abs(g_g)) * 2.0 ** -24 / GRAD_LR + 1e-30
                slack = LR * dg / (np.sqrt(v_new) + 1e-8) * 4 + 1e-3 * np.abs(upd) + 2.0 ** -23 * np.abs(w64)
                assert (np.abs(got - upd) <= slack).all(), ("update is not RMSProp of the gradient", s, k,
                                                            float(np.abs(got - upd).max()))
            for a, b in zip(now["mem"], after["mem"]):
                assert M.relerr(a, b) <= tol, ("memory", s)
    finally:
        for m in (chk, chk_sgd, gpu, gpu_sgd):
            m.close()
        _model(ref_host, M.TINY, 0).close()                              # the checker's bf16 switch back off
    return worst


@pytest.fixture(scope="module")
def hosts():
    return M.hip_host(), M.ref_host()


@pytest.mark.parametrize("variant,tol", [("fp32", 1e-5), ("bf16", 2e-2)])
def test_c3_full_size_eight_resynchronised_steps(hosts, variant, tol):
    cfg = bench.C3
    syms = bench.markov3_dirichlet(cfg["batch_size"] * cfg["seg_len"] * 8, seed=81)
    batches = M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], 8)
    worst = _resync(cfg, batches, int(variant == "bf16"), tol, hosts)
    print("worst over 8 steps:", worst)


def test_c1_hundred_resynchronised_steps(hosts):
    """configurations[0]'s model, 100 steps of its order-1 Markov stream; every 9th step (and
    the last) is compared, the checker's state going in each time."""
    cfg = M.C1
    syms = M.markov1(cfg["batch_size"] * cfg["seg_len"] * 100, cfg["n_symbols"], seed=82)
    batches = M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], 100)
    worst = _resync(cfg, batches, 0, 1e-5, hosts, every=9)
    print("worst over 100 steps:", worst)


# ---- configurations[3] at full depth and batch -------------------------------------------

@pytest.mark.parametrize("variant", ["bf16", "fp32"])
def test_c4_full_size_stream_properties(hosts, variant):
    hp = M.load_pkg().host
    cfg = bench.C4
    bf16 = int(variant == "bf16")
    n = cfg["batch_size"] * cfg["seg_len"] * 2
    syms = bench.bigram_zipf_dirichlet(n, n_symbols=cfg["n_symbols"], seed=83)
    mode = hp.MODE_SEGMENT | hp.CODER_CDF16
    enc = _model(hosts[0], cfg, 1, bf16=bf16)
    data, st = enc.compress(syms, mode)
    w_enc = {k: enc.get_param(k) for k in ("embed", "embed_out", "w_q_0", "ff2_19", "ln_g_39", "b_r_0")}
    enc.close()
    # every 16-bit CDF keeps each symbol at a count of 1 or more: at most 16 bits a token
    assert 0 < len(data) <= 2 * n + 64
    # an untrained model: the first segment is coded at log2(V) + (variance of random logits),
    # the second after one sign-like RMSProp step that overshoots - near the coder's cap
    bits = st.loss_bits / n
    assert np.isfinite(bits) and 6.0 < bits < 17.0, bits
    # (the summed code length of the float probabilities is an upper bound here: the CDF's
    # floor of one count makes symbols below 2^-16 cheaper than their probability)
    assert len(data) * 8 <= 1.02 * st.loss_bits + 1024, (len(data) * 8, st.loss_bits)
    again = _model(hosts[0], cfg, 1, bf16=bf16)
    data2, _ = again.compress(syms, mode)
    again.close()
    assert np.array_equal(data, data2)                 # run-to-run deterministic
    dec = _model(hosts[0], cfg, 1, bf16=bf16)
    back, _ = dec.decompress(data, n, mode)            # replay decoder: T + 1 evaluations per segment
    assert np.array_equal(back, syms)
    for k, w in w_enc.items():                         # the decoder replayed the training bit for bit
        assert np.array_equal(dec.get_param(k).view(np.uint32), w.view(np.uint32)), k
    dec.close()


# ---- configurations[4] at full size -------------------------------------------------------

def test_c5_full_size_cdf_and_lookups_equal_the_checker(hip, ref):
    """64 streams x 16384 logits (N(0, 3) plus the Zipf-shaped bias of bench.py) -> 16-bit CDF,
    then 10^6 uniform targets per stream: every CDF entry and every one of the 6.4 x 10^7
    symbols equals the checker's."""
    V, n, m = 16384, 64, 1000000
    rng = np.random.default_rng(5)
    bias = -np.log(rng.permutation(V) + 1.0)
    logits = (rng.normal(0, 3, (n, V)) + bias).astype(np.float32)
    targets = rng.integers(0, 65536, size=(n, m)).astype(np.uint16)
    targets[:, :4] = [0, 65535, 1, 65534]
    res = []
    for nc in (hip, ref):
        cdf = nc.nc_soft_max_cdf16(nc.tensor(logits))
        c = nc.numpy(cdf)
        res.append((c, nc.numpy(nc.nc_cdf_lookup(cdf, nc.tensor(targets)), free=True)))
    assert np.array_equal(res[0][0], res[1][0])
    assert np.array_equal(res[0][1], res[1][1])
    c = res[0][0].astype(np.int64)
    freq = np.diff(np.concatenate([c, np.full((n, 1), 65536)], axis=1), axis=1)
    assert (c[:, 0] == 0).all() and (freq >= 1).all() and (freq.sum(axis=1) == 65536).all()
