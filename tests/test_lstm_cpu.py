"""The LSTM model class of the host mirror (nncp.c:1565-2330) on the CPU
checker: forward against a float64 numpy restatement for every cell type and
wiring option, per-timestep == whole-segment evaluation, state carried across
segments, whole-model gradient against a directional difference, stream round
trips in all modes."""
import numpy as np
import pytest

import modelutil as M
import nputil as U

SMALL = dict(n_layer=3, lstm_n_cells=12, batch_size=3, seg_len=5, n_symbols=17, seed=5, use_device=0, nb_threads=2)


@pytest.fixture(scope="module")
def H():
    return M.ref_host()


def _model(H, **kw):
    pkg = M.load_pkg()
    return pkg.host.Model(H, pkg.host.make_lstm_config(**dict(SMALL, **kw)))


def _sig(x):
    return 1.0 / (1.0 + np.exp(-x))


def lstm_forward_np(w, tokens, cfg, h0=None, c0=None):
    """tokens (T, B).  Returns probabilities (T, B, V) and the final (h, c) lists.
    Parameters in numpy order: matrices (in, out) [libnc (out, in)]."""
    T, B = tokens.shape
    L, C1 = cfg["n_layer"], cfg["lstm_n_cells"]
    C2 = cfg.get("lstm_n_cells2", C1)
    typ = cfg.get("lstm_type", 1)
    mats = 3 if typ == 2 else 4
    full, ln = cfg.get("lstm_full_connect", 1), cfg.get("lstm_use_layer_norm", 1)
    n_out = cfg.get("lstm_n_embed_out", L)
    h = [np.zeros((B, C1)) if h0 is None else h0[l].copy() for l in range(L)]
    c = [np.zeros((B, C2)) if c0 is None else c0[l].copy() for l in range(L)]
    outs = np.zeros((T, L, B, C1))
    for l in range(L):
        u, ws = w["u%d" % l].astype(np.float64), w["ws%d" % l].astype(np.float64)
        for t in range(T):
            pre = ws[tokens[t]]                                        # (B, mats*C2)
            if l > 0:
                below = np.concatenate([outs[t, i] for i in range(l)], axis=1) if (full and l > 1) else outs[t, l - 1]
                pre = pre + below @ w["w%d" % l].astype(np.float64)
            z = h[l] @ u + pre
            gate = []
            for j in range(mats):
                zj = z[:, j * C2:(j + 1) * C2]
                if ln:
                    zj = zj / np.sqrt((zj ** 2).mean(axis=1, keepdims=True) + 1e-5) * float(w["g%d_%d" % (l, j)])
                gate.append(zj + w["b%d_%d" % (l, j)].astype(np.float64))
            fg, inp, og = _sig(gate[0]), np.tanh(gate[1]), _sig(gate[2])
            if typ == 0:
                c[l] = c[l] * fg + inp * _sig(gate[3])
                hh = og * np.tanh(c[l])
            elif typ == 1:
                c[l] = c[l] * fg + np.minimum(1 - fg, _sig(gate[3])) * inp
                hh = og * c[l]
            else:
                c[l] = inp * (1 - fg) + c[l] * fg
                hh = og * c[l]
            if C2 != C1:
                hh = hh @ w["p%d" % l].astype(np.float64)
            h[l] = hh
            outs[t, l] = hh
    q, r = divmod(L, n_out)
    groups, k = [], 0
    for i in range(n_out):
        n = q + (i < r)
        groups.append(outs[:, k:k + n].sum(axis=1))
        k += n
    x = np.concatenate(groups, axis=2)                                 # (T, B, n_out*C1)
    logits = x @ w["fc_w"].astype(np.float64) + w["fc_b"].astype(np.float64)
    e = np.exp(logits - logits.max(axis=2, keepdims=True))
    return e / e.sum(axis=2, keepdims=True), h, c


VARIANTS = {
    "clamped_full_ln": dict(),
    "normal": dict(lstm_type=0),
    "tied": dict(lstm_type=2),
    "chain_no_ln": dict(lstm_full_connect=0, lstm_use_layer_norm=0, lstm_forget_bias=1.0),
    "projection": dict(lstm_n_cells2=20),
    "grouped_output": dict(lstm_n_embed_out=2),
    "one_layer": dict(n_layer=1),
}


@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_forward_matches_numpy_and_state_is_carried(H, name):
    cfg = dict(SMALL, **VARIANTS[name])
    m = _model(H, **VARIANTS[name])
    rng = np.random.default_rng(3)
    for k in m.param_names():                 # biases and gains away from their initial 0 / 1
        if k[0] in "bg" or k == "fc_b":
            m.set_param(k, m.get_param(k) + rng.standard_normal(m.get_param(k).shape).astype(np.float32) * 0.3)
    w = m.params()
    T, B, V = cfg["seg_len"], cfg["batch_size"], cfg["n_symbols"]
    tok1 = rng.integers(0, V, size=(T, B)).astype(np.int32)
    tok2 = rng.integers(0, V, size=(T, B)).astype(np.int32)
    p1 = m.eval(tok1)
    p2 = m.eval(tok2)                         # continues from the state the first segment left
    m.close()
    want1, h, c = lstm_forward_np(w, tok1, cfg)
    want2, _, _ = lstm_forward_np(w, tok2, cfg, h, c)
    np.testing.assert_allclose(p1, want1, rtol=2e-5, atol=2e-7)
    np.testing.assert_allclose(p2, want2, rtol=2e-5, atol=2e-7)
    assert np.abs(want2 - lstm_forward_np(w, tok2, cfg)[0]).max() > 1e-4   # the carried state matters


def test_timestep_and_segment_evaluation_agree(H):
    """T per-timestep evaluations (graph continued through h and c) == one segment
    evaluation: same probabilities, same loss, same weights after the update."""
    syms = M.markov1(3 * 5 * 4, 17, seed=11)
    res = []
    for mode in (0, 1):
        m = _model(H, sgd_opt=M.rmsprop())
        data, st = m.compress(syms, mode)
        res.append((st.loss_bits, m.params(), len(data)))
        m.close()
    assert abs(res[0][0] - res[1][0]) <= 1e-5 * abs(res[1][0])
    for k in res[1][1]:
        assert M.tensors_close(res[0][1][k], res[1][1][k], 1e-5), k


@pytest.mark.parametrize("n", [3 * 5 * 4, 3 * 5 * 3 + 8, 7])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_stream_round_trip(H, n, mode):
    syms = M.markov1(n, 17, seed=n)
    enc = _model(H)
    data, st = enc.compress(syms, mode)
    enc.close()
    dec = _model(H)
    out, _ = dec.decompress(data, n, mode)
    dec.close()
    assert np.array_equal(out, syms)
    assert st.n_symbols == n


def test_training_reduces_the_loss_and_gradient_matches_a_directional_difference(H):
    cfg = dict(SMALL)
    T, B, V = cfg["seg_len"], cfg["batch_size"], cfg["n_symbols"]
    rng = np.random.default_rng(8)
    tok = rng.integers(0, V, size=(T, B)).astype(np.int32)
    tgt = rng.integers(0, V, size=(T, B)).astype(np.int32)
    # plain SGD: w' = w - lr * g, so the step reveals the gradient (a large rate keeps the
    # fp32 rounding of w' small against lr * g)
    lr = 0.25
    m = _model(H, sgd_opt=M.sgd(lr))
    w0 = m.params()
    p, loss0 = m.train_step(tok, tgt, lr)
    w1 = m.params()
    m.close()

    def loss_of(w):   # mean negative log-likelihood, as lstm_eval_gradient scales it
        pr, _, _ = lstm_forward_np(w, tok, cfg)
        return -np.log(np.take_along_axis(pr, tgt[:, :, None].astype(np.int64), axis=2)).mean()
    g = {k: (w0[k].astype(np.float64) - w1[k].astype(np.float64)) / lr for k in w0}
    d = {k: rng.standard_normal(w0[k].shape) for k in w0}
    eps = 1e-4
    wp = {k: w0[k].astype(np.float64) + eps * d[k] for k in w0}
    wm = {k: w0[k].astype(np.float64) - eps * d[k] for k in w0}
    fd = (loss_of(wp) - loss_of(wm)) / (2 * eps)
    an = sum(float((g[k] * d[k]).sum()) for k in w0)
    assert abs(fd - an) <= 2e-3 * (abs(fd) + abs(an))
    assert abs(loss0 / (T * B) - loss_of({k: v.astype(np.float64) for k, v in w0.items()})) < 1e-5
    # a few more steps on a learnable stream lower the coded size
    syms = np.tile(np.arange(15, dtype=np.uint16), 40)
    m = _model(H)
    _, st = m.compress(syms, 1, lr=4e-3)
    first = st.loss_bits / st.n_steps
    _, st2 = m.compress(syms, 1, lr=4e-3)
    m.close()
    assert st2.loss_bits / st2.n_steps < 0.8 * first
