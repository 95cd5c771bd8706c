"""Model-level behaviour of the host mirror on the CPU checker: the stream
round-trips, per-timestep and whole-segment evaluation agree (nncp.c's
seq_eval invariant), the fused entry points reproduce the op-by-op path, and
the whole-model gradient matches a directional finite difference."""
import numpy as np
import pytest

import modelutil as M


@pytest.fixture(scope="module")
def H():
    return M.ref_host()


def _model(H, **kw):
    pkg = M.load_pkg()
    base = dict(M.TINY, use_device=0, nb_threads=2)
    base.update(kw)
    return pkg.host.Model(H, pkg.host.make_config(**base))


@pytest.mark.parametrize("n", [3 * 8 * 5, 3 * 8 * 4 + 17, 11, 3 * 8 - 1])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_stream_round_trip(H, n, mode):
    """encode -> decode identity incl. block_len % B != 0, a tail shorter than
    a segment and a block shorter than one segment; all four mode/coder pairs."""
    syms = M.markov1(n, 40, seed=n)
    enc = _model(H)
    data, st = enc.compress(syms, mode)
    enc.close()
    dec = _model(H)
    out, _ = dec.decompress(data, n, mode)
    dec.close()
    assert np.array_equal(out, syms)
    assert st.n_symbols == n


def test_decoder_terminates_on_truncated_stream(H):
    syms = M.markov1(200, 40, seed=3)
    enc = _model(H)
    data, _ = enc.compress(syms, 0)
    enc.close()
    dec = _model(H)
    out, _ = dec.decompress(data[:len(data) // 2], 200, 0)  # zero padded past the end
    dec.close()
    assert out.shape == (200,) and (out < 40).all()
    assert not np.array_equal(out, syms)


def test_timestep_and_segment_evaluation_agree(H):
    """T per-timestep evaluations with merged backward == one segment
    evaluation: same probabilities, same weights after the update."""
    syms = M.markov1(3 * 8 * 3, 40, seed=11)
    res = []
    for mode in (0, 1):
        m = _model(H, sgd_opt=M.rmsprop())
        data, st = m.compress(syms, mode)
        res.append((st.loss_bits, m.params(), len(data)))
        m.close()
    assert abs(res[0][0] - res[1][0]) <= 1e-5 * abs(res[1][0])
    for k in res[0][1]:
        assert M.relerr(res[0][1][k], res[1][1][k]) <= 2e-5, k


@pytest.mark.parametrize("variant", [dict(), dict(ln_flags=2 | 4, ff_act=0, query_bias=1),
                                     dict(tied_w_r=0, tied_b_r=0, attn_len=[10, 16]),
                                     dict(use_w_r=0, ln_flags=1 | 16)])
def test_fused_path_matches_reference_path(H, variant):
    syms = M.markov1(3 * 8 * 3, 40, seed=5)
    batches = M.segment_batches(syms, 3, 8, 3)
    res = []
    for fused in (0, 1):
        m = _model(H, fused=fused, sgd_opt=M.rmsprop(3e-4), **variant)
        probs = [m.train_step(tok, tgt, 3e-4)[0] for tok, tgt in batches]
        res.append((probs, m.params()))
        m.close()
    for a, b in zip(res[0][0], res[1][0]):
        assert M.relerr(b, a) <= 1e-5
    for k in res[0][1]:
        assert M.relerr(res[1][1][k], res[0][1][k]) <= 1e-5, k


def test_whole_model_gradient_directional(H):
    syms = M.markov1(3 * 8, 40, seed=9)
    (tok, tgt), = M.segment_batches(syms, 3, 8, 1)
    lr = 1.0
    m = _model(H, sgd_opt=M.sgd(lr))
    w0 = m.params()
    _, loss0 = m.train_step(tok, tgt, lr)
    w1 = m.params()
    m.close()
    N = tok.size
    rng = np.random.default_rng(0)
    for name in ("w_q_0", "w_kv_1", "ff1_0", "w_r_0", "b_r_0", "ln_g_1", "embed", "embed_out", "w_o_1"):
        g = (w0[name] - w1[name]) / lr          # gradient of the mean loss
        d = rng.standard_normal(g.shape).astype(np.float32)
        d /= np.linalg.norm(d)
        eps = 2e-2
        vals = []
        for sign in (1, -1):
            mm = _model(H, sgd_opt=M.sgd(0.0))
            mm.set_param(name, w0[name] + sign * eps * d)
            _, l = mm.train_step(tok, tgt, 0.0)
            vals.append(l / N)
            mm.close()
        fd = (vals[0] - vals[1]) / (2 * eps)
        an = float((g * d).sum())
        assert abs(fd - an) <= 3e-2 * max(abs(an), 1e-3), (name, fd, an)


def test_probabilities_are_causal(H):
    """Column t of a segment evaluation does not depend on inputs after t
    (what lets a decoder replay whole-segment evaluations)."""
    rng = np.random.default_rng(1)
    tok = rng.integers(0, 40, size=(8, 3)).astype(np.int32)
    m = _model(H)
    p_full = m.eval(tok)
    for t in (0, 3, 7):
        tok2 = tok.copy()
        tok2[t + 1:] = 0
        p2 = m.eval(tok2)
        assert np.array_equal(p_full[:t + 1], p2[:t + 1])
    m.close()


def test_cached_timestep_evaluation_matches_segment(H):
    """trf_eval_step (K/V caches, fused entry points) reproduces the columns of
    the whole-segment evaluation, with a non-empty memory (second segment)."""
    syms = M.markov1(3 * 8 * 2, 40, seed=21)
    (tok0, tgt0), (tok1, _) = M.segment_batches(syms, 3, 8, 2)
    m = _model(H, fused=1, sgd_opt=M.rmsprop(3e-4))
    m.train_step(tok0, tgt0, 3e-4)  # fills the memory
    full = m.eval(tok1)
    full_logits = None
    step_p, step_l = m.eval_steps(tok1)
    m.eval(tok1, keep=True)
    full_logits = m.logits()
    m.L.trf_eval_end(m.ptr)
    m.close()
    assert step_p.shape == full.shape
    assert M.relerr(step_p, full) <= 1e-6
    assert M.relerr(step_l, full_logits) <= 1e-6


@pytest.mark.parametrize("n", [3 * 8 * 4 + 17, 11])
@pytest.mark.parametrize("coder", [0, 2])
def test_step_decode_round_trip(H, n, coder):
    """Whole-segment encoder, per-timestep cached decoder (NNCP_MODE_STEP_DECODE)."""
    mode = 1 | 4 | coder
    syms = M.markov1(n, 40, seed=n + 1)
    enc = _model(H, fused=1)
    data, st = enc.compress(syms, mode)
    enc.close()
    dec = _model(H, fused=1)
    out, _ = dec.decompress(data, n, mode)
    dec.close()
    assert np.array_equal(out, syms)
    assert st.n_symbols == n
