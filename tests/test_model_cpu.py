"""Model-level behaviour of the host mirror on the CPU checker: the stream
round-trips, per-timestep and whole-segment evaluation agree (nncp.c's
seq_eval invariant), the fused entry points reproduce the op-by-op path, and
the whole-model gradient matches a directional finite difference."""
import os

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


@pytest.mark.parametrize("n", [3 * 8 * 5, 3 * 8 * 4 + 17, 11, 3 * 8 - 1, 0, 1, 2])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_stream_round_trip(H, n, mode):
    """encode -> decode identity incl. block_len % B != 0, a tail shorter than
    a segment, a block shorter than one segment, fewer symbols than streams and
    the empty block; all four mode/coder pairs."""
    syms = M.markov1(max(n, 1), 40, seed=n)[:n]
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


# ---- retrain passes with dropout (nncp.c:2821-2941, 290-298) ----------------------
def test_fifo_symbol_is_oldest_first(H):
    """nncp_fifo_symbol against a plain Python FIFO: index 0 is the oldest symbol
    held, also after the ring has wrapped; negative indices read 0."""
    import ctypes as C
    rng = np.random.default_rng(5)
    size = 13
    ring = np.zeros(size, dtype=np.uint16)
    fifo, pos = [], 0
    for step in range(40):
        v = int(rng.integers(1, 1000))
        ring[pos] = v
        pos = (pos + 1) % size
        fifo = (fifo + [v])[-size:]
        held = len(fifo)
        # the reference passes (buffer, next write position, symbols held)
        for idx in {-2, -1, 0, min(1, held - 1), held // 2, held - 1}:
            want = 0 if idx < 0 else fifo[idx]
            got = H.lib.nncp_fifo_symbol(ring.ctypes.data_as(C.c_void_p), pos % held, held, idx)
            assert got == want, (step, idx)


@pytest.mark.parametrize("fused", [0, 1])
@pytest.mark.parametrize("own_lr", [False, True])
def test_retrain_round_trip(H, fused, own_lr):
    """Three blocks through one coder with a retrain pass (dropout on) after
    each: the decoder, replaying the passes on what it decoded, recovers the
    input and ends with the encoder's weights, bit for bit."""
    B, T = M.TINY["batch_size"], M.TINY["seg_len"]
    block = B * T * 3 + 5
    syms = M.markov1(3 * block - 7, 40, seed=21)
    kw = dict(fused=fused, sgd_opt=M.rmsprop(), dropout_prob=0.1, dropout_att_prob=0.05,
              retrain_period=1, retrain_len=2 * block)
    if own_lr:
        kw["retrain_lr"] = 1e-4
    enc = _model(H, **kw)
    data, st, rst = enc.compress_blocks(syms, block, 1)
    w_enc, steps_enc = enc.params(), enc.L.nncp_model_train_step(enc.ptr)
    enc.close()
    dec = _model(H, **kw)
    out, _, rst_d = dec.decompress_blocks(data, len(syms), block, 1)
    w_dec = dec.params()
    dec.close()
    assert np.array_equal(out, syms)
    for k in w_enc:
        assert np.array_equal(w_enc[k], w_dec[k]), k
    # passes over 1, 2 and 2 blocks of the buffer, (3 or 6) whole segments each... counted, not assumed:
    assert rst.n_steps == rst_d.n_steps > 0 and rst.n_symbols == rst.n_steps * B * T
    coded_steps = st.n_steps
    assert steps_enc == (coded_steps if own_lr else coded_steps + rst.n_steps)


def test_retrain_changes_the_model_and_dropout_is_seeded(H):
    B, T = M.TINY["batch_size"], M.TINY["seg_len"]
    block = B * T * 2
    syms = M.markov1(2 * block, 40, seed=4)
    res = {}
    for name, kw in (("plain", {}), ("retrain", dict(retrain_period=1, retrain_len=block)),
                     ("drop_a", dict(retrain_period=1, retrain_len=block, dropout_prob=0.2)),
                     ("drop_b", dict(retrain_period=1, retrain_len=block, dropout_prob=0.2))):
        m = _model(H, sgd_opt=M.rmsprop(), **kw)
        data, _, rst = m.compress_blocks(syms, block, 1)
        res[name] = (data.tobytes(), m.get_param("ff1_0"), rst.n_steps)
        m.close()
    assert res["plain"][2] == 0 and res["retrain"][2] > 0
    assert res["plain"][0] != res["retrain"][0]          # the second block is coded by a retrained model
    assert not np.array_equal(res["retrain"][1], res["drop_a"][1])   # masks act
    assert res["drop_a"][0] == res["drop_b"][0] and np.array_equal(res["drop_a"][1], res["drop_b"][1])


def test_dropout_path_equals_plain_path_at_probability_zero(H):
    """With dropout_prob = 0 trf_set_retrain(1) changes nothing (nncp.c:1240),
    in particular a fused model keeps its fused path."""
    tok = M.markov1(3 * 8, 40, seed=9).astype(np.int32).reshape(8, 3)
    for fused in (0, 1):
        m = _model(H, fused=fused)
        p0 = m.eval(tok)
        m.L.trf_set_retrain(m.ptr, 1)
        p1 = m.eval(tok)
        m.close()
        assert np.array_equal(p0, p1)


def test_dropout_masks_scale_and_rate(H):
    """Inverted dropout: the expectation of the masked evaluation is the plain
    one; checked through the mean of the mask itself (0 or 1/(1-p))."""
    pkg = M.load_pkg()
    nc = pkg.binding.NC(M.REF_LIB, use_device=False)
    x = nc.tensor(np.zeros((200, 300), np.float32))
    rs = nc.lib.nc_rnd_init(None, 77)
    nc.lib.nc_tensor_set_dropout(x, 0.25, rs)
    m = nc.numpy(x, free=True)
    nc.lib.nc_rnd_end(rs)
    nc.close()
    vals = np.unique(m)
    assert len(vals) == 2 and vals[0] == 0 and abs(vals[1] - 1 / 0.75) < 1e-6
    assert abs((m == 0).mean() - 0.25) < 0.01 and abs(m.mean() - 1.0) < 0.02


def test_c1_prefix_reference_and_fast_streams_agree_in_size(H):
    """BASELINE config 1 (2 layers, d_model 128, 4 x 32, d_ff 512, T = M = 20, batch 4, RMSProp
    3e-4) on a prefix of its order-1 Markov bytes: the reference-faithful stream (one evaluation
    per timestep, float symbol coder, cp_utils.c:299-323) and the fast stream (whole-segment
    evaluation, 16-bit integer CDF) both round-trip, and their sizes agree within 0.5 %.  (On the
    full 64 KiB both come to 55 719 bytes, 6.80 bits per symbol, after 819 steps and a 4-symbol
    tail; that run takes two minutes on the checker and is not repeated here.)"""
    pkg = M.load_pkg()
    hp = pkg.host
    n = 4 * 20 * 25 + 13
    syms = M.markov1(65536, 256, seed=1234)[:n]
    sizes = {}
    for name, mode, fused in (("reference", 0, 0), ("fast", hp.MODE_SEGMENT | hp.CODER_CDF16, 1)):
        cfg = dict(M.C1, use_device=0, nb_threads=4, fused=fused, sgd_opt=M.rmsprop(3e-4))
        enc = hp.Model(H, hp.make_config(**cfg))
        data, st = enc.compress(syms, mode)
        enc.close()
        assert st.n_steps == 25 and st.n_symbols == n
        dec = hp.Model(H, hp.make_config(**cfg))
        back, _ = dec.decompress(data, n, mode)
        dec.close()
        assert np.array_equal(back, syms), name
        sizes[name] = len(data)
    assert abs(sizes["fast"] - sizes["reference"]) <= 0.005 * sizes["reference"], sizes


def test_symbols_outside_the_alphabet_are_refused_on_the_host(H):
    """Symbols index device tables unchecked, so the host turns them away first: the Python
    layer raises, the C block loop ends the process with a message (checked in a child)."""
    import subprocess
    import sys
    m = _model(H)
    bad = np.zeros((8, 3), dtype=np.int32)
    bad[2, 1] = 40                                     # alphabet of TINY is 0..39
    with pytest.raises(ValueError):
        m.eval(bad)
    with pytest.raises(ValueError):
        m.train_step(np.zeros((8, 3), dtype=np.int32), bad, 3e-4)
    m.close()
    code = ("import sys; sys.path.insert(0, %r); import numpy as np, modelutil as M\n"
            "pkg = M.load_pkg(); m = pkg.host.Model(M.ref_host(), pkg.host.make_config(**dict(M.TINY, use_device=0)))\n"
            "m.compress(np.array([1, 2, 40, 3], dtype=np.uint16), 0)") % (os.path.dirname(os.path.abspath(__file__)),)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert r.returncode != 0 and "outside the model's alphabet" in r.stderr
