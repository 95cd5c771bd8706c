"""The whole Transformer-XL step of the host mirror + CPU checker against an
independent statement of the same mathematics in torch (CPU, float64), written
from the index-level formulas and not from the op sequence: relative-position
scores S[j,i] = (k_j.q_i + w_r[:, max(d_pos-1-d, 0), h].q_i + sqrt(dk*D) b_r[K-1-d, h]) / sqrt(dk)
with d = i + M - j, masked outside 0 <= d < attn_len (what nc_pad + nc_rel_shift +
the mask of nncp.c:352-365, 775-793 amount to), post-LayerNorm blocks
(nncp.c:896-987), mean negative log-likelihood (nncp.c:1170-1175) and the memory
shift of nncp.c:1205-1221.  Gradients come from autograd, so a dropped term, a
wrong sign or index, a transposed operand or a missing sum (memory columns of
w_kv, layers of the tied w_r / b_r, streams of w_r) in the checker's backward
shows up per parameter tensor."""
import math

import numpy as np
import pytest
import torch

import modelutil as M

CFG = dict(n_layer=2, d_model=32, n_head=2, d_inner=48, d_pos=6, mem_len=6, seg_len=4,
           batch_size=3, n_symbols=20, seed=11, query_bias=1, attn_len=[10, 7])
LN_POST, LN_PRE, LN_FINAL, LN_RMSNORM = 1, 2, 4, 16
FF_RELU, FF_GELU, FF_GEGLU = 0, 1, 2
VARIANTS = {
    # nncp's default structure (nncp.c:2489-2513) plus a query bias
    "default": dict(),
    # the structure of the enwik8 / enwik9 profiles (nncp.c:2515-2572): pre-norm with a final
    # norm, RMS norm, GEGLU, a position table per layer as long as the key axis
    "enwik": dict(ln_flags=LN_PRE | LN_FINAL | LN_RMSNORM, ff_act=FF_GEGLU, tied_w_r=0, d_pos=10, query_bias=0),
    # no position table (bias only, nncp.c:780-783), no bias vectors, ReLU
    "bare": dict(use_w_r=0, use_bias=0, ff_act=FF_RELU, query_bias=0),
}
LR = 0.5


def _norm(x, g, b, rms):
    if rms:
        return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + 1e-5) * g + b
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), g, b, 1e-5)


def _torch_step(w, cfg, tok, tgt, mem):
    """tok, tgt: (T, B) ints; mem: list of (B, M, D) tensors.  Returns
    (probabilities (T, B, V), mean nll, layer inputs [(T, B, D)])."""
    T, Bn = tok.shape
    D, H, Mlen, P = cfg["d_model"], cfg["n_head"], cfg["mem_len"], cfg["d_pos"]
    dk = D // H
    K = T + Mlen
    i = torch.arange(T).view(T, 1)
    j = torch.arange(K).view(1, K)
    delta = i + Mlen - j                                   # (T, K)
    pos_idx = (P - 1 - delta).clamp(min=0, max=P - 1)      # pi(delta); masked entries clamped into range
    bias_idx = (K - 1 - delta).clamp(min=0, max=K - 1)
    flags, act = cfg.get("ln_flags", LN_POST), cfg.get("ff_act", FF_GELU)
    rms = bool(flags & LN_RMSNORM)
    zero = torch.zeros((), dtype=torch.float64)
    x = w["embed"][torch.as_tensor(tok, dtype=torch.long)] * math.sqrt(D)
    inputs = []
    for l in range(cfg["n_layer"]):
        res = x
        if flags & LN_PRE:
            x = _norm(x, w["ln_g_%d" % (2 * l)], w["ln_b_%d" % (2 * l)], rms)
        inputs.append(x)                                   # what the memory keeps (nncp.c:647-657)
        q = (x @ w["w_q_%d" % l] + w.get("b_q_%d" % l, zero)).view(T, Bn, H, dk)
        kv_c = x @ w["w_kv_%d" % l]                        # (T, B, H*dk + H*dv)
        kv_m = mem[l] @ w["w_kv_%d" % l]                   # (B, M, ...): no gradient into the memory
        kv = torch.cat([kv_m, kv_c.transpose(0, 1)], dim=1)  # (B, K, ...), memory first
        k = kv[..., :H * dk].reshape(Bn, K, H, dk)
        v = kv[..., H * dk:].reshape(Bn, K, H, dk)
        s = torch.einsum("tbhd,bjhd->bhtj", q, k)
        if cfg.get("use_w_r", 1):
            w_r = w["w_r_%d" % (0 if cfg.get("tied_w_r", 1) else l)]  # tied: layer 0's table in every layer
            qr = torch.einsum("tbhd,hpd->bhtp", q, w_r)
            s = s + torch.gather(qr, 3, pos_idx.expand(Bn, H, T, K))
        b_r = w["b_r_%d" % (0 if cfg.get("tied_b_r", 1) else l)]      # tied: layer 0's bias in every layer
        s = s + math.sqrt(dk * D) * b_r[:, bias_idx].unsqueeze(0)
        s = s / math.sqrt(dk)
        valid = (delta >= 0) & (delta < cfg["attn_len"][l])
        s = s.masked_fill(~valid, float("-inf"))
        a = torch.softmax(s, dim=3)
        o = torch.einsum("bhtj,bjhd->tbhd", a, v).reshape(T, Bn, H * dk)
        x1 = o @ w["w_o_%d" % l] + res
        if flags & LN_POST:
            x1 = _norm(x1, w["ln_g_%d" % (2 * l)], w["ln_b_%d" % (2 * l)], rms)
        y = x1
        if flags & LN_PRE:
            y = _norm(y, w["ln_g_%d" % (2 * l + 1)], w["ln_b_%d" % (2 * l + 1)], rms)
        z = y @ w["ff1_%d" % l] + w.get("ff_bias1_%d" % l, zero)
        if act == FF_GEGLU:                                # first half gated by the second (nncp.c:950-956)
            F = cfg["d_inner"]
            z = torch.nn.functional.gelu(z[..., :F], approximate="tanh") * z[..., F:]
        elif act == FF_GELU:
            z = torch.nn.functional.gelu(z, approximate="tanh")
        else:
            z = torch.relu(z)
        x = z @ w["ff2_%d" % l] + w.get("ff_bias2_%d" % l, zero) + x1
        if flags & LN_POST:
            x = _norm(x, w["ln_g_%d" % (2 * l + 1)], w["ln_b_%d" % (2 * l + 1)], rms)
    if flags & LN_FINAL:
        x = _norm(x, w["ln_g_%d" % (2 * cfg["n_layer"])], w["ln_b_%d" % (2 * cfg["n_layer"])], rms)
    logits = x @ w["embed_out"] + w.get("out_bias", zero)
    logp = torch.log_softmax(logits, dim=2)
    nll = -logp.gather(2, torch.as_tensor(tgt, dtype=torch.long).unsqueeze(2)).mean()
    return logp.exp(), nll, inputs


@pytest.mark.parametrize("fused", [0, 1])
@pytest.mark.parametrize("variant", sorted(VARIANTS))
def test_three_steps_against_torch_autograd(variant, fused):
    pkg = M.load_pkg()
    cfg = dict(CFG, **VARIANTS[variant])
    model = pkg.host.Model(M.ref_host(), pkg.host.make_config(
        **dict(cfg, use_device=0, nb_threads=2, fused=fused, sgd_opt=M.sgd(LR))))
    rng = np.random.default_rng(3)
    # zero-initialised vectors and unit gains get values, so every term of the formulas counts
    for name in model.param_names():
        p = model.get_param(name)
        if name.startswith("ln_g"):
            model.set_param(name, (1.0 + 0.2 * rng.standard_normal(p.shape)).astype(np.float32))
        elif not p.any():
            model.set_param(name, (0.05 * rng.standard_normal(p.shape)).astype(np.float32))
    T, Bn, D, Mlen = cfg["seg_len"], cfg["batch_size"], cfg["d_model"], cfg["mem_len"]
    syms = M.markov1(Bn * T * 3, cfg["n_symbols"], seed=9)
    mem = [torch.zeros(Bn, Mlen, D, dtype=torch.float64) for _ in range(cfg["n_layer"])]
    for step, (tok, tgt) in enumerate(M.segment_batches(syms, Bn, T, 3)):
        w0 = model.params()
        if variant == "default":
            assert set(w0) == {"embed", "embed_out", "out_bias", "w_r_0", "b_r_0"} | {
                "%s_%d" % (n, l) for l in range(2)
                for n in ("w_q", "b_q", "w_kv", "w_o", "ff1", "ff_bias1", "ff2", "ff_bias2")
            } | {"ln_g_%d" % k for k in range(4)} | {"ln_b_%d" % k for k in range(4)}
        w = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in w0.items()}
        probs_t, nll_t, inputs = _torch_step(w, cfg, tok, tgt, mem)
        nll_t.backward()
        probs, loss = model.train_step(tok, tgt, LR)
        w1 = model.params()
        assert M.relerr(probs, probs_t.detach().numpy()) <= 5e-6, step
        assert abs(loss / (T * Bn) - nll_t.item()) <= 2e-5 * nll_t.item(), step
        for name in w0:
            g = (w0[name].astype(np.float64) - w1[name]) / LR
            g_t = w[name].grad.numpy()
            assert np.abs(g_t).max() > 0, name
            assert M.rel_l2(g, g_t) <= 1e-4, (step, name, M.rel_l2(g, g_t))
        # memory for the next segment: oldest T positions drop out, the layer inputs join at the end
        mem = [torch.cat([m[:, T:], x.detach().transpose(0, 1)], dim=1) for m, x in zip(mem, inputs)]
    model.close()
