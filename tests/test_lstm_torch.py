"""Gradients of the LSTM model class (lstm_eval_gradient, nncp.c:2085-2170, on the CPU checker)
against autograd: the float64 forward of tests/test_lstm_cpu.py restated in torch, every cell
type and wiring option, per parameter tensor, on a first segment and on a second one that starts
from the carried (constant) state."""
import numpy as np
import pytest
import torch

import modelutil as M
from test_lstm_cpu import SMALL, VARIANTS, _model

LR = 0.25


def lstm_forward_torch(w, tokens, cfg, h0=None, c0=None):
    """tokens (T, B).  Returns log-probabilities (T, B, V) and the final (h, c) lists."""
    T, B = tokens.shape
    L, C1 = cfg["n_layer"], cfg["lstm_n_cells"]
    C2 = cfg.get("lstm_n_cells2", C1)
    typ = cfg.get("lstm_type", 1)
    mats = 3 if typ == 2 else 4
    full, ln = cfg.get("lstm_full_connect", 1), cfg.get("lstm_use_layer_norm", 1)
    n_out = cfg.get("lstm_n_embed_out", L)
    f64 = torch.float64
    h = [torch.zeros(B, C1, dtype=f64) if h0 is None else h0[l] for l in range(L)]
    c = [torch.zeros(B, C2, dtype=f64) if c0 is None else c0[l] for l in range(L)]
    tok = torch.as_tensor(tokens, dtype=torch.long)
    outs = [[None] * L for _ in range(T)]
    for l in range(L):
        for t in range(T):
            pre = w["ws%d" % l][tok[t]]
            if l > 0:
                below = torch.cat([outs[t][i] for i in range(l)], dim=1) if (full and l > 1) else outs[t][l - 1]
                pre = pre + below @ w["w%d" % l]
            z = h[l] @ w["u%d" % l] + pre
            gate = []
            for j in range(mats):
                zj = z[:, j * C2:(j + 1) * C2]
                if ln:
                    zj = zj / torch.sqrt((zj ** 2).mean(dim=1, keepdim=True) + 1e-5) * w["g%d_%d" % (l, j)]
                gate.append(zj + w["b%d_%d" % (l, j)])
            fg, inp, og = torch.sigmoid(gate[0]), torch.tanh(gate[1]), torch.sigmoid(gate[2])
            if typ == 0:
                c[l] = c[l] * fg + inp * torch.sigmoid(gate[3])
                hh = og * torch.tanh(c[l])
            elif typ == 1:
                c[l] = c[l] * fg + torch.minimum(1 - fg, torch.sigmoid(gate[3])) * inp
                hh = og * c[l]
            else:
                c[l] = inp * (1 - fg) + c[l] * fg
                hh = og * c[l]
            if C2 != C1:
                hh = hh @ w["p%d" % l]
            h[l] = hh
            outs[t][l] = hh
    q, r = divmod(L, n_out)
    rows = []
    for t in range(T):
        groups, k = [], 0
        for i in range(n_out):
            n = q + (i < r)
            groups.append(sum(outs[t][k:k + n]))
            k += n
        rows.append(torch.cat(groups, dim=1))
    x = torch.stack(rows)                                              # (T, B, n_out*C1)
    return torch.log_softmax(x @ w["fc_w"] + w["fc_b"], dim=2), h, c


@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_lstm_gradients_match_autograd(name):
    cfg = dict(SMALL, **VARIANTS[name])
    m = _model(M.ref_host(), sgd_opt=M.sgd(LR), **VARIANTS[name])
    rng = np.random.default_rng(4)
    for k in m.param_names():                 # biases and gains away from their initial 0 / 1
        if k[0] in "bg" or k == "fc_b":
            m.set_param(k, m.get_param(k) + rng.standard_normal(m.get_param(k).shape).astype(np.float32) * 0.3)
    T, B, V = cfg["seg_len"], cfg["batch_size"], cfg["n_symbols"]
    h = c = None
    for step in range(2):
        tok = rng.integers(0, V, size=(T, B)).astype(np.int32)
        tgt = rng.integers(0, V, size=(T, B)).astype(np.int32)
        w0 = m.params()
        w = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in w0.items()}
        logp, h, c = lstm_forward_torch(w, tok, cfg, h, c)
        nll = -logp.gather(2, torch.as_tensor(tgt, dtype=torch.long).unsqueeze(2)).mean()
        nll.backward()
        h, c = [x.detach() for x in h], [x.detach() for x in c]       # the next segment sees constants
        p, loss = m.train_step(tok, tgt, LR)
        w1 = m.params()
        assert M.relerr(p, logp.exp().detach().numpy()) <= 1e-5, step
        assert abs(loss / (T * B) - nll.item()) <= 1e-5 * nll.item(), step
        for k in w0:
            g, g_t = (w0[k].astype(np.float64) - w1[k]) / LR, w[k].grad.numpy()
            # the step reveals the gradient up to the fp32 spacing of the weights it is taken from
            spacing = np.sqrt(g.size) * 1.2e-7 * np.abs(w0[k]).max() / LR
            assert np.linalg.norm(g - g_t) <= 1e-4 * np.linalg.norm(g_t) + spacing, (step, k, M.rel_l2(g, g_t))
    m.close()
