"""Helpers shared by the model-level tests: configurations, seeded data."""
import ctypes as C
import os

import numpy as np

from conftest import ROOT, REF_LIB, load_pkg

HOST_REF = os.path.join(ROOT, "oracle", "libnncp_host_ref.so")

TINY = dict(n_layer=2, d_model=32, n_head=2, d_inner=64, d_pos=12, mem_len=8, seg_len=8,
            batch_size=3, n_symbols=40, seed=7)
# BASELINE config 1 (2 layers, d_model 128, 4 heads x 32, d_ff 512, T = M = 20, batch 4)
C1 = dict(n_layer=2, d_model=128, n_head=4, d_inner=512, d_pos=40, mem_len=20, seg_len=20,
          batch_size=4, n_symbols=256, seed=123)


def ref_host():
    pkg = load_pkg()
    return pkg.host.Host(HOST_REF, REF_LIB)


def hip_host():
    """The product pair of libraries, or - when tests/test_kernels_on_cpu.py re-runs
    GPU tests without a GPU - the same sources built for the host (tests/hipcpu)."""
    pkg = load_pkg()
    emu, emu_host = os.environ.get("NNCP_TEST_HIP_LIB"), os.environ.get("NNCP_TEST_HOST_HIP_LIB")
    host = pkg.host.Host(emu_host, emu) if emu and emu_host else pkg.host.Host()
    # The library's HIP runtime comes up now, before any test has a chance to let torch bring
    # up the copy it bundles (its autograd engine counts the devices at its first backward
    # pass): the runtime that initialises second in a process finds no device, and the
    # library then ends the process ("no HIP device 0 (found 0)").
    nc = host.ncl
    ctx = nc.nc_context_init(1)
    nc.nc_new_cuda_device(ctx, 0)
    nc.nc_context_end(ctx)
    return host


def rmsprop(lr=3e-4):
    B = load_pkg().binding
    return B.SGDOptParams(algo=B.SGD_OPT_RMSPROP, beta1=0.0, beta2=0.99, eps=1e-8, gradient_clip=0.0, lr=lr)


def sgd(lr):
    B = load_pkg().binding
    return B.SGDOptParams(algo=B.SGD_OPT_BASIC, lr=lr)


def markov1(n, n_symbols=256, seed=1234, s=1.1):
    """Order-1 Markov source, each row Zipf(s) over a seeded permutation
    (BASELINE config 1 data)."""
    rng = np.random.default_rng(seed)
    ranks = np.arange(1, n_symbols + 1, dtype=np.float64) ** -s
    ranks /= ranks.sum()
    cum = np.cumsum(ranks)
    perms = np.stack([rng.permutation(n_symbols) for _ in range(n_symbols)])
    u = rng.random(n)
    out = np.zeros(n, dtype=np.uint16)
    cur = 0
    for i in range(n):
        r = int(np.searchsorted(cum, u[i]))
        cur = perms[cur, min(r, n_symbols - 1)]
        out[i] = cur
    return out


def relerr(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / (np.abs(b).max() + 1e-30))


def segment_batches(syms, B, T, n_steps):
    """(tokens, targets) pairs laid out as process_block does for a block that
    is an exact multiple of B*T: stream b owns syms[b*stride:(b+1)*stride]."""
    stride = len(syms) // B
    st = syms[:stride * B].reshape(B, stride).astype(np.int32)
    out = []
    for k in range(n_steps):
        tgt = st[:, k * T:(k + 1) * T]                       # (B, T)
        prev = np.concatenate([np.zeros((B, 1), np.int32) if k == 0 else st[:, k * T - 1:k * T],
                               tgt[:, :-1]], axis=1)
        out.append((prev.T.copy(), tgt.T.copy()))            # numpy (T, B)
    return out


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / (np.linalg.norm(b) + 1e-30))


def tensors_close(a, b, tol=1e-5, max_factor=30, outliers=1e-4):
    """Agreement bar for gradient and weight tensors: relative L2 error <= tol.
    Element-wise (relative to max|b|) the bound is max_factor*tol for all but a
    fraction `outliers` of the elements (at least one), and 4*max_factor*tol
    for those: single elements that are sums of cancelling terms (tiny
    gradients), and weights moved by the sign-like RMSProp update
    lr*g/(sqrt(v)+eps) of such elements, differ by fp32 re-ordering noise that
    is large relative to the element but not to the tensor (measured:
    gradients <= 5.4e-5; weights after 10 steps <= 4.2e-4 on 1 element of
    32768, all others <= 1.8e-4; every tensor <= 7.8e-6 in relative L2)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    scale = max(np.abs(b).max(), 1e-30)
    d = np.abs(a - b) / scale
    n_out = int((d > max_factor * tol).sum())
    return (rel_l2(a, b) <= tol and d.max() <= 4 * max_factor * tol
            and n_out <= max(1, int(outliers * d.size)))


def float64_trajectory(cfg, w0, batches, snapshots, lr=3e-4, beta2=0.99, eps=1e-8, threads=None):
    """The same RMSProp training steps evaluated in float64 by the torch statement of
    tests/test_model_torch.py (index-level formulas, autograd gradients), from the weights
    w0 and an empty memory.  Returns ([(probabilities (T, B, V), loss summed over the
    segment)], {step: {name: weights}}).  It is the arbiter where two fp32 evaluations differ
    by more than the bar: fp32 rounding noise, amplified by the sign-like RMSProp update of
    small gradients, is then measured on both sides against it."""
    import torch
    from test_model_torch import _torch_step
    if threads:
        torch.set_num_threads(threads)
    cfg = dict(cfg)
    cfg.setdefault("attn_len", [cfg["mem_len"] + cfg["seg_len"]] * cfg["n_layer"])
    B, T, D = cfg["batch_size"], cfg["seg_len"], cfg["d_model"]
    w = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in w0.items()}
    v2 = {k: torch.zeros_like(t) for k, t in w.items()}
    mem = [torch.zeros(B, cfg["mem_len"], D, dtype=torch.float64) for _ in range(cfg["n_layer"])]
    steps, weights = [], {}
    for step, (tok, tgt) in enumerate(batches, 1):
        probs, nll, inputs = _torch_step(w, cfg, tok, tgt, mem)
        nll.backward()
        with torch.no_grad():
            for k in w:
                g = w[k].grad
                v2[k] = beta2 * v2[k] + (1 - beta2) * g * g
                w[k] -= lr * g / (v2[k].sqrt() + eps)
                w[k].grad = None
        mem = [torch.cat([m[:, T:], x.detach().transpose(0, 1)], dim=1) for m, x in zip(mem, inputs)]
        steps.append((probs.detach().numpy(), nll.item() * B * T))
        if step in snapshots:
            weights[step] = {k: t.detach().numpy().copy() for k, t in w.items()}
    return steps, weights


def within_or_no_worse(err, yardstick, tol, factor=3.0):
    """err <= tol, or - where the reference's own fp32 arithmetic is further than tol from the
    float64 evaluation - err within `factor` of that yardstick: the same order of rounding noise."""
    return err <= max(tol, factor * yardstick)


def float64_gradients(cfg, w0, tok, tgt):
    """Gradient of the mean negative log-likelihood (the scaling of nncp.c:1175) at the weights
    w0 with an empty memory: torch float64 autograd over the statement of
    tests/test_model_torch.py."""
    import torch
    from test_model_torch import _torch_step
    cfg = dict(cfg)
    cfg.setdefault("attn_len", [cfg["mem_len"] + cfg["seg_len"]] * cfg["n_layer"])
    B, D = cfg["batch_size"], cfg["d_model"]
    w = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in w0.items()}
    mem = [torch.zeros(B, cfg["mem_len"], D, dtype=torch.float64) for _ in range(cfg["n_layer"])]
    _, nll, _ = _torch_step(w, cfg, tok, tgt, mem)
    nll.backward()
    return {k: t.grad.numpy() for k, t in w.items()}


def close_or_no_worse(a, chk, exact, tol, factor=3.0):
    """a within tol (relative L2) of the checker, or - where the checker's own fp32 arithmetic is
    further than that from the float64 value - no further from float64 than factor x the checker."""
    return rel_l2(a, chk) <= tol or within_or_no_worse(rel_l2(a, exact), rel_l2(chk, exact), tol, factor)
