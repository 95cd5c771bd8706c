"""Independent numpy (float64) restatements used to pin the CPU checker and,
through it, the GPU library.  Arrays are in numpy order, i.e. the reverse of
the libnc dims: libnc (D, N) is numpy (N, D); libnc axis 0 is numpy axis -1.
"""
import numpy as np


def softmax(x):
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def layer_norm(x, eps=1e-5, avg=True):
    mu = x.mean(axis=-1, keepdims=True) if avg else 0.0
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps)


def gelu(x):
    return 0.5 * x * (1.0 + np.tanh(0.7978845608 * (x + 0.044715 * x ** 3)))


def fd_grad(f, arrays, eps=1e-6):
    """Central finite differences of scalar f(*arrays) in float64."""
    arrays = [np.array(a, dtype=np.float64) for a in arrays]
    grads = []
    for a in arrays:
        g = np.zeros_like(a)
        it = np.nditer(a, flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            old = a[i]
            a[i] = old + eps
            fp = f(*arrays)
            a[i] = old - eps
            fm = f(*arrays)
            a[i] = old
            g[i] = (fp - fm) / (2 * eps)
        grads.append(g)
    return grads


def relpos_attention(q, kv, kvm, w_r, b_r, H, dk, attn_len, b_r_scale):
    """Direct restatement of the score formula (nncp.c:728-800).
    numpy shapes: q (T,B,H*dk), kv (T,B,H*dk+H*dv), kvm (M,B,.) or None,
    w_r (H,d_pos,dk) or None, b_r (H,K) or None.  Returns (T,B,H*dv)."""
    T, B, _ = q.shape
    M = 0 if kvm is None else kvm.shape[0]
    K = M + T
    dv = (kv.shape[2] - H * dk) // H
    allkv = kv if kvm is None else np.concatenate([kvm, kv], axis=0)  # (K,B,.)
    out = np.zeros((T, B, H * dv), dtype=np.float64)
    for b in range(B):
        for h in range(H):
            k = allkv[:, b, h * dk:(h + 1) * dk]                    # (K,dk)
            v = allkv[:, b, H * dk + h * dv:H * dk + (h + 1) * dv]   # (K,dv)
            for i in range(T):
                qi = q[i, b, h * dk:(h + 1) * dk]
                s = np.full(K, -np.inf)
                for j in range(K):
                    delta = i + M - j
                    if delta < 0 or delta >= attn_len:
                        continue
                    acc = k[j] @ qi
                    if w_r is not None:
                        d_pos = w_r.shape[1]
                        acc += w_r[h, max(d_pos - 1 - delta, 0)] @ qi
                    if b_r is not None:
                        acc += b_r_scale * b_r[h, K - 1 - delta]
                    s[j] = acc / np.sqrt(dk)
                a = np.exp(s - s.max())
                a /= a.sum()
                out[i, b, h * dv:(h + 1) * dv] = a @ v
    return out


def cdf16(logits):
    """Integer CDF spec of nc_soft_max_cdf16 with the exponential taken from
    the library under test (passed in already evaluated is not possible, so the
    caller supplies q = floor(exp_det(.) * 2^24) and this does the integer part).
    logits here IS that integer array q of shape (n, V)."""
    q = logits.astype(np.uint64)
    n, V = q.shape
    run = np.concatenate([np.zeros((n, 1), np.uint64), np.cumsum(q, axis=1)[:, :-1]], axis=1)
    tot = q.sum(axis=1, keepdims=True)
    return (run * np.uint64(65536 - V) // tot + np.arange(V, dtype=np.uint64)).astype(np.uint16)
