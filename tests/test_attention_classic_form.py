"""The classic Transformer-XL attention, S = ((q + u_h).k_j + (q + v_h).R[d]) / sqrt(dk) with a
sinusoidal table R shared by the heads and learned vectors u, v, is the relative-position form
of nc_relpos_attention (nncp.c:763-800) under a change of variables done on the host:
    q' = q + u,   w_r[:, d_pos-1-d, h] = R[d],   b_r[K-1-d, h] = (v_h - u_h).R[d],  b_r_scale = 1
and its gradients follow by the chain rule (du = sum dq' - dv,  dv_h = sum_d db_r[K-1-d, h] R[d]).
Checked on the CPU checker against a torch float64 statement of the classic form with autograd;
the GPU kernels go through the same comparison at the size of the isolated-attention
configuration (32 streams, 8 heads of 64, 64 queries against 64 + 64 keys)."""
import math

import numpy as np
import pytest
import torch

import cases


def _table(K, DK):
    d = np.arange(K, dtype=np.float64)[:, None]
    inv = 1.0 / 10000 ** (np.arange(0, DK, 2) / DK)
    r = np.zeros((K, DK))
    r[:, 0::2], r[:, 1::2] = np.sin(d * inv), np.cos(d * inv)
    return r  # R[d], d = distance from the key to the query


def _classic_against_torch(nc, H, DK, B, T, MEM, sigma, sigma_uv, tol):
    K = T + MEM
    rng = np.random.default_rng(21)
    q = rng.normal(0, sigma, (T, B, H, DK))
    kv = rng.normal(0, sigma, (T, B, 2 * H * DK))
    kvm = rng.normal(0, sigma, (MEM, B, 2 * H * DK))
    u, v = rng.normal(0, sigma_uv, (H, DK)), rng.normal(0, sigma_uv, (H, DK))
    weight = rng.normal(0, 1, (T, B, H * DK))
    R = _table(K, DK)

    # --- classic form in torch ---------------------------------------------------
    tq, tkv, tkvm, tu, tv = (torch.tensor(a, requires_grad=True) for a in (q, kv, kvm, u, v))
    tR = torch.tensor(R)
    allkv = torch.cat([tkvm, tkv], dim=0)                          # (K, B, 2*H*dk), memory first
    k = allkv[..., :H * DK].reshape(K, B, H, DK)
    val = allkv[..., H * DK:].reshape(K, B, H, DK)
    i, j = torch.arange(T).view(T, 1), torch.arange(K).view(1, K)
    delta = i + MEM - j
    content = torch.einsum("tbhd,jbhd->bhtj", tq + tu, k)
    position = torch.einsum("tbhd,pd->bhtp", tq + tv, tR)          # p = distance
    position = torch.gather(position, 3, delta.clamp(min=0).expand(B, H, T, K))
    s = ((content + position) / math.sqrt(DK)).masked_fill(delta < 0, float("-inf"))
    out_t = torch.einsum("bhtj,jbhd->tbhd", torch.softmax(s, dim=3), val).reshape(T, B, H * DK)
    (out_t * torch.tensor(weight)).sum().backward()

    # --- the same through nc_relpos_attention ------------------------------------
    w_r = np.broadcast_to(R[::-1], (H, K, DK)).copy()              # table index p <-> distance K-1-p
    b_r = np.einsum("hd,pd->hp", v - u, R)[:, ::-1].copy()         # column K-1-d holds distance d
    arrays = [a.astype(np.float32) for a in ((q + u).reshape(T, B, H * DK), kv, kvm, w_r, b_r)]
    case = cases.Case("classic", None,
                      lambda nc_, q_, kv_, kvm_, w_, b_: nc_.nc_relpos_attention(q_, kv_, kvm_, w_, b_, H, DK, K, 1.0),
                      None)
    out, (dq, dkv, dkvm, dw_r, db_r) = case.run(nc, arrays, weight)

    def close(a, b):
        return np.abs(a - b).max() <= tol * max(np.abs(b).max(), 1e-30)
    assert close(out, out_t.detach().numpy())
    assert close(dq.reshape(T, B, H, DK), tq.grad.numpy())
    assert close(dkv, tkv.grad.numpy())
    assert close(dkvm, tkvm.grad.numpy())
    dv = np.einsum("hp,pd->hd", db_r[:, ::-1].astype(np.float64), R)
    du = dq.reshape(T, B, H, DK).astype(np.float64).sum(axis=(0, 1)) - dv
    assert close(dv, tv.grad.numpy())
    assert close(du, tu.grad.numpy())


def test_classic_txl_attention_through_the_relpos_entry_point(ref):
    _classic_against_torch(ref, H=2, DK=8, B=2, T=6, MEM=6, sigma=0.5, sigma_uv=0.3, tol=2e-5)


@pytest.mark.gpu
def test_classic_txl_attention_on_gpu_at_the_isolated_attention_size(hip):
    """Q, K, V ~ N(0, 1/64), u, v ~ N(0, 0.02), upstream gradient ~ N(0, 1): the single-kernel
    forward and backward against torch float64 autograd of the classic form, 1e-5."""
    _classic_against_torch(hip, H=8, DK=64, B=32, T=64, MEM=64, sigma=0.125, sigma_uv=0.02, tol=1e-5)
