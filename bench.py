#!/usr/bin/env python3
"""Benchmark of the hot path: NNCP's online train+code step on one MI355X.

Workload (BASELINE.json configs[2]): Transformer-XL, 12 layers, d_model 512,
8 heads x 64, d_ff 2048, seg_len 64, mem_len 64, batch 32 streams, 256 symbols,
RMSProp (beta 0.99, eps 1e-8, lr 3e-4); data: a prefix of the seeded order-3
Markov byte stream whose contexts draw next-byte distributions from
Dirichlet(0.05); weights N(0, 0.02), seeded.

One step = one batch of 32 x 64 = 2048 symbols through the whole path:
whole-segment forward (fused HIP ops) -> logits -> 16-bit integer CDF on the
GPU -> copy to pinned host memory -> host range coder (integer symbol coder)
-> backward -> RMSProp update + memory shift.  The emitted stream is decodable
(tests/test_gpu_model.py round-trips the same code path).

Prints ONE JSON line (see the field list at the bottom).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

C3 = dict(n_layer=12, d_model=512, n_head=8, d_inner=2048, d_pos=128, mem_len=64, seg_len=64,
          batch_size=32, n_symbols=256, seed=123)
PEAK_TFLOPS = {"fp32": 157.3, "bf16": 2500.0}


PROFILES = os.path.join(ROOT, "profiles")


TRAFFIC_SUMMARY = {"fp32": "c3_fp32_hbm_traffic_pmc.txt", "bf16": "c3_bf16_hbm_traffic_pmc.txt"}


def measured_traffic(kernel, variant):
    """(HBM-side bytes per launch (read + written) of a kernel instantiation, where the figure
    comes from) out of the committed rocprofv3 summary of the variant (FETCH_SIZE / WRITE_SIZE
    runs of this script, scaled by a device copy of known size; a counter run cannot be taken
    from inside the timed run, so the figure is the committed one and `traffic_source` says
    so).  The summary's rows are `<kernel name> <launches> <FETCH KiB> <WRITE KiB> <read MB>
    <write MB>`; names are compared without blanks.  The event records name a kernel by its
    leading template arguments only, so a row matches when its name starts with the record's;
    two rows that both do are two instantiations the record cannot tell apart, and then no
    figure is given.  (None, None) when the summary does not hold the kernel."""
    summary = TRAFFIC_SUMMARY[variant]
    path = os.path.join(PROFILES, summary)
    if not os.path.exists(path):
        return None, None
    # (the grouped launch runs the same template as single launches: its record carries a
    # ",grouped" mark that kernel names do not have)
    want = kernel.replace(" ", "").replace(",grouped>", ">").rstrip(">")
    found = []
    for line in open(path):
        parts = line.rsplit(None, 5)
        if len(parts) != 6:
            continue
        name = parts[0].replace(" ", "")
        try:
            read_mb, write_mb = float(parts[4]), float(parts[5])
        except ValueError:
            continue
        if name.startswith(want) and name[len(want):len(want) + 1] in ("", ",", ">"):
            found.append((read_mb + write_mb) * 1e6)
    if len(found) != 1:
        return None, None
    return found[0], "profiles/%s (committed counter summary of this command; not re-measured in this run)" % summary


def markov3_dirichlet(n, seed=2024, alpha=0.05, n_symbols=256):
    """Order-3 Markov source: every visited 3-symbol context draws its next-
    symbol pmf from Dirichlet(alpha), lazily, seeded by (context, seed)."""
    out = np.zeros(n, dtype=np.uint16)
    cache = {}
    rng = np.random.default_rng(seed)
    u = rng.random(n)
    ctx = (0, 0, 0)
    for i in range(n):
        cdf = cache.get(ctx)
        if cdf is None:
            h = (ctx[0] * 65536 + ctx[1] * 256 + ctx[2]) ^ (seed * 2654435761 & 0xffffffff)
            p = np.random.default_rng(h).dirichlet(np.full(n_symbols, alpha))
            cdf = np.cumsum(p)
            cache[ctx] = cdf
        s = min(int(np.searchsorted(cdf, u[i] * cdf[-1])), n_symbols - 1)
        out[i] = s
        ctx = (ctx[1], ctx[2], s)
    return out


C4 = dict(n_layer=20, d_model=1024, n_head=16, d_inner=4096, d_pos=256, mem_len=192, seg_len=64,
          batch_size=64, n_symbols=16384, seed=123)


def bigram_zipf_dirichlet(n, n_symbols=16384, seed=2025, alpha=0.1, keep=256):
    """Token ids from a seeded bigram model (BASELINE configs[3]): the marginal is
    Zipf(1.0) under a seeded permutation of the ranks, the row of a previous
    token is drawn from Dirichlet(alpha * V * marginal) the first time that token
    is visited (seeded by (token, seed)); such rows are sparse, and only their
    `keep` largest entries are kept, renormalised."""
    rng = np.random.default_rng(seed)
    marg = 1.0 / (rng.permutation(n_symbols) + 1.0)
    marg /= marg.sum()
    shape = alpha * n_symbols * marg
    u = rng.random(n)
    out = np.zeros(n, dtype=np.uint16)
    rows = {}
    prev = 0
    for i in range(n):
        row = rows.get(prev)
        if row is None:
            g = np.random.default_rng((prev << 20) ^ seed).gamma(shape)
            idx = np.argpartition(g, -keep)[-keep:]
            cdf = np.cumsum(g[idx])
            row = rows[prev] = (idx, cdf)
        idx, cdf = row
        prev = int(idx[min(int(np.searchsorted(cdf, u[i] * cdf[-1])), len(idx) - 1)])
        out[i] = prev
    return out


def hip_runtime():
    """The HIP runtime instance that libnc_hip.so itself is linked to (already mapped into this
    process), and not whichever file the loader would pick for the bare name: with a second
    copy of the runtime in the process (a wheel that bundles one), events and waits issued
    through the wrong instance would not order with the library's kernels."""
    for line in open("/proc/self/maps"):
        path = line.split()[-1]
        if "libamdhip64" in os.path.basename(path):
            return C.CDLL(path)
    return C.CDLL("libamdhip64.so")


def say(what):
    """Progress on stderr, flushed before the step it names starts (stdout carries the one
    JSON line only)."""
    print("[bench] " + what, file=sys.stderr, flush=True)


def init_weights(model, seed=99, sigma=0.02):
    """N(0, sigma) for every matrix, 1 for LayerNorm gains, 0 for biases."""
    rng = np.random.default_rng(seed)
    for name in model.param_names():
        w = model.get_param(name)
        if name.startswith("ln_g"):
            new = np.ones_like(w)
        elif w.ndim >= 2 and not name.startswith("b_r"):
            new = rng.normal(0.0, sigma, size=w.shape).astype(np.float32)
        else:
            new = np.zeros_like(w)
        model.set_param(name, new)


def run_block(model, H, syms, mode):
    """Codes syms (a multiple of B*T) as one block; returns (seconds, bytes, stats)."""
    cap = syms.size * 4 + 4096
    out = np.zeros(cap, dtype=np.uint8)
    st = H.NNCPStats()
    sched = H.constant_lr(3e-4)
    model.nc.nc_synchronize(model.dev)
    t0 = time.perf_counter()
    n = model.L.nncp_compress(model.ptr, syms.ctypes.data, syms.size, out.ctypes.data, cap, mode,
                              C.byref(sched), C.byref(st))
    model.nc.nc_synchronize(model.dev)
    return time.perf_counter() - t0, n, st


def gemm_profile(model, H, syms, mode, hip_lib):
    """Times every GEMM launch of a few extra steps with HIP events on the
    launch stream; returns the per-instantiation rows."""
    lib = C.CDLL(hip_lib)
    lib.nchip_gemm_profile_enable(1)
    run_block(model, H, syms, mode)
    lib.nchip_gemm_profile_enable(0)
    names = ((C.c_char * 48) * 32)()
    launches = (C.c_int64 * 32)()
    flops = (C.c_double * 32)()
    secs = (C.c_double * 32)()
    lib.nchip_gemm_profile_read.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    n = lib.nchip_gemm_profile_read(32, names, launches, flops, secs)
    rows = []
    for i in range(n):
        rows.append(dict(kernel=names[i].value.decode(), launches=int(launches[i]),
                         flops=float(flops[i]), seconds=float(secs[i])))
    return rows


def attention_c2(pkg, iters=50):
    """Isolated rel-pos attention forward+backward at BASELINE configs[1]
    (B 32, H 8, d_head 64, 64 queries x 128 keys, sinusoidal position table,
    learned bias), through the raw kernel entry points on the null stream,
    timed with a HIP event pair around `iters` forward+backward pairs.
    Algorithmic bytes: fwd Q + K + V + P_table + O, bwd Q,K,V,O,dO in and
    dQ,dK,dV out = 72 MiB; dense flops 11 GEMM-likes x 268 M = 2.95 G."""
    nc = pkg.binding.NC(pkg.binding.HIP_LIB)
    lib = C.CDLL(pkg.binding.HIP_LIB)
    hip = hip_runtime()
    B, Hh, dk, T, M = 32, 8, 64, 64, 64
    K, d_pos = M + T, M + T
    rng = np.random.default_rng(0)
    q = rng.normal(0, 0.125, (T, B, Hh * dk)).astype(np.float32)
    kv = rng.normal(0, 0.125, (T, B, 2 * Hh * dk)).astype(np.float32)
    kvm = rng.normal(0, 0.125, (M, B, 2 * Hh * dk)).astype(np.float32)
    delta = (d_pos - 1 - np.arange(d_pos))[:, None]
    inv = 1.0 / 10000 ** (np.arange(0, dk, 2) / dk)
    tab = np.zeros((d_pos, dk), np.float32)
    tab[:, 0::2] = np.sin(delta * inv)
    tab[:, 1::2] = np.cos(delta * inv)
    w_r = np.broadcast_to(tab, (Hh, d_pos, dk)).copy()
    b_r = rng.normal(0, 0.02, (Hh, K)).astype(np.float32)
    dout = rng.normal(0, 1, (T, B, Hh * dk)).astype(np.float32)
    host = dict(q=q, kv=kv, kvm=kvm, w_r=w_r, b_r=b_r, dout=dout)
    dev = {k: nc.tensor(v) for k, v in host.items()}
    lib.nchip_relpos_attn_bwd_scratch.restype = C.c_size_t
    nscr = lib.nchip_relpos_attn_bwd_scratch(Hh, dk, B, T, M, d_pos)
    outs = dict(out=q.shape, probs=(B, Hh, T, K), rel=(B, Hh, T, d_pos), dq=q.shape, dkv=kv.shape,
                dkvm=kvm.shape, dw_r=w_r.shape, db_r=b_r.shape, scratch=(nscr,))
    for k, shp in outs.items():
        dev[k] = nc.tensor(np.zeros(shp, np.float32))
    P = {k: C.c_void_p(nc.lib.nc_tensor_get_ptr(v, None)) for k, v in dev.items()}
    i64, f32, i32 = C.c_int64, C.c_float, C.c_int
    ld, ldkv = i64(Hh * dk), i64(2 * Hh * dk)

    def fwd():
        return lib.nchip_relpos_attn_fwd(None, P["q"], ld, P["kv"], P["kvm"], ldkv, P["w_r"], P["b_r"],
                                         P["out"], ld, P["probs"], P["rel"], i32(Hh), i32(dk), i32(dk),
                                         i32(B), i32(T), i32(M), i32(d_pos), i32(K), f32(1.0), i32(0))

    def bwd():
        return lib.nchip_relpos_attn_bwd(None, P["q"], ld, P["kv"], P["kvm"], ldkv, P["w_r"], P["probs"],
                                         P["dout"], ld, P["dq"], P["dkv"], P["dkvm"], P["dw_r"], P["db_r"],
                                         i32(Hh), i32(dk), i32(dk), i32(B), i32(T), i32(M), i32(d_pos),
                                         i32(K), f32(1.0), i32(0), P["scratch"], i32(0))

    def timed(fns):
        e0, e1 = C.c_void_p(), C.c_void_p()
        hip.hipEventCreate(C.byref(e0))
        hip.hipEventCreate(C.byref(e1))
        for f in fns:
            assert f() == 0
        hip.hipDeviceSynchronize()
        hip.hipEventRecord(e0, None)
        for _ in range(iters):
            for f in fns:
                f()
        hip.hipEventRecord(e1, None)
        hip.hipEventSynchronize(e1)
        ms = C.c_float()
        hip.hipEventElapsedTime(C.byref(ms), e0, e1)
        hip.hipEventDestroy(e0)
        hip.hipEventDestroy(e1)
        return ms.value * 1e3 / iters

    us_f, us_b, us = timed([fwd]), timed([bwd]), timed([fwd, bwd])

    # the same head shape on the bf16 matrix cores (the bf16-operand variant's attention):
    # operands are the bf16 copies of the tensors above, made once outside the timed region
    # (in the step they come out of the producing products' epilogues)
    def u16(shape):
        return nc.tensor(np.zeros(shape, np.uint16))
    for k in ("q", "kv", "kvm", "w_r", "dout"):
        dev[k + "16"] = u16(host[k].shape)
        assert lib.nchip_cast_bf16(None, P[k], C.c_void_p(nc.lib.nc_tensor_get_ptr(dev[k + "16"], None)),
                                   i64(host[k].size)) == 0
    for k in ("out", "dq", "dkv", "dkvm"):
        dev[k + "16"] = u16(outs[k])
    dev["probs16"] = u16(outs["probs"])
    P = {k: C.c_void_p(nc.lib.nc_tensor_get_ptr(v, None)) for k, v in dev.items()}

    def fwd16():
        return lib.nchip_relpos_attn_fwd_bf16(None, P["q16"], ld, P["kv16"], P["kvm16"], ldkv, P["w_r16"], P["b_r"],
                                              P["out"], P["out16"], ld, P["probs16"], i32(Hh), i32(dk), i32(dk),
                                              i32(B), i32(T), i32(M), i32(d_pos), i32(K), f32(1.0))

    def bwd16():
        return lib.nchip_relpos_attn_bwd_bf16(None, P["q16"], ld, P["kv16"], P["kvm16"], ldkv, P["w_r16"],
                                              P["probs16"], P["dout16"], ld, P["dq"], P["dq16"], P["dkv"], P["dkv16"],
                                              P["dkvm"], P["dkvm16"], P["dw_r"], P["db_r"], i32(Hh), i32(dk), i32(dk),
                                              i32(B), i32(T), i32(M), i32(d_pos), i32(K), f32(1.0), P["scratch"])

    us16_f, us16_b, us16 = timed([fwd16]), timed([bwd16]), timed([fwd16, bwd16])
    for v in dev.values():
        nc.free(v)
    nc.close()
    # algorithmic bytes.  fp32: fwd Q + K + V + position table + O, bwd Q, K, V, O, dO in and
    # dQ, dK, dV out = 72 MiB.  bf16: the same tensors at 2 bytes where they are read, fp32 +
    # bf16 where they are written (results keep their fp32 form for the rest of the step)
    nbytes, flops = 72 * 2 ** 20, 2.95e9
    n_q, n_kv, n_w = q.size, kv.size + kvm.size, w_r.size
    nbytes16 = (2 * (n_q + n_kv + n_w) + 6 * n_q) + (2 * (2 * n_q + n_kv + n_w) + 6 * (n_q + n_kv))
    return {"workload": "BASELINE configs[1]: B32 H8 d64 T64 K128 fwd+bwd fp32",
            "us_fwd": round(us_f, 2), "us_bwd": round(us_b, 2), "us_fwd_bwd": round(us, 2),
            "algorithmic_GBps": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / 8000, 4),
            "dense_TFLOPs": round(flops / us / 1e6, 2), "mfma_fp32_frac": round(flops / us / 1e6 / 157.3, 4),
            "binding_bound": "mfma (39 flop/B > fp32 ridge 20)",
            "bf16": {"workload": "the same head shape, operands as bf16 copies, v_mfma_f32_16x16x32_bf16",
                     "us_fwd": round(us16_f, 2), "us_bwd": round(us16_b, 2), "us_fwd_bwd": round(us16, 2),
                     "algorithmic_bytes": nbytes16,
                     "algorithmic_GBps": round(nbytes16 / us16 / 1e3, 1), "hbm_frac": round(nbytes16 / us16 / 1e3 / 8000, 4),
                     "dense_TFLOPs": round(flops / us16 / 1e6, 2), "mfma_bf16_frac": round(flops / us16 / 1e6 / 2500, 4)}}


def cdf_c5(pkg, iters=50):
    """Coder-side probability path at BASELINE configs[4]: fp32 logits for 64
    streams x 16384 symbols (N(0, 3) plus a Zipf-shaped per-token bias
    -log(rank) under a seeded rank permutation) -> 16-bit integer CDF, then
    10^6 uniform 16-bit targets per stream -> symbol index by
    cumulative-frequency search.  Raw kernel entry points on the null stream,
    HIP event pair around `iters` launches.  Algorithmic bytes: CDF build
    4 MiB read + 2 MiB written; lookup 2 B target + 2 B symbol each."""
    nc = pkg.binding.NC(pkg.binding.HIP_LIB)
    lib = C.CDLL(pkg.binding.HIP_LIB)
    hip = hip_runtime()
    V, n, m = 16384, 64, 1000000
    rng = np.random.default_rng(5)
    bias = -np.log(rng.permutation(V) + 1.0)
    logits = (rng.normal(0, 3, (n, V)) + bias).astype(np.float32)
    targets = rng.integers(0, 65536, size=(n, m)).astype(np.uint16)
    d_log, d_t = nc.tensor(logits), nc.tensor(targets)
    d_cdf = nc.tensor(np.zeros((n, V), np.uint16))
    d_sym = nc.tensor(np.zeros((n, m), np.uint16))
    P = [C.c_void_p(nc.lib.nc_tensor_get_ptr(t, None)) for t in (d_log, d_cdf, d_t, d_sym)]
    i64, i32 = C.c_int64, C.c_int

    def build():
        return lib.nchip_softmax_cdf16(None, P[0], P[1], i32(V), i64(n))

    def lookup():
        return lib.nchip_cdf_lookup(None, P[1], P[2], P[3], i32(V), i64(m), i64(n))

    def timed(f, k):
        e0, e1 = C.c_void_p(), C.c_void_p()
        hip.hipEventCreate(C.byref(e0))
        hip.hipEventCreate(C.byref(e1))
        assert f() == 0
        hip.hipDeviceSynchronize()
        hip.hipEventRecord(e0, None)
        for _ in range(k):
            f()
        hip.hipEventRecord(e1, None)
        hip.hipEventSynchronize(e1)
        ms = C.c_float()
        hip.hipEventElapsedTime(C.byref(ms), e0, e1)
        hip.hipEventDestroy(e0)
        hip.hipEventDestroy(e1)
        return ms.value * 1e3 / k

    us_b, us_l = timed(build, iters), timed(lookup, max(1, iters // 5))
    # the CDF is a function of integers only past the exponential: check it
    cdf = nc.numpy(d_cdf).astype(np.int64)
    freq = np.diff(np.concatenate([cdf, np.full((n, 1), 65536)], axis=1), axis=1)
    sym = nc.numpy(d_sym).astype(np.int64)
    rows = np.arange(n)[:, None]
    t64 = targets.astype(np.int64)
    hi = np.where(sym + 1 < V, np.take_along_axis(cdf, np.minimum(sym + 1, V - 1), axis=1), 65536)
    ok = bool((cdf[:, 0] == 0).all() and (freq >= 1).all() and (freq.sum(axis=1) == 65536).all()
              and (cdf[rows, sym] <= t64).all() and (t64 < hi).all())
    for t in (d_log, d_t, d_cdf, d_sym):
        nc.free(t)
    nc.close()
    b_bytes, l_bytes = n * V * 6, n * m * 4
    return {"workload": "BASELINE configs[4]: 64 streams x V16384 logits -> cdf16; 1e6 lookups per stream",
            "us_cdf_build": round(us_b, 2), "cdf_build_GBps": round(b_bytes / us_b / 1e3, 1),
            "us_lookup": round(us_l, 2), "lookups_per_s": round(n * m / us_l * 1e6, 0),
            "lookup_GBps": round(l_bytes / us_l / 1e3, 1), "lookup_hbm_frac": round(l_bytes / us_l / 1e3 / 8000, 4),
            "invariants_ok": ok}


def copy_floor(iters=50):
    """What a kernel that only moves bytes costs at the sizes of this workload's bandwidth kernels:
    device-to-device copies (the runtime's own copy kernel) of 4, 8 and 64 MiB, back to back on
    the null stream between two HIP events.  A norm kernel of the headline step reads 4 MiB and
    writes 8 MiB; its time is to be read against the copy that moves as much, not against
    8 TB/s, which a transfer of this size cannot reach (launch, ramp and drain are microseconds)."""
    hip = hip_runtime()
    out = {}
    for mib in (4, 8, 64):
        n = mib << 20
        src, dst = C.c_void_p(), C.c_void_p()
        assert hip.hipMalloc(C.byref(src), C.c_size_t(n)) == 0 and hip.hipMalloc(C.byref(dst), C.c_size_t(n)) == 0
        hip.hipMemset(src, 1, C.c_size_t(n))
        e0, e1 = C.c_void_p(), C.c_void_p()
        hip.hipEventCreate(C.byref(e0))
        hip.hipEventCreate(C.byref(e1))
        for _ in range(3):
            hip.hipMemcpyAsync(dst, src, C.c_size_t(n), 3, None)
        hip.hipDeviceSynchronize()
        hip.hipEventRecord(e0, None)
        for _ in range(iters):
            hip.hipMemcpyAsync(dst, src, C.c_size_t(n), 3, None)       # hipMemcpyDeviceToDevice
        hip.hipEventRecord(e1, None)
        hip.hipEventSynchronize(e1)
        ms = C.c_float()
        hip.hipEventElapsedTime(C.byref(ms), e0, e1)
        us = ms.value * 1e3 / iters
        out["%d_MiB" % mib] = {"us": round(us, 2), "moved_MB": round(2 * n / 1e6, 1), "GBps": round(2 * n / us / 1e3, 1)}
        hip.hipEventDestroy(e0)
        hip.hipEventDestroy(e1)
        hip.hipFree(src)
        hip.hipFree(dst)
    return out


def norms_isolated(pkg, iters=50):
    """The norm kernels of the headline step (d 512, 2048 columns: LayerNorm forward reads x and
    writes y and the normalised values, 12.6 MB; backward reads g and xhat and writes dx, 12.6 MB
    plus the partial rows of the gain / bias gradients), through the raw entry points, back to
    back on the null stream on resident buffers - measured the way copy_floor measures the copies
    they are to be read against (in the step their inputs come cold from the producing kernel)."""
    nc = pkg.binding.NC(pkg.binding.HIP_LIB)
    lib = C.CDLL(pkg.binding.HIP_LIB)
    hip = hip_runtime()
    d, n = 512, 2048
    rng = np.random.default_rng(1)
    t = {k: nc.tensor(rng.standard_normal(shape).astype(np.float32)) for k, shape in
         (("x", (n, d)), ("w", (d,)), ("b", (d,)), ("g", (n, d)))}
    rows = lib.nchip_norm_bwd_partial_rows(C.c_int64(n))
    for k, shape in (("y", (n, d)), ("xhat", (n, d)), ("rstd", (n,)), ("dx", (n, d)), ("dw", (d,)), ("db", (d,)),
                     ("partial", (rows * 2 * d,))):
        t[k] = nc.tensor(np.zeros(shape, np.float32))
    P = {k: C.c_void_p(nc.lib.nc_tensor_get_ptr(v, None)) for k, v in t.items()}

    def fwd():
        return lib.nchip_norm_fwd(None, P["x"], P["w"], P["b"], P["y"], P["xhat"], P["rstd"], C.c_int(d), C.c_int64(n),
                                  C.c_float(1e-5), C.c_int(1))

    def bwd():
        # (dw = db = NULL: the partial rows are left to the caller, as in the step, where one launch
        # sums the rows of all norms of the backward pass)
        return lib.nchip_norm_bwd(None, P["g"], P["xhat"], P["rstd"], P["w"], P["dx"], None, None, None, P["partial"],
                                  C.c_int(d), C.c_int64(n), C.c_int(1))

    def timed(f):
        e0, e1 = C.c_void_p(), C.c_void_p()
        hip.hipEventCreate(C.byref(e0))
        hip.hipEventCreate(C.byref(e1))
        for _ in range(3):
            assert f() == 0
        hip.hipDeviceSynchronize()
        hip.hipEventRecord(e0, None)
        for _ in range(iters):
            f()
        hip.hipEventRecord(e1, None)
        hip.hipEventSynchronize(e1)
        ms = C.c_float()
        hip.hipEventElapsedTime(C.byref(ms), e0, e1)
        hip.hipEventDestroy(e0)
        hip.hipEventDestroy(e1)
        return ms.value * 1e3 / iters

    us_f, us_b = timed(fwd), timed(bwd)
    nbytes = 3 * d * n * 4
    for v in t.values():
        nc.free(v)
    nc.close()
    return {"workload": "LayerNorm d512 x 2048 columns, isolated, back to back", "us_fwd": round(us_f, 2),
            "us_bwd": round(us_b, 2), "algorithmic_MB": round(nbytes / 1e6, 1),
            "fwd_GBps": round(nbytes / us_f / 1e3, 1), "bwd_GBps": round(nbytes / us_b / 1e3, 1),
            "fwd_hbm_frac": round(nbytes / us_f / 1e3 / 8000, 4), "bwd_hbm_frac": round(nbytes / us_b / 1e3 / 8000, 4)}


def cpu_baseline(pkg, data, n_steps, threads):
    """The CPU checker driving the reference op sequence (whole-segment
    evaluation, float symbol coder: what `nncp --encode_only` does) on the
    host cores, on the first n_steps batches of the same workload."""
    H = pkg.host
    host = H.Host(os.path.join(ROOT, "oracle", "libnncp_host_ref.so"),
                  os.path.join(ROOT, "oracle", "libnc_ref.so"))
    opt = pkg.binding.SGDOptParams(algo=pkg.binding.SGD_OPT_RMSPROP, beta2=0.99, eps=1e-8, lr=3e-4)
    m = H.Model(host, H.make_config(**dict(C3, use_device=0, fused=0, nb_threads=threads, sgd_opt=opt)))
    init_weights(m)
    n = n_steps * C3["batch_size"] * C3["seg_len"]
    sec, _, _ = run_block(m, H, data[:n], H.MODE_SEGMENT | H.CODER_FLOAT)
    m.close()
    return n / sec


def decode_c3(pkg, data, n_segments, variant):
    """Decoding rate of the same workload: n_segments trained segments encoded by the
    whole-segment encoder, then decoded by the per-timestep decoder with K/V caches
    (NNCP_MODE_STEP_DECODE; it evaluates one token column per timestep and replays the
    training step once per segment) - timed, and checked to return the input."""
    H = pkg.host
    opt = pkg.binding.SGDOptParams(algo=pkg.binding.SGD_OPT_RMSPROP, beta2=0.99, eps=1e-8, lr=3e-4)
    per_step = C3["batch_size"] * C3["seg_len"]
    syms = np.ascontiguousarray(data[:n_segments * per_step])
    mode = H.MODE_SEGMENT | H.MODE_STEP_DECODE | H.CODER_CDF16

    def model():
        m = H.Model(H.Host(), H.make_config(**dict(C3, use_device=1, fused=1, sgd_opt=opt,
                                                   param_bf16=int(variant == "bf16_params"))))
        init_weights(m)
        m.nc.nc_set_matmul_bf16(m.ctx, 0 if variant == "fp32" else 1)
        return m
    enc = model()
    stream = np.zeros(syms.size * 4 + 4096, dtype=np.uint8)
    st = H.NNCPStats()
    sched = H.constant_lr(3e-4)
    enc.nc.nc_synchronize(enc.dev)
    t0 = time.perf_counter()
    n = enc.L.nncp_compress(enc.ptr, syms.ctypes.data, syms.size, stream.ctypes.data, stream.size, mode,
                            C.byref(sched), C.byref(st))
    enc.nc.nc_synchronize(enc.dev)
    t_enc = time.perf_counter() - t0
    enc.close()
    dec = model()
    out = np.zeros(syms.size, dtype=np.uint16)
    dec.nc.nc_synchronize(dec.dev)
    t0 = time.perf_counter()
    dec.L.nncp_decompress(dec.ptr, stream.ctypes.data, n, out.ctypes.data, syms.size, mode, C.byref(sched), C.byref(st))
    dec.nc.nc_synchronize(dec.dev)
    sec = time.perf_counter() - t0
    dec.close()
    return {"value": round(syms.size / sec, 1), "unit": "symbols/s", "ms_per_segment": round(sec / n_segments * 1e3, 2),
            "segments": n_segments, "decoder": "per-timestep with K/V caches + one training step per segment",
            "encode_ms_per_segment_same_mode": round(t_enc / n_segments * 1e3, 2),
            "round_trip_ok": bool(np.array_equal(out, syms))}


def measure_c4(pkg, variant, warmup, steps, profile_steps):
    """BASELINE configs[3] (not the headline metric): 20 layers, d_model 1024, 16 heads x 64,
    d_ff 4096, 64 + 192 keys, batch 64, V 16384; one step = 4096 tokens.  Same library calls
    as the default workload.  Returns the fields of its line / of the `c4` object."""
    H = pkg.host
    B, T = C4["batch_size"], C4["seg_len"]
    per_step = B * T
    data = bigram_zipf_dirichlet((warmup + steps + profile_steps) * per_step)
    opt = pkg.binding.SGDOptParams(algo=pkg.binding.SGD_OPT_RMSPROP, beta2=0.99, eps=1e-8, lr=3e-4)
    model = H.Model(H.Host(), H.make_config(**dict(C4, use_device=1, fused=1, sgd_opt=opt,
                                                   param_bf16=int(variant == "bf16_params"))))
    init_weights(model)
    model.nc.nc_set_matmul_bf16(model.ctx, 0 if variant == "fp32" else 1)
    mode = H.MODE_SEGMENT | H.CODER_CDF16
    pos = 0
    if warmup:
        say("C4 %s: %d warm-up steps" % (variant, warmup))
        run_block(model, H, data[pos:pos + warmup * per_step], mode)
        pos += warmup * per_step
    say("C4 %s: %d timed steps" % (variant, steps))
    l0 = model.nc.nc_get_launch_count(model.ctx)
    sec, nbytes, st = run_block(model, H, data[pos:pos + steps * per_step], mode)
    launches = model.nc.nc_get_launch_count(model.ctx) - l0
    pos += steps * per_step
    roof = None
    if profile_steps:
        say("C4 %s: %d steps with per-launch GEMM events" % (variant, profile_steps))
        rows = gemm_profile(model, H, data[pos:pos + profile_steps * per_step], mode, pkg.binding.HIP_LIB)
        if rows:
            dom = max(rows, key=lambda r: r["seconds"])
            peak = PEAK_TFLOPS["fp32" if variant == "fp32" else "bf16"]
            achieved = dom["flops"] / dom["seconds"] / 1e12
            tot_f, tot_s = sum(r["flops"] for r in rows), sum(r["seconds"] for r in rows)
            roof = {"bound": "mfma", "kernel": dom["kernel"], "achieved": round(achieved, 3), "peak": peak,
                    "unit": "TFLOP/s", "frac": round(achieved / peak, 4), "traffic": None,
                    "launches_per_step": dom["launches"] / profile_steps,
                    "avg_launch_us": round(dom["seconds"] / dom["launches"] * 1e6, 2),
                    "all_gemm_tflops": round(tot_f / tot_s / 1e12, 3),
                    "all_gemm_ms_per_step": round(tot_s / profile_steps * 1e3, 3)}
    model.close()
    return {"metric": "tokens/sec compressed (train+code) 20L d1024 V16384",
            "value": round(steps * per_step / sec, 1), "unit": "tokens/s", "steps": steps, "warmup": warmup,
            "ms_per_step": round(sec / steps * 1e3, 3),
            "dtype": "f32" if variant == "fp32" else "bf16-in/f32-acc",
            "config": {"workload": "BASELINE configs[3]: 20L d1024 16x64 ff4096 T64 M192 B64 V16384, RMSProp, seeded "
                                   "bigram Zipf(1.0) x Dirichlet(0.1) tokens, weights N(0,0.02)",
                       "tokens_per_step": per_step, "coder": "gpu cdf16 + host range coder", "variant": variant},
            "bits_per_token": round(nbytes * 8 / (steps * per_step), 4),
            "kernel_launches_per_step": launches / steps, "roofline": roof}


def main_c4(args):
    """`--workload c4`: the configs[3] measurement as a line of its own."""
    import __graft_entry__ as G
    r = measure_c4(G._load_pkg(), args.variant, args.warmup, args.steps, args.profile_steps)
    r.update({"n_gpus": 1, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
              "data": "synthetic", "cpu_baseline": None})
    print(json.dumps(r))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--workload", choices=["c3", "c4"], default="c3",
                    help="c3: the headline workload (BASELINE configs[2]); c4: the large-context token model "
                         "(configs[3]); its CPU baseline is not taken (one step is about an hour of host time)")
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--variant", choices=["fp32", "bf16", "bf16_params"], default="fp32",
                    help="fp32: the reference's arithmetic; bf16: matrix products on bf16 operands, f32 parameters; "
                         "bf16_params: parameters stored as NC_TYPE_BF16 as well (nncp --bf16's param_type)")
    ap.add_argument("--also", default="bf16,bf16_params", help="further variants measured after the headline one and "
                                                   "reported under `variants` (comma separated, empty for none)")
    ap.add_argument("--cpu-steps", type=int, default=4, help="0 skips the CPU baseline")
    ap.add_argument("--cpu-single-steps", type=int, default=1, help="steps of the single-thread CPU baseline (0 skips it)")
    ap.add_argument("--decode-segments", type=int, default=4, help="segments decoded for the `decode` object (0 skips it)")
    ap.add_argument("--profile-steps", type=int, default=2)
    ap.add_argument("--c4-steps", type=int, default=3,
                    help="timed steps of BASELINE configs[3] in its bf16-operand variant for the `c4` object of "
                         "the default line (after 1 warm-up step, plus 1 step under GEMM events; 0 skips it)")
    ap.add_argument("--decodable-steps", type=int, default=10,
                    help="timed steps of the width-invariant encoder (the stream format the per-timestep "
                         "decoder reads) for `encode_step_decodable` (0 skips it)")
    ap.add_argument("--attention-iters", type=int, default=50, help="0 skips the isolated attention timing")
    ap.add_argument("--cdf-iters", type=int, default=50, help="0 skips the coder-side CDF timing")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="first issue one device-to-device copy of this many MiB (a kernel of known "
                         "traffic, to scale FETCH_SIZE / WRITE_SIZE readings of a counter run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (one compression job per GPU, no "
                 "collectives); run it with --gpus 1")
    if args.workload == "c4":
        return main_c4(args)

    import __graft_entry__ as G
    pkg = G._load_pkg()
    H = pkg.host
    if not os.path.exists(H.HOST_HIP_LIB) or not os.path.exists(pkg.binding.HIP_LIB):
        G.build()
    B, T = C3["batch_size"], C3["seg_len"]
    per_step = B * T
    total_steps = args.warmup + args.steps + args.profile_steps
    data = markov3_dirichlet(max(total_steps, args.warmup + args.decodable_steps, args.cpu_steps,
                                 args.decode_segments) * per_step)
    opt = pkg.binding.SGDOptParams(algo=pkg.binding.SGD_OPT_RMSPROP, beta2=0.99, eps=1e-8, lr=3e-4)
    mode = H.MODE_SEGMENT | H.CODER_CDF16

    if args.calibrate_copy_mib:
        hip = hip_runtime()
        nbytes_cal = args.calibrate_copy_mib << 20
        src, dst = C.c_void_p(), C.c_void_p()
        assert hip.hipMalloc(C.byref(src), C.c_size_t(nbytes_cal)) == 0
        assert hip.hipMalloc(C.byref(dst), C.c_size_t(nbytes_cal)) == 0
        hip.hipMemset(src, 1, C.c_size_t(nbytes_cal))
        hip.hipDeviceSynchronize()
        assert hip.hipMemcpy(dst, src, C.c_size_t(nbytes_cal), 3) == 0  # hipMemcpyDeviceToDevice
        hip.hipDeviceSynchronize()
        hip.hipFree(src)
        hip.hipFree(dst)

    def measure(variant, mode=mode, steps=args.steps, profile_steps=args.profile_steps):
        """warm-up, the timed steps and the per-launch GEMM timing of one arithmetic variant"""
        model = H.Model(H.Host(), H.make_config(**dict(C3, use_device=1, fused=1, sgd_opt=opt,
                                                       param_bf16=int(variant == "bf16_params"))))
        init_weights(model)
        model.nc.nc_set_matmul_bf16(model.ctx, 0 if variant == "fp32" else 1)
        pos = 0
        if args.warmup:
            say("C3 %s: %d warm-up steps" % (variant, args.warmup))
            run_block(model, H, data[pos:pos + args.warmup * per_step], mode)
            pos += args.warmup * per_step
        say("C3 %s: %d timed steps" % (variant, steps))
        l0 = model.nc.nc_get_launch_count(model.ctx)
        sec, nbytes, st = run_block(model, H, data[pos:pos + steps * per_step], mode)
        launches = model.nc.nc_get_launch_count(model.ctx) - l0
        pos += steps * per_step
        roof = None
        if profile_steps:
            say("C3 %s: %d steps with per-launch GEMM events" % (variant, profile_steps))
            rows = gemm_profile(model, H, data[pos:pos + profile_steps * per_step], mode,
                                pkg.binding.HIP_LIB)
            if rows:
                dom = max(rows, key=lambda r: r["seconds"])
                achieved = dom["flops"] / dom["seconds"] / 1e12
                peak = PEAK_TFLOPS["fp32" if variant == "fp32" else "bf16"]
                tot_f = sum(r["flops"] for r in rows)
                tot_s = sum(r["seconds"] for r in rows)
                traffic, traffic_source = measured_traffic(dom["kernel"], "fp32" if variant == "fp32" else "bf16")
                roof = {"bound": "mfma", "kernel": dom["kernel"], "achieved": round(achieved, 3),
                        "peak": peak, "unit": "TFLOP/s", "frac": round(achieved / peak, 4),
                        "traffic": traffic, "traffic_source": traffic_source,
                        "launches_per_step": dom["launches"] / profile_steps,
                        "avg_launch_us": round(dom["seconds"] / dom["launches"] * 1e6, 2),
                        "flops_per_launch": dom["flops"] / dom["launches"],
                        "all_gemm_tflops": round(tot_f / tot_s / 1e12, 3),
                        "all_gemm_ms_per_step": round(tot_s / profile_steps * 1e3, 3)}
        model.close()
        return {"value": round(steps * per_step / sec, 1), "ms_per_step": round(sec / steps * 1e3, 3),
                "dtype": {"fp32": "f32", "bf16": "bf16-in/f32-acc",
                          "bf16_params": "bf16 parameters (f32 master in the optimiser), bf16-in/f32-acc"}[variant],
                "bits_per_symbol": round(nbytes * 8 / (steps * per_step), 4),
                "kernel_launches_per_step": launches / steps,
                "host_seconds": {"eval_and_copy": round(st.t_eval, 4), "code": round(st.t_code, 4),
                                 "grad": round(st.t_grad, 4), "update": round(st.t_update, 4)},
                "roofline": roof}

    head = measure(args.variant)
    variants = {args.variant: {k: head[k] for k in ("value", "ms_per_step", "dtype", "bits_per_symbol")}}
    for v in args.also.split(","):
        if v and v != args.variant:
            r = measure(v)
            variants[v] = {k: r[k] for k in ("value", "ms_per_step", "dtype", "bits_per_symbol")}
            variants[v]["all_gemm_tflops"] = r["roofline"]["all_gemm_tflops"] if r["roofline"] else None
            variants[v]["kernel_launches_per_step"] = r["kernel_launches_per_step"]
            variants[v]["roofline"] = r["roofline"]

    step_dec = None
    if args.decodable_steps:
        # the same workload coded in the stream format of the per-timestep decoder: forward
        # products in their width-invariant form (what `decode` below reads back)
        r = measure(args.variant, mode | H.MODE_STEP_DECODE, args.decodable_steps, 0)
        step_dec = {"value": r["value"], "unit": "symbols/s", "ms_per_step": r["ms_per_step"],
                    "steps": args.decodable_steps, "warmup": args.warmup, "variant": args.variant,
                    "kernel_launches_per_step": r["kernel_launches_per_step"],
                    "mode": "NNCP_MODE_SEGMENT | NNCP_MODE_STEP_DECODE | NNCP_CODER_CDF16"}

    attn = cdf = dec = None
    floor = copy_floor() if args.cdf_iters else None
    norms = norms_isolated(pkg) if args.cdf_iters else None
    if args.attention_iters:
        say("isolated attention, B32 H8 d64 T64 K128, %d forward+backward pairs" % args.attention_iters)
        attn = attention_c2(pkg, args.attention_iters)
    if args.cdf_iters:
        say("coder-side CDF path, 64 x 16384 logits, %d iterations" % args.cdf_iters)
        cdf = cdf_c5(pkg, args.cdf_iters)
    if args.decode_segments:
        say("decoding %d segments with the per-timestep decoder" % args.decode_segments)
        dec = decode_c3(pkg, data, args.decode_segments, args.variant)
    c4 = None
    if args.c4_steps:
        c4 = measure_c4(pkg, "bf16", 1, args.c4_steps, 1)

    cpu = None
    if args.cpu_steps:
        # the box's CPU share for one GPU is 16 threads, whatever the machine shows
        threads = min(os.cpu_count() or 1, 16)
        say("CPU checker, %d steps on %d threads" % (args.cpu_steps, threads))
        v = cpu_baseline(pkg, data, args.cpu_steps, threads)
        cpu = {"value": round(v, 1), "unit": "symbols/s", "cores": threads, "kind": "port",
               "sample": "first %d steps (%d symbols) of the same workload, CPU checker driving the "
                         "reference op sequence, whole-segment evaluation, float symbol coder"
                         % (args.cpu_steps, args.cpu_steps * per_step)}
        if args.cpu_single_steps:
            say("CPU checker, %d step(s) on 1 thread" % args.cpu_single_steps)
            v1 = cpu_baseline(pkg, data, args.cpu_single_steps, 1)
            cpu["single_thread"] = {"value": round(v1, 1), "cores": 1,
                                    "sample": "first %d step(s)" % args.cpu_single_steps}

    print(json.dumps({
        "metric": "symbols/sec compressed (train+code) 12L d512",
        "value": head["value"], "unit": "symbols/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: 12L d512 8x64 ff2048 T64 M64 B32 V256, RMSProp, "
                               "order-3 Markov Dirichlet(0.05) prefix, weights N(0,0.02)",
                   "symbols_per_step": per_step, "coder": "gpu cdf16 + host range coder",
                   "variant": args.variant,
                   "encoder": "whole-segment encoder (NNCP_MODE_SEGMENT | NNCP_CODER_CDF16): its stream is read "
                              "back by a decoder that replays the segment evaluation per timestep; the stream "
                              "format of the per-timestep decoder is timed under encode_step_decodable"},
        "bits_per_symbol": head["bits_per_symbol"],
        "kernel_launches_per_step": head["kernel_launches_per_step"],
        "host_seconds": head["host_seconds"],
        "roofline": head["roofline"], "encode_step_decodable": step_dec, "variants": variants,
        "c4": c4, "attention": attn, "cdf": cdf, "norms": norms, "copy_floor": floor, "decode": dec,
        "cpu_baseline": cpu}))


if __name__ == "__main__":
    main()
