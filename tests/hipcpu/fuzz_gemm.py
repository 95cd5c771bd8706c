"""Test infrastructure: random GEMM shapes, layouts, tile configurations and epilogue options
through the raw entry points of the CPU build, every operand in an exact-size buffer that ends
at a guard page (an out-of-range access is a SIGSEGV), results against float64 numpy.
Usage: fuzz_gemm.py <seed> <cases>, library path in NNCP_TEST_HIP_LIB."""
import ctypes as C, os, sys, time, faulthandler
import numpy as np
faulthandler.enable()
lib = C.CDLL(os.environ['NNCP_TEST_HIP_LIB'])
lib.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
i64, f32, i32, vp = C.c_int64, C.c_float, C.c_int, C.c_void_p
lib.nchip_gemm2.argtypes = [vp, i32, i32, i32, i32, i32, f32, vp, i64, i64, i64, vp, i64, i64, i64, f32, vp, i64, i64, i64,
                            i32, i32, vp, i32, vp, i32, i32, vp]
lib.nchip_gemm_add.argtypes = [vp, i32, i32, i32, i32, i32, f32, vp, i64, i64, vp, i64, i64, vp, i64, i64, i32, vp, i32, vp, vp, i32, i32, vp]
lib.nchip_gemm_dact.argtypes = [vp, i32, i32, i32, i32, i32, f32, vp, i64, vp, i64, vp, i64, vp, i32, i32, i32, vp]

def dev(arr):
    """exact-size guarded device buffer holding arr (float32)"""
    arr = np.ascontiguousarray(arr, dtype=np.float32)
    p = C.c_void_p()
    assert lib.hipMalloc(C.byref(p), arr.nbytes) == 0
    C.memmove(p, arr.ctypes.data, arr.nbytes)
    return p
def back(p, n):
    lib.hipcpu_flush_copies()  # the stand-in runs queued launches at a wait
    out = np.empty(n, np.float32); C.memmove(out.ctypes.data, p, n * 4); return out
def bf16r(x):
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000
    return u.astype(np.uint32).view(np.float32)

rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 0)
n_cases = int(sys.argv[2]) if len(sys.argv) > 2 else 60
t0 = time.time()
for case in range(n_cases):
    ta, tb = int(rng.integers(2)), int(rng.integers(2))
    m, n, k = (int(rng.choice([1, 3, 8, 31, 64, 65, 100, 128, 129, 200, 257, 300, 513])) for _ in range(3))
    k = int(rng.choice([0, 1, 5, 16, 31, 32, 33, 64, 70, 96, 130, 257, 400]))
    lib.nchip_gemm_force_config(int(rng.choice([0, 0, 0, 4, 7, 8, 9, 5, 1, 2, 3, 6, 10, 11, 13])))
    batch = int(rng.choice([1, 1, 1, 2, 3]))
    prec = int(rng.choice([0, 0, 1]))
    mode = int(rng.choice([0, 1, 2]))
    inv = int(rng.integers(4) == 0)
    ksplit = int(rng.choice([1, 1, 1, 2, 3])) if (not inv and k >= 32) else 1
    pad_a, pad_b, pad_c = (int(rng.choice([0, 0, 1, 4])) for _ in range(3))
    ra, ca = (k, m) if ta else (m, k)       # stored rows (contiguous), cols
    rb, cb = (n, k) if tb else (k, n)
    lda, ldb, ldc = ra + pad_a, rb + pad_b, m + pad_c
    A = rng.standard_normal((batch, max(ca, 1), lda)).astype(np.float32)
    Bm = rng.standard_normal((batch, max(cb, 1), ldb)).astype(np.float32)
    Cin = rng.standard_normal((batch, n, ldc)).astype(np.float32)
    use_bias, act, use_pre, use_add = int(rng.integers(2)), int(rng.integers(3)), int(rng.integers(2)), int(rng.integers(2))
    beta = float(rng.choice([0.0, 0.0, 0.5])) if not use_add else 0.0
    alpha = float(rng.choice([1.0, 0.5]))
    bias = rng.standard_normal(m).astype(np.float32)
    add = rng.standard_normal((batch, n, ldc)).astype(np.float32)
    lib.nchip_gemm_bf16_source(mode)
    dA, dB, dC = dev(A), dev(Bm), dev(Cin)
    dbias = dev(bias) if use_bias else None
    dpre = dev(np.zeros_like(Cin)) if use_pre else None
    dadd = dev(add) if use_add else None
    ws = dev(np.zeros(batch * ksplit * m * n + 1)) if ksplit > 1 else None
    precision = prec | (0x100 if inv else 0)
    if use_add:
        rc = lib.nchip_gemm_add(None, ta, tb, m, n, k, alpha, dA, lda, A[0].size, dB, ldb, Bm[0].size, dC, ldc, n * ldc, batch,
                                dbias, act, dpre, dadd, precision, ksplit, ws)
    else:
        rc = lib.nchip_gemm2(None, ta, tb, m, n, k, alpha, dA, lda, A[0].size, 0, dB, ldb, Bm[0].size, 0, beta, dC, ldc, n * ldc, 0,
                             batch, 1, dbias, act, dpre, precision, ksplit, ws)
    assert rc == 0, rc
    got = back(dC, Cin.size).reshape(Cin.shape)
    # numpy reference
    Ae = A[:, :ca, :ra]; Be = Bm[:, :cb, :rb]
    opA = Ae if ta else np.swapaxes(Ae, 1, 2)          # (batch, m... ) careful: arrays are (cols, rows) in numpy
    # column-major: stored matrix X (rows r, cols c) is numpy[c, r].  op(A) is m x k.
    A_mk = np.swapaxes(Ae, 1, 2) if not ta else Ae     # -> numpy (batch, m?,..)
    # build explicit (batch, m, k) and (batch, k, n)
    if ta: Amk = Ae.copy()                              # stored (k rows, m cols) -> numpy [m, k]
    else: Amk = np.swapaxes(Ae, 1, 2).copy()            # stored (m rows, k cols) -> numpy [k, m] -> [m, k]
    if tb: Bkn = Be.copy()                              # stored (n rows, k cols) -> numpy [k, n]
    else: Bkn = np.swapaxes(Be, 1, 2).copy()            # stored (k rows, n cols) -> numpy [n, k] -> [k, n]
    if prec: Amk, Bkn = bf16r(Amk), bf16r(Bkn)
    if k == 0: prod = np.zeros((batch, m, n))
    else: prod = Amk.astype(np.float64) @ Bkn.astype(np.float64)
    v = alpha * prod
    if beta: v = v + beta * np.swapaxes(Cin[:, :, :m], 1, 2)
    if use_bias: v = v + bias[None, :, None]
    pre = v.copy()
    if act == 1: v = 0.5 * v * (1 + np.tanh(0.7978845608 * (v + 0.044715 * v ** 3)))
    elif act == 2: v = np.maximum(v, 0)
    if use_add: v = v + np.swapaxes(add[:, :, :m], 1, 2)
    want = np.swapaxes(v, 1, 2)
    err = np.abs(got[:, :, :m] - want).max() / (np.abs(want).max() + 1e-9)
    assert err < 2e-5, (case, err, ta, tb, m, n, k, batch, prec, mode, inv, ksplit)
    if pad_c: assert np.array_equal(got[:, :, m:], Cin[:, :, m:]), "padding rows of C written"
    if use_pre:
        gp = back(dpre, Cin.size).reshape(Cin.shape)[:, :, :m]
        assert np.abs(gp - np.swapaxes(pre, 1, 2)).max() / (np.abs(pre).max() + 1e-9) < 2e-5
    for p in (dA, dB, dC, dbias, dpre, dadd, ws):
        if p: lib.hipFree(p)
# the few-column kernels of the width-invariant class (16x16x4 MFMA, vector ALU, 32x32x2 MFMA)
# against the tile kernel, bit for bit, at exact-size operands
lib.nchip_gemm_force_config(0)
for case in range(max(4, n_cases // 8)):
    m = 32 * int(rng.integers(1, 9)); n = int(rng.integers(1, 65)); k = 32 * int(rng.choice([1, 2, 3, 8, 9, 16, 24, 40, 72]))
    lda, ldb, ldc = m + 4 * int(rng.integers(3)), k + 4 * int(rng.integers(3)), m + int(rng.choice([0, 1, 4]))
    A = rng.standard_normal((k, lda)).astype(np.float32); Bm = rng.standard_normal((n, ldb)).astype(np.float32)
    bias = rng.standard_normal(m).astype(np.float32); add = rng.standard_normal((n, ldc)).astype(np.float32)
    use_bias, act, use_pre, use_add = int(rng.integers(2)), int(rng.integers(3)), int(rng.integers(2)), int(rng.integers(2))
    dA, dB = dev(A), dev(Bm)
    dbias = dev(bias) if use_bias else None
    dadd = dev(add) if use_add else None
    outs = []
    for kernel in (0, 1, 2, 3):
        lib.nchip_gemm_few_columns_kernel(kernel)
        dC = dev(np.full((n, ldc), 9.0, np.float32)); dpre = dev(np.zeros((n, ldc), np.float32)) if use_pre else None
        if use_add:
            rc = lib.nchip_gemm_add(None, 0, 0, m, n, k, 1.0, dA, lda, 0, dB, ldb, 0, dC, ldc, 0, 1, dbias, act, dpre, dadd, 0x100, 1, None)
        else:
            rc = lib.nchip_gemm2(None, 0, 0, m, n, k, 1.0, dA, lda, 0, 0, dB, ldb, 0, 0, 0.0, dC, ldc, 0, 0, 1, 1, dbias, act, dpre, 0x100, 1, None)
        assert rc == 0, rc
        outs.append((back(dC, n * ldc), back(dpre, n * ldc) if use_pre else None))
        for q in (dC, dpre):
            if q: lib.hipFree(q)
    lib.nchip_gemm_few_columns_kernel(3)
    # the same product from a k-major copy of A (element (i, kk) at kk + i * ldat), exact size
    ldat = k + 4 * int(rng.integers(3))
    At = np.zeros((m, ldat), np.float32); At[:, :k] = A[:, :m].T
    dAt = dev(At)
    dC = dev(np.full((n, ldc), 9.0, np.float32)); dpre = dev(np.zeros((n, ldc), np.float32)) if use_pre else None
    if use_add:
        rc = lib.nchip_gemm_add(None, 1, 0, m, n, k, 1.0, dAt, ldat, 0, dB, ldb, 0, dC, ldc, 0, 1, dbias, act, dpre, dadd, 0x100, 1, None)
    else:
        rc = lib.nchip_gemm2(None, 1, 0, m, n, k, 1.0, dAt, ldat, 0, 0, dB, ldb, 0, 0, 0.0, dC, ldc, 0, 0, 1, 1, dbias, act, dpre, 0x100, 1, None)
    assert rc == 0, rc
    outs.append((back(dC, n * ldc), back(dpre, n * ldc) if use_pre else None))
    for q in (dC, dpre, dAt):
        if q: lib.hipFree(q)
    for o, pz in outs[1:]:
        assert np.array_equal(o.view(np.uint32), outs[0][0].view(np.uint32)), ("few-column kernels differ", m, n, k, act, use_bias, use_add)
        if use_pre: assert np.array_equal(pz.view(np.uint32), outs[0][1].view(np.uint32))
    v = Bm[:, :k].astype(np.float64) @ A[:, :m].astype(np.float64)
    if use_bias: v = v + bias[None, :]
    if act == 1: v = 0.5 * v * (1 + np.tanh(0.7978845608 * (v + 0.044715 * v ** 3)))
    elif act == 2: v = np.maximum(v, 0)
    if use_add: v = v + add[:, :m]
    got = outs[0][0].reshape(n, ldc)
    assert np.abs(got[:, :m] - v).max() / (np.abs(v).max() + 1e-9) < 2e-5
    if ldc > m: assert np.all(got[:, m:] == 9.0), "padding rows of C written"
    for q in (dA, dB, dbias, dadd):
        if q: lib.hipFree(q)
print("ok: %d cases in %.1fs" % (n_cases, time.time() - t0))
