"""Test infrastructure: random attention shapes (single-kernel and batched-GEMM paths, with
and without memory / position table) through the raw entry points of the CPU build, exact-size
guarded buffers; forward against the numpy restatement, backward for addresses and against a
directional central difference, the single-query step bit-identical to its column.
Usage: fuzz_attn.py <seed> <cases>, library path in NNCP_TEST_HIP_LIB."""
import ctypes as C, os, sys, time, os, faulthandler
import numpy as np
faulthandler.enable()
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), '..'))
import nputil as U
lib = C.CDLL(os.environ['NNCP_TEST_HIP_LIB'])
lib.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
lib.nchip_relpos_attn_bwd_scratch.restype = C.c_size_t
i64, f32, i32, vp = C.c_int64, C.c_float, C.c_int, C.c_void_p
lib.nchip_relpos_attn_fwd.argtypes = [vp, vp, i64, vp, vp, i64, vp, vp, vp, i64, vp, vp] + [i32] * 8 + [f32, i32]
lib.nchip_relpos_attn_bwd.argtypes = [vp, vp, i64, vp, vp, i64, vp, vp, vp, i64, vp, vp, vp, vp, vp] + [i32] * 8 + [f32, i32, vp, i32]
lib.nchip_relpos_attn_fwd_step.argtypes = [vp, vp, i64, vp, vp, i64, vp, vp, vp, i64] + [i32] * 8 + [f32, i32]
def dev(arr):
    arr = np.ascontiguousarray(arr, dtype=np.float32)
    p = C.c_void_p(); assert lib.hipMalloc(C.byref(p), max(arr.nbytes, 4)) == 0
    C.memmove(p, arr.ctypes.data, arr.nbytes); return p
def back(p, shape):
    lib.hipcpu_flush_copies()  # the stand-in runs queued launches at a wait
    out = np.empty(shape, np.float32); C.memmove(out.ctypes.data, p, out.nbytes); return out
rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 0)
n_cases = int(sys.argv[2]) if len(sys.argv) > 2 else 30
t0 = time.time()
for case in range(n_cases):
    dk = int(rng.choice([32, 64, 16, 8, 48]))
    H, B = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    T = int(rng.choice([1, 7, 16, 20, 33, 64]))
    M = int(rng.choice([0, 5, 16, 20, 64, 100, 192]))
    if rng.integers(3) == 0: T = int(rng.choice([80, 96]))     # beyond the single-kernel limit
    K = T + M
    use_wr = int(rng.integers(4) != 0)
    d_pos = int(rng.integers(1, K + 1))
    attn_len = int(rng.integers(1, K + 2))
    dv = dk
    q = rng.standard_normal((T, B, H * dk)) * 0.5
    kv = rng.standard_normal((T, B, H * (dk + dv))) * 0.5
    kvm = rng.standard_normal((max(M, 1), B, H * (dk + dv))) * 0.5
    w_r = rng.standard_normal((H, d_pos, dk)) * 0.5
    b_r = rng.standard_normal((H, K)) * 0.5
    dout = rng.standard_normal((T, B, H * dv))
    scale = float(rng.choice([1.0, 2.5]))
    P = dict(q=dev(q), kv=dev(kv), kvm=dev(kvm[:M]) if M else None, w_r=dev(w_r) if use_wr else None, b_r=dev(b_r),
             out=dev(np.zeros((T, B, H * dv))), probs=dev(np.zeros((B, H, T, K))), rel=dev(np.zeros((B, H, T, d_pos))),
             dout=dev(dout), dq=dev(np.zeros_like(q)), dkv=dev(np.zeros_like(kv)), dkvm=dev(np.zeros((M, B, H * (dk + dv)))) if M else None,
             dw_r=dev(np.zeros_like(w_r)) if use_wr else None, db_r=dev(np.zeros_like(b_r)))
    nscr = lib.nchip_relpos_attn_bwd_scratch(H, dk, B, T, M, d_pos)
    P["scr"] = dev(np.zeros(nscr))
    rc = lib.nchip_relpos_attn_fwd(None, P["q"], H * dk, P["kv"], P["kvm"], H * (dk + dv), P["w_r"], P["b_r"], P["out"], H * dv,
                                   P["probs"], P["rel"], H, dk, dv, B, T, M, d_pos, attn_len, scale, 0)
    assert rc == 0
    out = back(P["out"], (T, B, H * dv))
    want = U.relpos_attention(q, kv, kvm[:M] if M else None, w_r if use_wr else None, b_r, H, dk, attn_len, scale)
    # rows whose window is empty are undefined in the restatement (0/0): only compare finite ones
    ok = np.isfinite(want)
    err = np.abs(out[ok] - want[ok]).max() / (np.abs(want[ok]).max() + 1e-9) if ok.any() else 0.0
    assert err < 3e-5, ("fwd", case, err, dk, H, B, T, M, d_pos, attn_len, use_wr)
    rc = lib.nchip_relpos_attn_bwd(None, P["q"], H * dk, P["kv"], P["kvm"], H * (dk + dv), P["w_r"], P["probs"], P["dout"], H * dv,
                                   P["dq"], P["dkv"], P["dkvm"], P["dw_r"], P["db_r"], H, dk, dv, B, T, M, d_pos, attn_len, scale, 0,
                                   P["scr"], 0)
    assert rc in (0, 1), rc
    dq = back(P["dq"], q.shape)
    # directional finite difference on q
    if ok.all():
        d = rng.standard_normal(q.shape); eps = 1e-3
        f = lambda qq: float((U.relpos_attention(qq, kv, kvm[:M] if M else None, w_r if use_wr else None, b_r, H, dk, attn_len, scale) * dout).sum())
        fd = (f(q + eps * d) - f(q - eps * d)) / (2 * eps)
        an = float((dq * d).sum())
        assert abs(fd - an) <= 2e-3 * (abs(fd) + abs(an) + 1e-3), ("bwd", case, fd, an, dk, H, B, T, M, d_pos, attn_len, use_wr)
    # single-query step where the shape allows it
    if dk in (32, 64) and T <= 64 and K <= 128 and (not use_wr or d_pos <= 128):
        t = int(rng.integers(T))
        o1 = dev(np.zeros((B, H * dv)))
        qt = dev(q[t])
        rc = lib.nchip_relpos_attn_fwd_step(None, qt, H * dk, P["kv"], P["kvm"], H * (dk + dv), P["w_r"], P["b_r"], o1, H * dv,
                                            H, dk, dv, B, T, M, d_pos, attn_len, scale, t)
        assert rc == 0
        assert np.array_equal(back(o1, (B, H * dv)), out[t]), ("step", case)
        lib.hipFree(o1); lib.hipFree(qt)
    for p in P.values():
        if p: lib.hipFree(p)
print("ok: %d cases in %.1fs" % (n_cases, time.time() - t0))
