"""Test infrastructure: integer CDF build and symbol lookup of the CPU build at vocabulary sizes
around every kernel-variant boundary, exact-size guarded buffers, bit-exact against the CPU
checker and numpy searchsorted.  Usage: fuzz_cdf.py <seed> <cases>, library path in
NNCP_TEST_HIP_LIB."""
import ctypes as C, os, sys, time, faulthandler
import numpy as np
faulthandler.enable()
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), '..'))
from conftest import load_pkg, REF_LIB
B = load_pkg().binding
ref = B.NC(REF_LIB, use_device=False)
lib = C.CDLL(os.environ['NNCP_TEST_HIP_LIB'])
lib.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
i64, i32, vp = C.c_int64, C.c_int, C.c_void_p
lib.nchip_softmax_cdf16.argtypes = [vp, vp, vp, i32, i64]
lib.nchip_cdf_lookup.argtypes = [vp, vp, vp, vp, i32, i64, i64]
def dev(arr):
    arr = np.ascontiguousarray(arr)
    p = C.c_void_p(); assert lib.hipMalloc(C.byref(p), max(arr.nbytes, 2)) == 0
    C.memmove(p, arr.ctypes.data, arr.nbytes); return p
def back(p, shape, dt):
    lib.hipcpu_flush_copies()  # the stand-in runs queued launches at a wait
    out = np.empty(shape, dt); C.memmove(out.ctypes.data, p, out.nbytes); return out
rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 0)
n_cases = int(sys.argv[2]) if len(sys.argv) > 2 else 40
t0 = time.time()
for case in range(n_cases):
    V = int(rng.choice([1, 2, 3, 5, 64, 255, 256, 257, 1000, 1023, 1024, 1025, 4095, 4096, 4100, 16383, 16384, 16385, 30000, 65535]))
    n = int(rng.choice([1, 2, 3, 4, 5, 7, 9]))
    x = (rng.standard_normal((n, V)) * rng.choice([0.01, 3, 30])).astype(np.float32)
    if rng.integers(3) == 0: x[0] = 0
    dx, dc = dev(x), dev(np.zeros((n, V), np.uint16))
    assert lib.nchip_softmax_cdf16(None, dx, dc, V, n) == 0
    got = back(dc, (n, V), np.uint16)
    want = ref.numpy(ref.nc_soft_max_cdf16(ref.tensor(x)), free=True)
    assert np.array_equal(got, want), ("cdf", case, V, n)
    m = int(rng.choice([1, 3, 100, 1001, 4096])) if case % 10 else 262144 + int(rng.choice([0, 3]))
    if m > 100000 and V > 20000: n = min(n, 2)
    t = rng.integers(0, 65536, size=(n, m)).astype(np.uint16)
    dt_, ds = dev(t), dev(np.zeros((n, m), np.uint16))
    assert lib.nchip_cdf_lookup(None, dc, dt_, ds, V, m, n) == 0
    sym = back(ds, (n, m), np.uint16).astype(np.int64)
    for r in range(n):
        assert np.array_equal(sym[r], np.searchsorted(want[r].astype(np.int64), t[r].astype(np.int64), side="right") - 1), ("lookup", case, V, m)
    for p in (dx, dc, dt_, ds): lib.hipFree(p)
print("ok: %d cases in %.1fs" % (n_cases, time.time() - t0))
