"""nchip_norm_bwd_static - the norm backward for callers that cannot allocate: its partial
rows live in a device array the library itself holds - against nchip_norm_bwd with a buffer
of the caller, through the C ABI: bit-identical dx, dw, db on two calls in a row, the second
with a smaller input (the shared buffer keeps the first call's contents), and a size beyond
the buffer is turned away before anything is launched.  Collected last (file name)."""
import ctypes as C

import numpy as np
import pytest

from conftest import hip_lib_path, load_pkg

pytestmark = pytest.mark.gpu


def _both_ways(nc, lib, rng, d, n, avg, affine):
    g = rng.standard_normal((n, d)).astype(np.float32)
    xhat = rng.standard_normal((n, d)).astype(np.float32)
    rstd = (0.5 + rng.random(n)).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    add = rng.standard_normal((n, d)).astype(np.float32)
    rows = lib.nchip_norm_bwd_partial_rows(C.c_int64(n))
    host = dict(g=g, xhat=xhat, rstd=rstd, w=w, add=add)
    outs = dict(dx_a=(n, d), dx_b=(n, d), dw_a=(d,), dw_b=(d,), db_a=(d,), db_b=(d,), partial=(rows * 2 * d,))
    dev = {k: nc.tensor(v) for k, v in host.items()}
    # different fill values, so that an output left unwritten cannot compare equal
    dev.update({k: nc.tensor(np.full(s, 1.0 + i, np.float32)) for i, (k, s) in enumerate(outs.items())})
    # the kernels go on the tensor library's own stream, in order with its uploads and read-backs
    st = C.c_void_p(nc.nc_context_stream(nc.ctx))
    P = {k: C.c_void_p(nc.lib.nc_tensor_get_ptr(v, None)) for k, v in dev.items()}
    wp = P["w"] if affine else None
    dwa, dba, dwb, dbb = (P["dw_a"], P["db_a"], P["dw_b"], P["db_b"]) if affine else (None,) * 4
    rc = lib.nchip_norm_bwd(st, P["g"], P["xhat"], P["rstd"], wp, P["dx_a"], P["add"], dwa, dba, P["partial"],
                            C.c_int(d), C.c_int64(n), C.c_int(avg))
    assert rc == 0
    rc = lib.nchip_norm_bwd_static(st, P["g"], P["xhat"], P["rstd"], wp, P["dx_b"], P["add"], dwb, dbb,
                                   C.c_int(d), C.c_int64(n), C.c_int(avg))
    assert rc == 0
    res = {k: nc.numpy(dev[k]) for k in outs if k != "partial"}
    nc.free(*dev.values())
    assert np.array_equal(res["dx_a"].view(np.uint32), res["dx_b"].view(np.uint32))
    assert np.isfinite(res["dx_a"]).all() and np.abs(res["dx_a"]).max() > 0
    if affine:
        for k in ("dw", "db"):
            assert np.array_equal(res[k + "_a"].view(np.uint32), res[k + "_b"].view(np.uint32)), k
            assert np.ptp(res[k + "_a"]) > 0                        # written, not the fill value


@pytest.mark.parametrize("d,sizes", [(512, (2048, 333)), (1024, (4096, 64)), (96, (700, 33)), (256, (5, 3))])
def test_norm_backward_without_allocation_matches_the_caller_buffer_form(d, sizes):
    pkg = load_pkg()
    path = hip_lib_path(pkg)
    nc = pkg.binding.NC(path, use_device=True)
    lib = C.CDLL(path)
    lib.nchip_norm_bwd_static_capacity.restype = C.c_size_t
    assert lib.nchip_norm_bwd_static_capacity() == 2 << 20
    rng = np.random.default_rng(d)
    for i, n in enumerate(sizes):                        # second call smaller than the first
        _both_ways(nc, lib, rng, d, n, avg=1 - (i & 1), affine=True)
    _both_ways(nc, lib, rng, d, sizes[1], avg=1, affine=False)
    nc.close()


def test_norm_backward_without_allocation_rejects_what_does_not_fit():
    """Turned away on the host, before any pointer is touched or kernel launched."""
    pkg = load_pkg()
    lib = C.CDLL(hip_lib_path(pkg))
    one = C.c_void_p(16)                                 # never dereferenced
    rc = lib.nchip_norm_bwd_static(None, one, one, one, one, one, None, one, one,
                                   C.c_int(40000), C.c_int64(1024), C.c_int(1))
    assert rc == -3
