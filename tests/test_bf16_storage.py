"""NC_TYPE_BF16 as a storage type (nncp's param_type under --bf16, nncp.c:343-346): 2-byte
tensors, conversions, ops on bf16 operands, parameters with an fp32 master in the optimiser.

The libnc that defines the reference's bf16 arithmetic is not part of the reference tree, so
what is pinned here is what the type's definition fixes: the rounding (torch's float32 ->
bfloat16 conversion, bit for bit), exact widening, the identity gradient of a conversion, and
- for parameters - an independent route to the same numbers: a model with f32 parameters that
start at bf16-representable values and products that round their operands computes the same
first gradient, so after one plain-SGD step its weights are the bf16 model's master values and
their rounding is the bf16 model's parameters.  The CPU checker is tested here; the GPU library
against the checker in test_gpu_zz_new_paths.py."""
import ctypes as C

import numpy as np
import pytest

import modelutil as M


def _corner_values():
    rng = np.random.default_rng(12)
    vals = (rng.standard_normal(4000) * 10.0 ** rng.integers(-30, 30, 4000)).astype(np.float32)
    bits = rng.integers(0, 1 << 31, 3000, dtype=np.int64).astype(np.uint32)
    ties = (bits & np.uint32(0xFFFF0000)) | np.uint32(0x8000)               # exactly halfway
    near = np.concatenate([ties - np.uint32(1), ties + np.uint32(1)])
    special = np.array([0x00000001, 0x00008000, 0x00018000, 0x007FFFFF, 0x80000000, 0x7F7F0000, 0x7F7F7FFF,
                        0x7F800000, 0xFF800000, 0x7FC00000, 0x7F800001], dtype=np.uint32)
    allbits = np.concatenate([vals.view(np.uint32), ties, near, special, ties | np.uint32(0x80000000)])
    return allbits.view(np.float32)


def check_conversions(nc, B):
    """nc_convert both ways on library `nc` against torch, bit for bit"""
    import torch
    a = _corner_values()
    x = nc.tensor(a)
    h = nc.nc_convert(x, B.BF16)
    assert nc.nc_tensor_get_item_type(h) == B.BF16
    host = nc.nc_tensor_to_cpu_device(nc.dup(h))
    got_bits = np.frombuffer((C.c_char * (2 * a.size)).from_address(nc.nc_tensor_get_ptr(host, None)),
                             dtype=np.uint16).copy()
    nc.free(host)
    want = torch.from_numpy(a.copy()).to(torch.bfloat16)
    want_bits = want.view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(a)
    assert np.array_equal(got_bits[~nan], want_bits[~nan])
    assert np.isnan(B.bf16_widen(got_bits[nan])).all()                      # NaN stays NaN
    back = nc.numpy(nc.nc_convert(h, B.F32), free=True)                     # exact widening
    assert np.array_equal(back[~nan].view(np.uint32), want.to(torch.float32).numpy()[~nan].view(np.uint32))


def test_conversions_round_to_nearest_even_and_widen_exactly(ref, pkg):
    check_conversions(ref, pkg.binding)


def test_ops_on_bf16_tensors_are_the_ops_on_their_widened_values(ref, pkg, rng):
    B = pkg.binding
    a = rng.standard_normal((4, 7)).astype(np.float32)
    b = rng.standard_normal((4, 7)).astype(np.float32)
    ar, br = B.bf16_widen(B.bf16_bits(a)), B.bf16_widen(B.bf16_bits(b))
    ta, tb = ref.nc_convert(ref.tensor(a), B.BF16), ref.nc_convert(ref.tensor(b), B.BF16)
    s = ref.nc_add(ref.dup(ta), ref.dup(tb))
    assert ref.nc_tensor_get_item_type(s) == B.F32
    assert np.array_equal(ref.numpy(s, free=True), ar + br)
    pr = ref.numpy(ref.nc_mul(ref.dup(ta), ref.tensor(b)), free=True)       # mixed operands
    assert np.array_equal(pr, ar * b)
    sm = ref.numpy(ref.nc_soft_max(ref.dup(ta)), free=True)
    want = ref.numpy(ref.nc_soft_max(ref.tensor(ar)), free=True)
    assert np.array_equal(sm, want)
    ref.free(ta, tb)


def test_gradient_passes_a_conversion_unchanged(ref, pkg, rng):
    """d/dw sum(c * widen(round(w))) is c itself: the rounding has the identity as gradient"""
    B = pkg.binding
    w = rng.standard_normal((3, 8)).astype(np.float32)
    c = rng.standard_normal((3, 8)).astype(np.float32)
    holder, p = ref.param(w, "w")
    wt = C.c_void_p(holder.value)
    y = ref.nc_sum(ref.nc_mul(ref.nc_convert(ref.nc_convert(ref.dup(wt), B.BF16), B.F32), ref.tensor(c)))
    g = ref.backward(y)
    ref.free(y)
    (gw,) = g.values()
    assert np.array_equal(gw, c)


def _model(host, cfg, **kw):
    H = M.load_pkg().host
    return H.Model(host, H.make_config(**dict(cfg, **kw)))


def _master(m, name):
    t = m.L.nncp_model_opt_state(m.ptr, name.encode(), 2)
    assert t, name
    a = m._to_numpy(t)
    m.nc.nc_free_tensor(t)
    return a


def check_master_and_parameters_against_the_f32_route(host, dev, fused=0):
    """module docstring: one plain-SGD step, bf16 parameters against f32 parameters that start
    at the same (bf16-representable) values with operand-rounding products"""
    B = M.load_pkg().binding
    cfg = dict(M.TINY, fused=fused, use_device=dev, nb_threads=4, sgd_opt=M.sgd(0.5))
    Bs, T, V = cfg["batch_size"], cfg["seg_len"], cfg["n_symbols"]
    (tok, tgt), = M.segment_batches(M.markov1(Bs * T, V, seed=3), Bs, T, 1)
    a = _model(host, cfg, param_bf16=1)
    w0 = a.params()
    for k, v in w0.items():                                                # stored values are bf16 values
        assert np.array_equal(B.bf16_widen(B.bf16_bits(v)), v), k
    for k in w0:                                                            # the master starts as the parameter
        assert np.array_equal(_master(a, k).ravel(), w0[k].ravel()), k
    pa, la = a.train_step(tok, tgt, 0.5)
    wa = a.params()
    ma = {k: _master(a, k).reshape(w0[k].shape) for k in w0}
    a.close()
    b = _model(host, cfg)
    b.nc.nc_set_matmul_bf16(b.ctx, 1)
    for k, v in w0.items():
        b.set_param(k, v)
    pb, lb = b.train_step(tok, tgt, 0.5)
    wb = b.params()
    b.nc.nc_set_matmul_bf16(b.ctx, 0)
    b.close()
    return (pa, la, wa, ma), (pb, lb, wb), w0


def test_bf16_parameters_follow_the_f32_route_on_the_checker():
    (pa, la, wa, ma), (pb, lb, wb), w0 = check_master_and_parameters_against_the_f32_route(M.ref_host(), 0)
    B = M.load_pkg().binding
    assert np.array_equal(pa, pb) and la == lb
    moved = 0
    for k in w0:
        assert np.array_equal(ma[k], wb[k]), k                              # master = the f32 model's weights
        assert np.array_equal(wa[k], B.bf16_widen(B.bf16_bits(ma[k]))), k   # parameter = rounding of the master
        moved += int((ma[k] != w0[k]).sum())
    assert moved > 1000                                                     # (the step did change them)


def test_bf16_parameter_files_hold_two_bytes_per_element(tmp_path):
    """save / load of a bf16 model: records carry type NC_TYPE_BF16 and 2 bytes per element, and
    a second model loads exactly the saved values"""
    cfg = dict(M.TINY, fused=0, use_device=0, nb_threads=2, sgd_opt=M.rmsprop(3e-4), param_bf16=1)
    a = _model(M.ref_host(), cfg)
    Bs, T, V = cfg["batch_size"], cfg["seg_len"], cfg["n_symbols"]
    for tok, tgt in M.segment_batches(M.markov1(Bs * T * 2, V, seed=4), Bs, T, 2):
        a.train_step(tok, tgt, 3e-4)
    wa = a.params()
    path = str(tmp_path / "w.bin")
    a.L.nncp_model_save_coefs(a.ptr, path.encode())
    a.close()
    n = sum(v.size for v in wa.values())
    import os
    size = os.path.getsize(path)
    assert 2 * n < size < 2 * n + 200 * len(wa)                             # 2 bytes per element + record headers
    b = _model(M.ref_host(), dict(cfg, seed=99))
    b.L.nncp_model_load_coefs(b.ptr, path.encode())
    wb = b.params()
    b.close()
    for k in wa:
        assert np.array_equal(wa[k], wb[k]), k
