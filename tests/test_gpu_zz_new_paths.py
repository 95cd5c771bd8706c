"""GPU tests of the paths either side of the step: the retrain pass (nncp_retrain_block,
dropout), the LSTM model class and the file container - the same host C code as on the CPU
checker, linked against libnc_hip.so - the bitwise bf16 operand rounding, nc_soft_max_int, the
1e-5 bar after 100 steps and the round trip of the headline configuration at its full size.
tests/test_kernels_on_cpu.py re-runs them on the CPU build of the kernels (the two long ones
only in a small form).  Collected after the other GPU tests (file name)."""
import os

import numpy as np
import pytest

import modelutil as M

pytestmark = [pytest.mark.gpu]


@pytest.fixture(scope="module")
def hosts():
    return M.hip_host(), M.ref_host()


@pytest.mark.parametrize("fused", [0, 1])
def test_retrain_round_trip_on_gpu_and_size_against_checker(hosts, fused):
    pkg = M.load_pkg()
    cfg = dict(M.TINY, fused=fused, sgd_opt=M.rmsprop(), dropout_prob=0.1, dropout_att_prob=0.05,
               retrain_period=1)
    B, T = cfg["batch_size"], cfg["seg_len"]
    block = B * T * 2 + 5
    cfg["retrain_len"] = 2 * block
    syms = M.markov1(3 * block - 7, 40, seed=21)

    def model(host, dev):
        return pkg.host.Model(host, pkg.host.make_config(**dict(cfg, use_device=dev, nb_threads=4)))
    enc = model(hosts[0], 1)
    data, st, rst = enc.compress_blocks(syms, block, 1)
    w_enc = enc.params()
    enc.close()
    dec = model(hosts[0], 1)
    out, _, _ = dec.decompress_blocks(data, len(syms), block, 1)
    w_dec = dec.params()
    dec.close()
    assert np.array_equal(out, syms)
    for k in w_enc:
        assert np.array_equal(w_enc[k], w_dec[k]), k
    # the dropout masks come from the same host-side stream in both libraries, so the
    # checker follows the same trajectory up to fp32 reordering: size within 0.5 %
    ref = model(hosts[1], 0)
    data_ref, _, rst_ref = ref.compress_blocks(syms, block, 1)
    w_ref = ref.params()
    ref.close()
    assert rst.n_steps == rst_ref.n_steps > 0
    assert abs(len(data) - len(data_ref)) <= max(2, 0.005 * len(data_ref))
    for k in w_ref:
        assert M.tensors_close(w_enc[k], w_ref[k], 1e-5), (k, M.rel_l2(w_enc[k], w_ref[k]))


LSTM = dict(n_layer=3, lstm_n_cells=24, batch_size=4, seg_len=6, n_symbols=40, seed=5)


@pytest.mark.parametrize("variant", [dict(), dict(lstm_type=0, lstm_n_cells2=32, lstm_full_connect=0)])
def test_lstm_training_steps_match_checker_and_stream_round_trips(hosts, variant):
    pkg = M.load_pkg()
    # plain SGD: RMSProp turns the fp32 noise of near-zero bias gradients into visible steps
    cfg = dict(LSTM, sgd_opt=M.sgd(0.05), **variant)
    B, T, V = cfg["batch_size"], cfg["seg_len"], cfg["n_symbols"]
    hip = pkg.host.Model(hosts[0], pkg.host.make_lstm_config(**dict(cfg, use_device=1)))
    ref = pkg.host.Model(hosts[1], pkg.host.make_lstm_config(**dict(cfg, use_device=0, nb_threads=4)))
    syms = M.markov1(B * T * 4, V, seed=77)
    for step, (tok, tgt) in enumerate(M.segment_batches(syms, B, T, 4), 1):
        ph, lh = hip.train_step(tok, tgt, 0.05)
        pr, lr_ = ref.train_step(tok, tgt, 0.05)
        assert M.relerr(ph, pr) <= 1e-5, step
        assert abs(lh - lr_) <= 1e-5 * abs(lr_), step
    w_h, w_r = hip.params(), ref.params()
    for k in w_r:
        assert M.tensors_close(w_h[k], w_r[k], 1e-5), (k, M.rel_l2(w_h[k], w_r[k]))
    hip.close()
    ref.close()
    n = B * T * 3 + 5
    data_syms = M.markov1(n, V, seed=3)
    for mode in (0, 1 | 2):
        enc = pkg.host.Model(hosts[0], pkg.host.make_lstm_config(**dict(cfg, use_device=1)))
        data, _ = enc.compress(data_syms, mode)
        enc.close()
        dec = pkg.host.Model(hosts[0], pkg.host.make_lstm_config(**dict(cfg, use_device=1)))
        out, _ = dec.decompress(data, n, mode)
        dec.close()
        assert np.array_equal(out, data_syms), mode


@pytest.mark.parametrize("stream", ["reference", "fast", "fast_bf16"])
def test_file_container_round_trip_on_gpu(hosts, tmp_path, stream):
    """nncp_encode_file / nncp_decode_file with the product library: the decoded file
    equals the input, and the compressed size is within 0.5 % (bf16: 2 %) of the
    checker's for the same file and parameters."""
    hp = M.load_pkg().host
    n = 200
    mode = 0 if stream == "reference" else hp.MODE_SEGMENT | hp.CODER_CDF16
    kw = dict(M.TINY, fused=int(stream != "reference"), sgd_opt=M.rmsprop(), nb_threads=4)
    syms = M.markov1(n, 40, seed=17)
    src = str(tmp_path / "in.bin")
    syms.astype(np.uint8).tofile(src)
    sizes = []
    for host, dev in ((hosts[0], 1), (hosts[1], 0)):
        cfg = hp.make_config(**dict(kw, use_device=dev))
        fp = hp.file_params(host, "3e-4,8,1e-4", "96,200,120", use_bf16=int(stream == "fast_bf16"), mode=mode)
        packed, back = str(tmp_path / ("out%d.nncp" % dev)), str(tmp_path / ("back%d.bin" % dev))
        st, _ = hp.encode_file(host, src, packed, cfg, fp)
        hp.decode_file(host, packed, back, use_device=dev, nb_threads=4)
        assert open(back, "rb").read() == open(src, "rb").read()
        assert st.n_symbols == n
        sizes.append(os.path.getsize(packed))
    assert abs(sizes[0] - sizes[1]) <= max(3, (0.02 if stream == "fast_bf16" else 0.005) * sizes[1])


@pytest.mark.parametrize("source", [0, 2])
def test_bf16_operand_rounding_is_bitwise_the_checkers(source):
    """A * I with the bf16 switch on returns the rounded operand itself: the kernels' rounding
    (inside the tile loader, source 0, and in the streaming cast pass, source 2) must be the
    checker's round-to-nearest-even bit for bit - ties, values next to ties, subnormals."""
    import ctypes as C
    from conftest import REF_LIB, hip_lib_path
    pkg = M.load_pkg()
    rng = np.random.default_rng(12)
    vals = (rng.standard_normal(2000) * 10.0 ** rng.integers(-30, 30, 2000)).astype(np.float32)
    ties = (rng.integers(0, 1 << 31, 1000, dtype=np.int64).astype(np.uint32) & np.uint32(0xFFFF0000)) | np.uint32(0x8000)
    bits = np.concatenate([vals.view(np.uint32), ties, ties - np.uint32(1), ties + np.uint32(1),
                           np.array([1, 0x8000, 0x18000, 0x7FFFFF], dtype=np.uint32)])
    a = bits.view(np.float32)
    a = a[np.isfinite(a) & (np.abs(a) < 1e38)]
    a = a[: a.size // 64 * 64].reshape(-1, 64)
    eye = np.eye(64, dtype=np.float32)
    outs = []
    lib = C.CDLL(hip_lib_path(pkg))
    for path, dev in ((hip_lib_path(pkg), True), (REF_LIB, False)):
        nc = pkg.binding.NC(path, use_device=dev)
        nc.nc_set_matmul_bf16(nc.ctx, 1)
        if dev:
            lib.nchip_gemm_bf16_source(source)
        outs.append(nc.numpy(nc.nc_matmul(nc.tensor(eye), nc.tensor(a)), free=True))
        nc.nc_set_matmul_bf16(nc.ctx, 0)
        nc.close()
    lib.nchip_gemm_bf16_source(1)
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))


def _fast_stream_properties(host, cfg, syms, variant):
    """Two encodings give the same bytes; the replaying decoder and the cached per-timestep
    decoder both return the input."""
    hp = M.load_pkg().host
    n = len(syms)

    def model():
        m = hp.Model(host, hp.make_config(**cfg))
        m.nc.nc_set_matmul_bf16(m.ctx, int(variant == "bf16"))
        return m
    for mode in (hp.MODE_SEGMENT | hp.CODER_CDF16, hp.MODE_SEGMENT | hp.MODE_STEP_DECODE | hp.CODER_CDF16):
        streams = []
        for _ in range(2):
            enc = model()
            data, st = enc.compress(syms, mode)
            enc.close()
            streams.append(data)
        assert np.array_equal(streams[0], streams[1]), mode
        assert st.n_symbols == n and 0 < len(streams[0]) < 2 * n, mode
        dec = model()
        back, _ = dec.decompress(streams[0], n, mode)
        dec.close()
        assert np.array_equal(back, syms), mode


@pytest.mark.parametrize("variant", ["fp32", "bf16"])
def test_fast_stream_properties_small(hosts, variant):
    # heads of 32: the cached per-timestep decoder needs the single-kernel attention shapes
    cfg = dict(n_layer=2, d_model=64, n_head=2, d_inner=96, d_pos=13, mem_len=7, seg_len=9, batch_size=3,
               n_symbols=40, seed=7, fused=1, sgd_opt=M.rmsprop(3e-4), use_device=1)
    _fast_stream_properties(hosts[0], cfg, M.markov1(3 * 9 * 2 + 3 * 2 + 1, 40, seed=5), variant)


@pytest.mark.parametrize("variant", ["fp32", "bf16"])
def test_full_size_c3_stream_round_trip_on_gpu(hosts, variant):
    """The headline configuration at its real size (12 layers, d_model 512, 8 x 64, d_ff 2048,
    64 + 64 keys, 32 streams, bytes): three trained segments and a ragged tail through the fast
    stream, checked through properties that do not depend on the size."""
    cfg = dict(n_layer=12, d_model=512, n_head=8, d_inner=2048, d_pos=128, mem_len=64, seg_len=64,
               batch_size=32, n_symbols=256, seed=123, fused=1, sgd_opt=M.rmsprop(3e-4), use_device=1)
    _fast_stream_properties(hosts[0], cfg, M.markov1(32 * 64 * 3 + 32 * 5 + 7, 256, seed=2024), variant)


@pytest.mark.parametrize("V,n", [(256, 64), (16384, 5), (3, 7), (1000, 33), (1, 4), (65535, 2)])
def test_soft_max_int_bit_exact(V, n):
    """nc_soft_max_int of the product against the checker, integer for integer."""
    from conftest import REF_LIB, hip_lib_path
    pkg = M.load_pkg()
    rng = np.random.default_rng(V)
    x = (rng.normal(0, 3, (n, V)) - np.log(rng.permutation(V) + 1.0)).astype(np.float32)
    x[0, : min(V, 4)] = [-1e30, 80.0, -80.0, 0.0][: min(V, 4)]       # clamped tail, dominant symbol
    for mult in (65536.0, 1000.5, 2.0 ** 31, 0.0):
        outs = []
        for path, dev in ((hip_lib_path(pkg), True), (REF_LIB, False)):
            nc = pkg.binding.NC(path, use_device=dev)
            outs.append(nc.numpy(nc.nc_soft_max_int(nc.tensor(x), mult), free=True))
            nc.close()
        assert outs[0].dtype == np.int32 and np.array_equal(outs[0], outs[1]), mult


def test_parameter_files_cross_between_the_gpu_and_the_checker(hosts, tmp_path):
    """nc_save_coefs / nc_load_coefs (libnc.h:530, 536): parameters trained on the GPU, saved by
    the product library and loaded by the checker's own reader are the same bits, and so the
    other way round (the two libraries implement the file layout separately); the loaded GPU
    model then evaluates like the model that was saved."""
    pkg = M.load_pkg()
    cfg = dict(M.TINY, fused=1, sgd_opt=M.rmsprop(3e-3))
    B, T = cfg["batch_size"], cfg["seg_len"]
    syms = M.markov1(B * T * 4, cfg["n_symbols"], seed=5)
    batches = list(M.segment_batches(syms, B, T, 4))
    gpu = pkg.host.Model(hosts[0], pkg.host.make_config(**dict(cfg, use_device=1)))
    for tok, tgt in batches[:3]:
        gpu.train_step(tok, tgt, 3e-3)
    gpu.save_coefs(str(tmp_path / "from_gpu.bin"))
    ref = pkg.host.Model(hosts[1], pkg.host.make_config(**dict(cfg, seed=7, use_device=0, nb_threads=2)))
    ref.load_coefs(str(tmp_path / "from_gpu.bin"))
    for n in gpu.param_names():
        assert np.array_equal(gpu.get_param(n), ref.get_param(n)), n
    ref.save_coefs(str(tmp_path / "from_checker.bin"))
    assert (tmp_path / "from_checker.bin").read_bytes() == (tmp_path / "from_gpu.bin").read_bytes()
    gpu2 = pkg.host.Model(hosts[0], pkg.host.make_config(**dict(cfg, seed=8, use_device=1)))
    gpu2.load_coefs(str(tmp_path / "from_checker.bin"))
    tok, tgt = batches[3]
    p1 = gpu.eval(tok)       # the memory of both models is empty for gpu2 only: compare a fresh segment
    gpu.close()
    gpu3 = pkg.host.Model(hosts[0], pkg.host.make_config(**dict(cfg, seed=9, use_device=1)))
    gpu3.load_coefs(str(tmp_path / "from_gpu.bin"))
    assert np.array_equal(gpu2.eval(tok), gpu3.eval(tok))
    assert p1.shape == (T, B, cfg["n_symbols"])
    for m in (ref, gpu2, gpu3):
        m.close()


@pytest.mark.parametrize("cfg_name", ["TINY", "C1"])
def test_training_100_steps_match_checker(hosts, cfg_name):
    """The 1e-5 bar after 1, 10 and 100 steps of the fused path (probabilities, loss, every
    parameter tensor), with a float64 evaluation of the same trajectory (the torch statement of
    tests/test_model_torch.py plus RMSProp in float64) as the arbiter: the fp32 checker is itself
    up to 1e-5 away from float64 in single tensors (zero-initialised bias vectors that consist of
    sign-like RMSProp updates of small gradients), so the kernels must be within 1e-5 of the
    float64 trajectory, and their distance to the checker may exceed 1e-5 only by the checker's
    own distance from float64.  Measured on an MI355X at the larger configuration: kernels to
    float64 <= 7.1e-6 on every tensor at every checked step, checker to float64 <= 1.03e-5."""
    import torch
    from test_model_torch import _torch_step
    pkg = M.load_pkg()
    cfg = dict(getattr(M, cfg_name))
    cfg["attn_len"] = [cfg["mem_len"] + cfg["seg_len"]] * cfg["n_layer"]
    lr, beta2, eps = 3e-4, 0.99, 1e-8
    hip = pkg.host.Model(hosts[0], pkg.host.make_config(**dict(cfg, use_device=1, fused=1, sgd_opt=M.rmsprop(lr))))
    ref = pkg.host.Model(hosts[1], pkg.host.make_config(**dict(cfg, use_device=0, nb_threads=8, fused=1,
                                                               sgd_opt=M.rmsprop(lr))))
    B, T, V, D = cfg["batch_size"], cfg["seg_len"], cfg["n_symbols"], cfg["d_model"]
    w64 = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in ref.params().items()}
    v64 = {k: torch.zeros_like(v) for k, v in w64.items()}
    mem = [torch.zeros(B, cfg["mem_len"], D, dtype=torch.float64) for _ in range(cfg["n_layer"])]
    syms = M.markov1(B * T * 100, V, seed=77)
    for step, (tok, tgt) in enumerate(M.segment_batches(syms, B, T, 100), 1):
        ph, lh = hip.train_step(tok, tgt, lr)
        pr, lr_ = ref.train_step(tok, tgt, lr)
        p64, nll64, inputs = _torch_step(w64, cfg, tok, tgt, mem)
        nll64.backward()
        with torch.no_grad():
            for k in w64:
                g = w64[k].grad
                v64[k] = beta2 * v64[k] + (1 - beta2) * g * g
                w64[k] -= lr * g / (v64[k].sqrt() + eps)
                w64[k].grad = None
        mem = [torch.cat([m[:, T:], x.detach().transpose(0, 1)], dim=1) for m, x in zip(mem, inputs)]
        if step in (1, 10, 100):
            assert M.relerr(ph, pr) <= 1e-5, step
            assert M.relerr(ph, p64.detach().numpy()) <= 1e-5, step
            assert abs(lh - lr_) <= 1e-5 * abs(lr_), step
            w_h, w_r = hip.params(), ref.params()
            for k in w_r:
                exact = w64[k].detach().numpy()
                own = M.rel_l2(w_r[k], exact)                  # the checker's fp32 noise
                assert M.rel_l2(w_h[k], exact) <= 1e-5, (step, k, M.rel_l2(w_h[k], exact))
                assert M.rel_l2(w_h[k], w_r[k]) <= 1e-5 + own, (step, k, M.rel_l2(w_h[k], w_r[k]), own)
    hip.close()
    ref.close()


# ---- parameters stored as bf16 (NC_TYPE_BF16, nncp.c:343-346) ------------------------------

def test_bf16_conversions_on_the_gpu(hip):
    """nc_convert f32 -> bf16 -> f32 on the device against torch's conversion, bit for bit
    (ties, neighbours of ties, subnormals, infinities; NaN stays NaN)"""
    import test_bf16_storage as S
    S.check_conversions(hip, M.load_pkg().binding)


@pytest.mark.parametrize("fused", [0, 1])
def test_bf16_parameters_follow_the_f32_route_on_the_gpu(hosts, fused):
    """One plain-SGD step of a model whose parameters are 2-byte tensors against the same model
    with f32 parameters that start at the same bf16-representable values and bf16-operand
    products: the same kernels meet the same operand bits, so probabilities and loss are equal,
    the f32 model's new weights are the bf16 model's master values, and the bf16 parameters are
    their rounding."""
    import test_bf16_storage as S
    B = M.load_pkg().binding
    (pa, la, wa, ma), (pb, lb, wb), w0 = S.check_master_and_parameters_against_the_f32_route(hosts[0], 1, fused)
    assert np.array_equal(pa, pb) and la == lb
    for k in w0:
        assert np.array_equal(ma[k], wb[k]), k
        assert np.array_equal(wa[k], B.bf16_widen(B.bf16_bits(ma[k]))), k


@pytest.mark.parametrize("fused,tol", [(0, 2e-2), (1, 2e-2)])
def test_bf16_parameter_model_matches_checker(hosts, fused, tol):
    """Four RMSProp steps with bf16 parameter storage, GPU against the checker (which emulates
    the operand rounding of the products).  Op by op both sides round the same values at the
    same places, but a value that fp32 noise carries across a rounding boundary changes an
    operand (or a stored parameter) by a whole bf16 unit, 2^-8 of its size: the results agree
    to 2e-7 on the smallest model and to a few 1e-3 here - not to fp32 accuracy - and most
    stored parameters are equal bit for bit.  The fused evaluation rounds activations at other
    places (product epilogues, attention operands).  One bar for both: the bf16 variant's 2e-2."""
    hp = M.load_pkg().host
    cfg = dict(M.C1, sgd_opt=M.rmsprop(3e-4), param_bf16=1)
    Bs, T, V = cfg["batch_size"], cfg["seg_len"], cfg["n_symbols"]
    batches = M.segment_batches(M.markov1(Bs * T * 4, V, seed=21), Bs, T, 4)
    gpu = hp.Model(hosts[0], hp.make_config(**dict(cfg, fused=fused, use_device=1)))
    ref = hp.Model(hosts[1], hp.make_config(**dict(cfg, fused=0, use_device=0, nb_threads=8)))
    ref.nc.nc_set_matmul_bf16(ref.ctx, 1)
    try:
        for k, v in ref.params().items():
            assert np.array_equal(gpu.get_param(k), v), k
        for tok, tgt in batches:
            ph, lh = gpu.train_step(tok, tgt, 3e-4)
            pr, lr_ = ref.train_step(tok, tgt, 3e-4)
            assert M.relerr(ph, pr) <= tol
            assert abs(lh - lr_) <= tol * abs(lr_)
        wh, wr = gpu.params(), ref.params()
    finally:
        ref.nc.nc_set_matmul_bf16(ref.ctx, 0)
        gpu.close()
        ref.close()
    for k in wr:
        if wr[k].ndim >= 2 and not k.startswith("b_r"):
            assert M.rel_l2(wh[k], wr[k]) <= 2e-2, (k, M.rel_l2(wh[k], wr[k]))
            if not fused:
                assert (wh[k] == wr[k]).mean() > 0.75, (k, (wh[k] == wr[k]).mean())  # (w_r: sign-like updates of tiny gradients)


def test_bf16_parameter_stream_round_trips_through_the_container(hosts, tmp_path):
    """use_bf16 = 2 in the file header: encoder and decoder both build the model with bf16
    parameters (the decoder learns it from the header), the file decodes to the input, and the
    size is within 2 % of the f32-parameter bf16 variant's."""
    hp = M.load_pkg().host
    n = 200
    mode = hp.MODE_SEGMENT | hp.CODER_CDF16
    syms = M.markov1(n, 40, seed=17)
    src = str(tmp_path / "in.bin")
    syms.astype(np.uint8).tofile(src)
    sizes = {}
    for use_bf16 in (1, 2):
        cfg = hp.make_config(**dict(M.TINY, fused=1, sgd_opt=M.rmsprop(), nb_threads=4, use_device=1))
        fp = hp.file_params(hosts[0], "3e-4,8,1e-4", "96,200,120", use_bf16=use_bf16, mode=mode)
        packed, back = str(tmp_path / ("out%d.nncp" % use_bf16)), str(tmp_path / ("back%d.bin" % use_bf16))
        st, _ = hp.encode_file(hosts[0], src, packed, cfg, fp)
        hp.decode_file(hosts[0], packed, back, use_device=1, nb_threads=4)
        assert open(back, "rb").read() == open(src, "rb").read()
        sizes[use_bf16] = os.path.getsize(packed)
    assert abs(sizes[2] - sizes[1]) <= max(3, 0.02 * sizes[1]), sizes


def test_bf16_parameter_files_cross_between_the_gpu_and_the_checker(hosts, tmp_path):
    """bf16 records (2 bytes per element) written by the product library and read by the
    checker's reader, and back: the same bytes"""
    hp = M.load_pkg().host
    cfg = dict(M.TINY, fused=1, sgd_opt=M.rmsprop(3e-3), param_bf16=1)
    Bs, T = cfg["batch_size"], cfg["seg_len"]
    gpu = hp.Model(hosts[0], hp.make_config(**dict(cfg, use_device=1)))
    for tok, tgt in M.segment_batches(M.markov1(Bs * T * 3, cfg["n_symbols"], seed=5), Bs, T, 3):
        gpu.train_step(tok, tgt, 3e-3)
    gpu.save_coefs(str(tmp_path / "from_gpu.bin"))
    ref = hp.Model(hosts[1], hp.make_config(**dict(cfg, fused=0, seed=7, use_device=0, nb_threads=2)))
    ref.load_coefs(str(tmp_path / "from_gpu.bin"))
    n = 0
    for k in gpu.param_names():
        assert np.array_equal(gpu.get_param(k), ref.get_param(k)), k
        n += gpu.get_param(k).size
    ref.save_coefs(str(tmp_path / "from_checker.bin"))
    assert (tmp_path / "from_checker.bin").read_bytes() == (tmp_path / "from_gpu.bin").read_bytes()
    assert os.path.getsize(str(tmp_path / "from_gpu.bin")) < 2 * n + 200 * len(gpu.param_names())
    gpu.close()
    ref.close()


def test_enwik8_profile_round_trips_a_small_file_on_gpu(hosts, tmp_path):
    """nncp's enwik8 profile as `nncp_profile` fills it (nncp.c:2515-2572: 20 layers of d1024, 8 heads of
    128, gated GELU 3072, RMSNorm before every block and at the end, 64 + 256 keys with per-layer
    position tables, Adam with clipping, bf16 products, a retrain pass with dropout after the
    block) on a file of two one-segment blocks and a ragged tail, through the file container: the decoder
    rebuilds the model from the header and returns the input."""
    hp = M.load_pkg().host
    cfg, fp = hp.profile(hosts[0], "enwik8")
    assert (cfg.n_layer, cfg.d_model, cfg.n_head, cfg.d_key, cfg.d_inner, cfg.mem_len, cfg.d_pos) == (20, 1024, 8, 128, 3072, 256, 320)
    cfg.use_device, cfg.fused, cfg.nb_threads = 1, 1, 4
    fp.mode = hp.MODE_SEGMENT | hp.CODER_CDF16
    # one training step per block instead of the profile's 100 000 symbols, so that this small
    # file has blocks to retrain between (the pass runs after every block but the last)
    import ctypes as C
    assert hosts[0].lib.nncp_parse_interp(C.byref(fp.block_len), b"2048") == 0
    n = cfg.batch_size * cfg.seg_len * 2 + 77
    syms = M.markov1(n, 256, seed=23)
    src, packed, back = (str(tmp_path / f) for f in ("in.bin", "out.nncp", "back.bin"))
    syms.astype(np.uint8).tofile(src)
    st, rst = hp.encode_file(hosts[0], src, packed, cfg, fp)
    assert st.n_symbols == n and st.n_steps == 2
    assert rst.n_steps >= 1                                   # the retrain pass ran (dropout on, op by op)
    assert 0 < os.path.getsize(packed) < n * 1.1              # an untrained model: about 8 bits a byte
    hp.decode_file(hosts[0], packed, back, use_device=1, nb_threads=4)
    assert open(back, "rb").read() == open(src, "rb").read()


@pytest.mark.gpu
@pytest.mark.parametrize("bf16", [0, 1])
def test_memory_window_moves_and_starts_over_without_changing_a_bit(monkeypatch, bf16):
    """A memory longer than the segment lives, on the GPU, in a store with room behind it: an
    update writes the new segment behind the window and moves the window instead of shifting the
    rows, and at the end of the store the rows that stay go back to its start.  Seven steps with
    room for one segment (the window starts over at every other update), with the default room
    (it does not) and on the checker (which shifts, nncp.c:1205-1221): the two GPU runs agree
    bit for bit in probabilities, loss and memories, and with the checker at the variant's bar.
    With bf16 products the consistency checker of the operand copies is on: the copy of the
    store is kept up to date over each written range, and a stale one ends the process."""
    hp = M.load_pkg().host
    cfg = dict(n_layer=2, d_model=128, n_head=2, d_inner=256, d_pos=48, mem_len=40, seg_len=16,
               batch_size=8, n_symbols=64, seed=5)
    n_steps = 7
    syms = M.markov1(cfg["batch_size"] * cfg["seg_len"] * n_steps, cfg["n_symbols"], seed=6)
    batches = M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], n_steps)
    runs = []
    for host, dev, room in ((M.hip_host(), 1, "1"), (M.hip_host(), 1, None), (M.ref_host(), 0, None)):
        if room:
            monkeypatch.setenv("NNCP_MEM_SLACK_SEGMENTS", room)
        else:
            monkeypatch.delenv("NNCP_MEM_SLACK_SEGMENTS", raising=False)
        m = hp.Model(host, hp.make_config(**dict(cfg, use_device=dev, fused=1, nb_threads=4, sgd_opt=M.rmsprop(3e-4))))
        m.nc.nc_set_matmul_bf16(m.ctx, bf16)
        old = m.nc.nc_set_bf16_shadow_check(bf16)
        out = []
        for tok, tgt in batches:
            p, loss = m.train_step(tok, tgt, 3e-4)
            out.append((p, loss, m.state()["mem"]))
        m.nc.nc_set_bf16_shadow_check(old)
        m.nc.nc_set_matmul_bf16(m.ctx, 0)
        m.close()
        runs.append(out)
    tol = 2e-2 if bf16 else 1e-5
    for (pa, la, ma), (pb, lb, mb), (pr, lr_, mr) in zip(*runs):
        assert np.array_equal(pa, pb) and la == lb
        for x, y, z in zip(ma, mb, mr):
            assert x.shape == z.shape
            assert np.array_equal(x, y)
            assert M.rel_l2(x, z) <= tol     # (hidden states: in the norm the variant's bar is stated in)
        assert M.relerr(pa, pr) <= tol and abs(la - lr_) <= tol * abs(lr_)
