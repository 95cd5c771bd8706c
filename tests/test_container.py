"""File container of the host side (host/container.c) on the CPU checker:
profiles, schedule text, the big-endian header against bytes assembled with the
reference's own writers (cutils.c / cp_utils.c compiled in place into
oracle/_ref), block lengths, and whole files through encode -> decode."""
import ctypes as C
import os

import numpy as np
import pytest

import modelutil as M
from conftest import ROOT, REF_LIB

REF_CODER = os.path.join(ROOT, "oracle", "_ref", "libnncp_coder_ref.so")


@pytest.fixture(scope="module")
def H():
    return M.ref_host()


@pytest.fixture(scope="module")
def pkg():
    return M.load_pkg()


class RefInterp(C.Structure):  # cp_utils.h:62-67
    _fields_ = [("n_steps", C.c_int), ("val", C.c_float * 9), ("pos", C.c_int64 * 8),
                ("decay_power", C.c_float)]


@pytest.fixture(scope="module")
def refc():
    if not os.path.exists(REF_CODER):
        pytest.skip("oracle/_ref not built")
    lib = C.CDLL(REF_CODER)
    libc = C.CDLL(None)
    libc.tmpfile.restype = C.c_void_p
    libc.fclose.argtypes = [C.c_void_p]
    libc.rewind.argtypes = [C.c_void_p]
    libc.fread.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
    libc.fread.restype = C.c_size_t
    for name, arg in (("fput_u8", C.c_uint8), ("fput_be16", C.c_uint16), ("fput_be32", C.c_uint32),
                      ("fput_f32", C.c_float)):
        getattr(lib, name).argtypes = [C.c_void_p, arg]
    lib.fput_sgd_opt.argtypes = [C.c_void_p, C.c_void_p]
    lib.parse_interp_param.argtypes = [C.POINTER(RefInterp), C.c_char_p]
    lib.dump_interp_param.argtypes = [C.c_void_p, C.POINTER(RefInterp)]
    lib.get_interp_param.restype = C.c_float
    lib.get_interp_param.argtypes = [C.POINTER(RefInterp), C.c_int64]
    lib.libc = libc
    return lib


class RefFile:
    """A tmpfile the reference's fput_* write into."""

    def __init__(self, refc):
        self.r, self.f = refc, refc.libc.tmpfile()

    def u8(self, v): self.r.fput_u8(self.f, v)
    def be16(self, v): self.r.fput_be16(self.f, v)
    def be32(self, v): self.r.fput_be32(self.f, v)
    def f32(self, v): self.r.fput_f32(self.f, v)

    def interp(self, p):  # fput_interp_params, nncp.c:1297-1306
        self.u8(p.n_steps)
        for i in range(p.n_steps + 1):
            self.f32(p.val[i])
        for i in range(p.n_steps):
            self.be32(p.pos[i])
        self.f32(p.decay_power)

    def bytes(self):
        self.r.libc.rewind(self.f)
        buf = C.create_string_buffer(4096)
        n = self.r.libc.fread(buf, 1, 4096, self.f)
        self.r.libc.fclose(self.f)
        return buf.raw[:n]


SCHEDULES = ["3e-4", "500000", "1.6e-4,10000,1.0e-4,p0.5", "100000,500000,100000,500000,500000",
             "0.5,10,0.25,20,0.125,30,1,40,2,50,3,60,4,70,5,80,6", "1,100,0,p2"]


@pytest.mark.parametrize("text", SCHEDULES)
def test_schedule_text_matches_reference_parser(H, refc, pkg, text):
    mine, theirs = pkg.host.NNCPInterp(), RefInterp()
    assert H.lib.nncp_parse_interp(C.byref(mine), text.encode()) == 0
    refc.parse_interp_param(C.byref(theirs), text.encode())
    assert mine.n_steps == theirs.n_steps and mine.decay_power == theirs.decay_power
    assert list(mine.val)[:mine.n_steps + 1] == list(theirs.val)[:mine.n_steps + 1]
    assert list(mine.pos)[:mine.n_steps] == list(theirs.pos)[:mine.n_steps]
    for pos in (0, 1, 9999, 10000, 10001, 123456, 5 * 10 ** 6):
        assert H.lib.nncp_interp(C.byref(mine), pos) == refc.get_interp_param(C.byref(theirs), pos)
    # text form: dump_interp_param into a tmpfile
    f = RefFile(refc)
    refc.dump_interp_param(f.f, C.byref(theirs))
    want = f.bytes().decode()
    buf = C.create_string_buffer(256)
    n = H.lib.nncp_format_interp(buf, 256, C.byref(mine))
    assert buf.value.decode() == want and n == len(want)


@pytest.mark.parametrize("text", ["", "x", "1,", "1,2", "1,2,", "1,p", "1,p2x", "1,2,3,4", "1,2,3;",
                                  "1," + ",".join("1,1" for _ in range(9))])
def test_schedule_syntax_errors(H, pkg, text):
    assert H.lib.nncp_parse_interp(C.byref(pkg.host.NNCPInterp()), text.encode()) == -1


def test_profiles(H, pkg):
    """batch_size / seg_len / n_symbols are the values the reference's own test and
    profile table state (tests/cuda_compatibility_tests_simple.c:33-52,
    src/neural/config/cuda_profiles.c); the rest is nncp_init_params, nncp.c:2464-2636."""
    hp = pkg.host
    want = {"default": (16, 32, 256), "enwik8": (32, 64, 256), "enwik9": (32, 64, 256), "lstm": (32, 20, 256),
            "lstm_fast": (256, 20, 256)}
    for name, (b, t, v) in want.items():
        cfg, fp = hp.profile(H, name)
        assert (cfg.batch_size, cfg.seg_len, cfg.n_symbols, cfg.seed) == (b, t, v, 123), name
        assert fp.max_size == -1 and fp.mode == 0
    cfg, fp = hp.profile(H, "default")
    assert (cfg.model_type, cfg.n_layer, cfg.d_model, cfg.n_head, cfg.d_key, cfg.d_inner, cfg.d_pos, cfg.mem_len) == \
        (0, 4, 256, 8, 32, 512, 32, 32)
    assert list(cfg.attn_len)[:5] == [64, 64, 64, 64, 0] and cfg.ln_flags == hp.LN_POST and cfg.ff_act == hp.FF_GELU
    assert (fp.lr.n_steps, fp.lr.pos[0], fp.block_len.val[0], fp.use_bf16) == (1, 156250, 500000, 0)
    assert abs(fp.lr.val[0] - 3e-4) < 1e-10 and abs(fp.lr.val[1] - 1e-4) < 1e-10 and cfg.retrain_period == 0
    for name, rlen in (("enwik8", 15000000), ("enwik9", 7500000)):
        cfg, fp = hp.profile(H, name)
        assert (cfg.n_layer, cfg.d_model, cfg.n_head, cfg.d_key, cfg.d_value, cfg.d_inner, cfg.d_pos, cfg.mem_len) == \
            (20, 1024, 8, 128, 128, 3072, 320, 256)
        assert cfg.ff_act == hp.FF_GEGLU and cfg.ln_flags == hp.LN_PRE | hp.LN_FINAL | hp.LN_RMSNORM
        assert (cfg.tied_w_r, cfg.tied_b_r, cfg.use_w_r, cfg.use_bias) == (0, 1, 1, 1)
        assert (cfg.retrain_period, cfg.retrain_len, cfg.has_retrain_lr, fp.use_bf16) == (1, rlen, 1, 1)
        assert abs(cfg.dropout_prob - 0.19) < 1e-7 and abs(cfg.sgd_opt.gradient_clip - 0.05) < 1e-8
        assert abs(cfg.init_range - 0.79) < 1e-7 and all(a == 320 for a in list(cfg.attn_len)[:20])
        assert fp.lr.decay_power == 0.5 and fp.lr.pos[0] == 10000 and cfg.retrain_lr.decay_power == 0.5
        assert fp.block_len.n_steps == (2 if name == "enwik8" else 0)
    cfg, fp = hp.profile(H, "lstm")
    assert (cfg.model_type, cfg.n_layer, cfg.lstm_n_cells, cfg.lstm_n_cells2, cfg.lstm_n_embed_out, cfg.lstm_type,
            cfg.lstm_full_connect, cfg.lstm_use_layer_norm) == (1, 4, 352, 352, 4, hp.LSTM_CLAMPED, 1, 1)
    assert abs(fp.lr.val[0] - 4e-3) < 1e-9 and abs(cfg.sgd_opt.eps - 1e-10) < 1e-16 and cfg.sgd_opt.gradient_clip == 0
    cfg, fp = hp.profile(H, "lstm_fast")
    assert cfg.lstm_n_cells == 512 and fp.block_len.val[0] == 1e8 and abs(fp.lr.val[0] - 1e-2) < 1e-9
    with pytest.raises(ValueError):
        hp.profile(H, "enwik10")


def _expected_header(refc, cfg, fp):
    """The header as the reference writes it: nncp_write_file_header (nncp.c:2665-2690)
    then trf_write_params (nncp.c:1333-1365) or lstm_write_params (nncp.c:2198-2211),
    every field through the reference's own fput_* and fput_sgd_opt."""
    f = RefFile(refc)
    f.be32(0xb727ac58); f.be16(1); f.u8(cfg.use_device); f.u8(fp.use_bf16)
    f.be16(cfg.batch_size); f.be16(cfg.seg_len); f.be16(cfg.n_symbols); f.be32(cfg.seed)
    f.interp(fp.lr); f.interp(fp.block_len)
    f.be32(cfg.retrain_period)
    if cfg.retrain_period:
        f.be32(cfg.retrain_len); f.u8(cfg.has_retrain_lr)
        if cfg.has_retrain_lr:
            f.interp(cfg.retrain_lr)
    f.u8(cfg.model_type)
    if cfg.model_type == 0:
        f.u8(cfg.n_layer); f.u8(cfg.n_head)
        for v in (cfg.d_key, cfg.d_value, cfg.d_inner, cfg.d_pos, cfg.mem_len):
            f.be16(v)
        for i in range(cfg.n_layer):
            f.be16(cfg.attn_len[i])
        for v in (0, cfg.use_bias, cfg.use_w_r, cfg.tied_w_r, cfg.tied_b_r, cfg.query_bias, 0, cfg.ln_flags):
            f.u8(v)
        f.f32(cfg.init_range); f.f32(cfg.embed_mult); f.u8(cfg.ff_act)
        refc.fput_sgd_opt(f.f, C.byref(cfg.sgd_opt))
        if cfg.retrain_period:
            f.f32(cfg.dropout_prob); f.f32(cfg.dropout_att_prob)
        f.u8(0)
    else:
        f.u8(cfg.lstm_type); f.u8(cfg.n_layer); f.u8(cfg.lstm_n_embed_out)
        f.be16(cfg.lstm_n_cells); f.be16(cfg.seg_len)
        f.u8(cfg.lstm_use_layer_norm | cfg.lstm_full_connect << 1)
        refc.fput_sgd_opt(f.f, C.byref(cfg.sgd_opt))
        f.f32(0.0); f.f32(cfg.lstm_forget_bias); f.u8(0)
    return f.bytes()


def _header(H, cfg, fp):
    buf = C.create_string_buffer(1024)
    n = H.lib.nncp_header_write(buf, 1024, C.byref(cfg), C.byref(fp))
    assert n > 0
    return buf.raw[:n]


CFG_FIELDS = ["n_layer", "d_model", "n_head", "d_key", "d_value", "d_inner", "d_pos", "mem_len", "use_bias", "use_w_r",
              "tied_w_r", "tied_b_r", "query_bias", "ln_flags", "ff_act", "init_range", "embed_mult", "batch_size",
              "seg_len", "n_symbols", "seed", "use_device", "dropout_prob", "dropout_att_prob", "retrain_period",
              "retrain_len", "has_retrain_lr", "model_type", "lstm_n_cells", "lstm_n_cells2", "lstm_n_embed_out",
              "lstm_type", "lstm_full_connect", "lstm_use_layer_norm", "lstm_forget_bias"]


def _interp_tuple(p):
    return (p.n_steps, list(p.val)[:p.n_steps + 1], list(p.pos)[:p.n_steps], p.decay_power)


@pytest.mark.parametrize("name", ["default", "enwik8", "enwik9", "lstm", "lstm_fast", "tiny_variant"])
def test_header_bytes_and_round_trip(H, refc, pkg, name):
    hp = pkg.host
    if name == "tiny_variant":
        cfg = hp.make_config(**dict(M.TINY, query_bias=1, tied_b_r=0, attn_len=[10, 16], ff_act=hp.FF_RELU,
                                    use_device=0, retrain_period=700, retrain_len=4000, dropout_prob=0.1,
                                    sgd_opt=pkg.binding.SGDOptParams(algo=0, lr=0.1)))
        fp = hp.file_params(H, "1e-3,100,1e-4", "600,1500,1200", use_bf16=0)
    else:
        cfg, fp = hp.profile(H, name)
    got = _header(H, cfg, fp)
    assert got == _expected_header(refc, cfg, fp)
    cfg2, fp2, used = hp.NNCPConfig(), hp.NNCPFileParams(), C.c_size_t()
    assert H.lib.nncp_header_read(got + b"tail", len(got) + 4, C.byref(cfg2), C.byref(fp2), C.byref(used)) == 0
    assert used.value == len(got)
    for k in CFG_FIELDS:
        assert getattr(cfg2, k) == getattr(cfg, k), k
    assert list(cfg2.attn_len) == list(cfg.attn_len)
    o1, o2 = cfg.sgd_opt, cfg2.sgd_opt
    assert o1.algo == o2.algo
    if o1.algo:
        assert (o1.beta1, o1.beta2, o1.eps, o1.gradient_clip) == (o2.beta1, o2.beta2, o2.eps, o2.gradient_clip)
    assert _interp_tuple(fp2.lr) == _interp_tuple(fp.lr) and _interp_tuple(fp2.block_len) == _interp_tuple(fp.block_len)
    if cfg.has_retrain_lr:
        assert _interp_tuple(cfg2.retrain_lr) == _interp_tuple(cfg.retrain_lr)
    assert fp2.use_bf16 == fp.use_bf16 and _header(H, cfg2, fp2) == got


def test_header_rejects_what_it_cannot_hold(H, pkg):
    hp = pkg.host
    cfg, fp = hp.profile(H, "default")
    good = _header(H, cfg, fp)
    out = (hp.NNCPConfig(), hp.NNCPFileParams())

    def read(data):
        return H.lib.nncp_header_read(data, len(data), C.byref(out[0]), C.byref(out[1]), None)
    assert read(good) == 0
    assert read(b"\x00" + good[1:]) == -1                       # magic
    assert read(good[:5] + b"\x02" + good[6:]) == -1            # version
    for n in range(len(good)):
        assert read(good[:n]) == -1                             # truncated anywhere
    off_model = good.index(bytes([0, 4, 8, 0, 32]))             # model id, n_layer, n_head, d_key
    tied_embed = off_model + 1 + 2 + 2 * 5 + 2 * 4
    assert read(good[:tied_embed] + b"\x01" + good[tied_embed + 1:]) == -2
    assert read(good[:tied_embed + 6] + b"\x01" + good[tied_embed + 7:]) == -2      # rot_pos
    assert read(good[:off_model] + b"\x07" + good[off_model + 1:]) == -1            # unknown model id
    # sizes a model cannot be built from (they would divide by zero or end the process in the
    # model constructor) make the header invalid
    assert read(good[:8] + b"\x00\x00" + good[10:]) == -1                           # batch_size 0
    assert read(good[:10] + b"\x00\x00" + good[12:]) == -1                          # seg_len 0
    assert read(good[:12] + b"\x00\x01" + good[14:]) == -1                          # one symbol
    assert read(good[:off_model + 1] + b"\x00" + good[off_model + 2:]) == -1         # no layers
    assert read(good[:off_model + 2] + b"\x00" + good[off_model + 3:]) == -1         # no heads
    assert read(good[:off_model + 3] + b"\x00\x00" + good[off_model + 5:]) == -1    # d_key 0
    ff_act = tied_embed + 8 + 8
    assert good[ff_act] == hp.FF_GELU and read(good[:ff_act] + b"\x09" + good[ff_act + 1:]) == -1
    nan = b"\x7f\xc0\x00\x00"
    assert read(good[:ff_act - 8] + nan + good[ff_act - 4:]) == -1                   # init_range NaN
    assert H.lib.nncp_header_write(C.create_string_buffer(20), 20, C.byref(cfg), C.byref(fp)) == 0
    # this build's RMSProp travels as algorithm 16 with Adam's four fields
    cfg.sgd_opt = M.rmsprop()
    assert read(_header(H, cfg, fp)) == 0 and out[0].sgd_opt.algo == 16 and abs(out[0].sgd_opt.beta2 - 0.99) < 1e-7


def test_block_len_schedule(H, pkg):
    """nncp.c:3452-3457 restated: lrintf of the schedule, whole steps, at least one."""
    hp = pkg.host
    cfg = hp.make_config(**M.TINY)                              # 3 streams x 8 = 24 symbols a step
    fp = hp.file_params(H, block_len="100,1000,400,2000,10")
    for pos, remaining in ((0, 10 ** 6), (500, 10 ** 6), (1000, 10 ** 6), (1999, 10 ** 6), (2000, 10 ** 6), (0, 50),
                           (5000, 7)):
        v = int(np.rint(np.float32(H.lib.nncp_interp(C.byref(fp.block_len), pos))))
        want = min(max(v // 24, 1) * 24, remaining)
        assert H.lib.nncp_block_len(C.byref(cfg), C.byref(fp.block_len), pos, remaining) == want, pos


def test_coder_sink_gives_the_same_bytes(H, pkg):
    hp = pkg.host
    rng = np.random.default_rng(3)
    probs, bits = rng.integers(1, 32768, 30000).tolist(), rng.integers(0, 2, 30000).tolist()
    big = np.zeros(80000, np.uint8)
    st = hp.NNCPPutBit()
    H.lib.nncp_put_bit_init(C.byref(st), big.ctypes.data, big.size)
    for p, b in zip(probs, bits):
        H.lib.nncp_put_bit(C.byref(st), p, b)
    want = bytes(big[:H.lib.nncp_put_bit_flush(C.byref(st))])
    out = bytearray()
    SINK = C.CFUNCTYPE(None, C.c_void_p, C.POINTER(C.c_uint8), C.c_size_t)
    cb = SINK(lambda opaque, p, n: out.extend(bytes(p[:n])))
    small = np.zeros(97, np.uint8)
    st = hp.NNCPPutBit()
    H.lib.nncp_put_bit_init(C.byref(st), small.ctypes.data, small.size)
    H.lib.nncp_put_bit_set_sink(C.byref(st), C.cast(cb, C.c_void_p), None)
    for p, b in zip(probs, bits):
        H.lib.nncp_put_bit(C.byref(st), p, b)
    assert H.lib.nncp_put_bit_flush(C.byref(st)) == len(want) and bytes(out) == want and not st.overflow


# ---- whole files ---------------------------------------------------------------------
def _write(path, syms, wide):
    data = np.asarray(syms)
    (data.astype(">u2") if wide else data.astype(np.uint8)).tofile(path)


@pytest.mark.parametrize("case", ["reference_stream", "fast_stream", "wide_symbols", "retrain", "lstm"])
def test_file_round_trip(H, pkg, tmp_path, case):
    hp = pkg.host
    n = 1500
    kw, mode, blocks, wide = dict(M.TINY, use_device=0), 0, "480,900,240", False
    if case == "fast_stream":
        kw["fused"], mode = 1, hp.MODE_SEGMENT | hp.CODER_CDF16
    elif case == "wide_symbols":
        kw["n_symbols"], wide, mode = 300, True, hp.MODE_SEGMENT
    elif case == "retrain":
        kw.update(retrain_period=400, retrain_len=1000, dropout_prob=0.1, retrain_lr=1e-4)
        mode = hp.MODE_SEGMENT
    if case == "lstm":
        cfg = hp.make_lstm_config(n_layer=2, lstm_n_cells=12, batch_size=3, seg_len=8, n_symbols=40, use_device=0)
        mode = hp.MODE_SEGMENT
    else:
        cfg = hp.make_config(**kw)
    syms = M.markov1(n, cfg.n_symbols, seed=31)
    src, packed, back = (str(tmp_path / x) for x in ("in.bin", "out.nncp", "back.bin"))
    _write(src, syms, wide)
    fp = hp.file_params(H, "3e-4,50,1e-4", blocks, mode=mode)
    st, rst = hp.encode_file(H, src, packed, cfg, fp)
    assert st.n_symbols == n and (rst.n_steps > 0) == (case == "retrain")
    st2, rst2 = hp.decode_file(H, packed, back, use_device=0)
    assert open(back, "rb").read() == open(src, "rb").read()
    assert st2.n_symbols == n and rst2.n_steps == rst.n_steps
    # layout: header, flag byte, 32-bit count, payload
    raw = open(packed, "rb").read()
    head = _header(H, cfg, fp)
    assert raw[:len(head)] == head
    assert raw[len(head)] == (mode & 7) << 1 | (cfg.fused << 4)
    assert int.from_bytes(raw[len(head) + 1:len(head) + 5], "big") == n
    if case in ("reference_stream", "fast_stream"):
        # the payload is what the in-memory block loop writes for the same block lengths
        m = hp.Model(H, cfg)
        out, pos = bytearray(), 0
        cap = 8 * n + 1024
        buf = np.zeros(cap, np.uint8)
        pb = hp.NNCPPutBit()
        H.lib.nncp_put_bit_init(C.byref(pb), buf.ctypes.data, cap)
        stats = hp.NNCPStats()
        while pos < n:
            ln = H.lib.nncp_block_len(C.byref(cfg), C.byref(fp.block_len), pos, n - pos)
            blk = syms[pos:pos + ln].astype(np.uint16)
            H.lib.nncp_process_block(m.ptr, C.byref(pb), None, blk.ctypes.data, ln, 0, mode, C.byref(fp.lr),
                                     C.byref(stats))
            pos += ln
        out = bytes(buf[:H.lib.nncp_put_bit_flush(C.byref(pb))])
        m.close()
        assert raw[len(head) + 5:] == out


def test_file_edge_cases(H, pkg, tmp_path, capfd):
    hp = pkg.host
    cfg = hp.make_config(**dict(M.TINY, use_device=0))
    fp = hp.file_params(H, block_len="240", mode=hp.MODE_SEGMENT)
    src, packed, back = (str(tmp_path / x) for x in ("in.bin", "out.nncp", "back.bin"))
    # empty input: header and a zero count, decodes to an empty file
    _write(src, [], False)
    hp.encode_file(H, src, packed, cfg, fp)
    hp.decode_file(H, packed, back, use_device=0)
    assert os.path.getsize(back) == 0
    # max_size truncates (nncp --max_size)
    syms = M.markov1(700, 40, seed=2)
    _write(src, syms, False)
    fp.max_size = 333
    st, _ = hp.encode_file(H, src, packed, cfg, fp)
    hp.decode_file(H, packed, back, use_device=0)
    assert st.n_symbols == 333 and open(back, "rb").read() == bytes(syms[:333].astype(np.uint8))
    # a symbol outside the alphabet, a missing file, a file from the preprocessor, garbage
    fp.max_size = -1
    _write(src, [1, 2, 40, 3], False)
    with pytest.raises(RuntimeError):
        hp.encode_file(H, src, packed, cfg, fp)
    assert "outside the alphabet" in capfd.readouterr().err
    with pytest.raises(RuntimeError):
        hp.encode_file(H, str(tmp_path / "missing"), packed, cfg, fp)
    _write(src, syms, False)
    hp.encode_file(H, src, packed, cfg, fp)
    raw = bytearray(open(packed, "rb").read())
    flag_at = len(_header(H, cfg, fp))
    raw[flag_at] |= 1
    open(packed, "wb").write(bytes(raw))
    with pytest.raises(RuntimeError):
        hp.decode_file(H, packed, back, use_device=0)
    assert "preprocessor" in capfd.readouterr().err
    open(packed, "wb").write(b"not an nncp file")
    with pytest.raises(RuntimeError):
        hp.decode_file(H, packed, back, use_device=0)
    assert "invalid file header" in capfd.readouterr().err
