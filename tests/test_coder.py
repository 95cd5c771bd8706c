"""The host coders against the reference's own arith.c / cp_utils.c, compiled
in place into oracle/_ref/libnncp_coder_ref.so (see oracle/Makefile).  Skipped
when that library was not built (no reference tree at build time)."""
import ctypes as C
import os

import numpy as np
import pytest

from conftest import ROOT, REF_LIB

REF_CODER = os.path.join(ROOT, "oracle", "_ref", "libnncp_coder_ref.so")
HOST_REF = os.path.join(ROOT, "oracle", "libnncp_host_ref.so")

WRITE_FUNC = C.CFUNCTYPE(None, C.c_void_p, C.POINTER(C.c_uint8), C.c_size_t)
READ_FUNC = C.CFUNCTYPE(C.c_ssize_t, C.c_void_p, C.POINTER(C.c_uint8), C.c_size_t)


class RefPutBit(C.Structure):  # arith.h:32-43
    _fields_ = [("range", C.c_uint32), ("low", C.c_uint32), ("current_byte", C.c_uint8),
                ("n_bytes", C.c_uint32), ("buf", C.POINTER(C.c_uint8)), ("buf_size", C.c_size_t),
                ("idx", C.c_size_t), ("write_func", WRITE_FUNC), ("opaque", C.c_void_p),
                ("byte_count", C.c_uint64)]


class RefGetBit(C.Structure):  # arith.h:50-61
    _fields_ = [("buf", C.POINTER(C.c_uint8)), ("buf_len", C.c_int), ("buf_size", C.c_int),
                ("idx", C.c_int), ("low", C.c_uint32), ("range", C.c_uint32),
                ("eof_reached", C.c_int), ("read_func", READ_FUNC), ("opaque", C.c_void_p),
                ("byte_count", C.c_uint64)]


@pytest.fixture(scope="module")
def refc():
    if not os.path.exists(REF_CODER):
        pytest.skip("oracle/_ref not built")
    # (vec_sum_f32 comes from the checker library the reference objects were linked against;
    # nothing is loaded into the global namespace, where it would capture the nc_* calls of
    # every library loaded later)
    lib = C.CDLL(REF_CODER)
    lib.put_bit_init.argtypes = [C.POINTER(RefPutBit), C.POINTER(C.c_uint8), C.c_int, WRITE_FUNC, C.c_void_p]
    lib.put_bit.argtypes = [C.POINTER(RefPutBit), C.c_int, C.c_int]
    lib.put_bit_flush.restype = C.c_int64
    lib.put_bit_flush.argtypes = [C.POINTER(RefPutBit)]
    lib.get_bit_init.argtypes = [C.POINTER(RefGetBit), C.POINTER(C.c_uint8), C.c_size_t, READ_FUNC, C.c_void_p]
    lib.get_bit.argtypes = [C.POINTER(RefGetBit), C.c_int]
    lib.write_sym.argtypes = [C.POINTER(RefPutBit), C.POINTER(C.c_float), C.c_int, C.c_int]
    lib.read_sym.argtypes = [C.POINTER(RefGetBit), C.POINTER(C.c_float), C.c_int]
    lib.get_interp_param.restype = C.c_float
    return lib


@pytest.fixture(scope="module")
def hostc(pkg_mod):
    return pkg_mod.host.Host(HOST_REF, REF_LIB)


@pytest.fixture(scope="module")
def pkg_mod():
    from conftest import load_pkg
    return load_pkg()


class RefEncoder:
    def __init__(self, lib):
        self.lib, self.out = lib, bytearray()
        self.buf = (C.c_uint8 * 4096)()
        self.cb = WRITE_FUNC(lambda opaque, p, n: self.out.extend(bytes(p[:n])))
        self.st = RefPutBit()
        lib.put_bit_init(C.byref(self.st), self.buf, 4096, self.cb, None)

    def finish(self):
        self.lib.put_bit_flush(C.byref(self.st))
        return bytes(self.out)


def _host_encoder(pkg_mod, hostc, cap):
    st = pkg_mod.host.NNCPPutBit()
    buf = np.zeros(cap, dtype=np.uint8)
    hostc.lib.nncp_put_bit_init(C.byref(st), buf.ctypes.data, cap)
    return st, buf


@pytest.mark.parametrize("kind", ["uniform", "skewed", "carry"])
def test_range_coder_is_bit_compatible_with_reference(refc, hostc, pkg_mod, kind):
    rng = np.random.default_rng(5)
    n = 20000
    if kind == "uniform":
        probs = rng.integers(1, 32768, n)
        bits = rng.integers(0, 2, n)
    elif kind == "skewed":
        probs = np.where(rng.random(n) < 0.5, 32767, 1)
        bits = (rng.random(n) < probs / 32768.0).astype(int) ^ 1
    else:  # long runs of the likely symbol at extreme probabilities: 0xff carry chains
        probs = np.full(n, 32767)
        bits = np.zeros(n, dtype=int)
        bits[::977] = 1
    ref = RefEncoder(refc)
    st, buf = _host_encoder(pkg_mod, hostc, n * 2 + 64)
    for p, b in zip(probs.tolist(), bits.tolist()):
        refc.put_bit(C.byref(ref.st), p, b)
        hostc.lib.nncp_put_bit(C.byref(st), p, b)
    expect = ref.finish()
    got = bytes(buf[:hostc.lib.nncp_put_bit_flush(C.byref(st))])
    assert got == expect
    # both decoders read the stream back
    gb = pkg_mod.host.NNCPGetBit()
    data = np.frombuffer(got, dtype=np.uint8).copy()
    hostc.lib.nncp_get_bit_init(C.byref(gb), data.ctypes.data, data.size)
    rgb = RefGetBit()
    rbuf = (C.c_uint8 * len(expect)).from_buffer_copy(expect)
    refc.get_bit_init(C.byref(rgb), rbuf, len(expect), READ_FUNC(), None)
    for p, b in zip(probs.tolist(), bits.tolist()):
        assert hostc.lib.nncp_get_bit(C.byref(gb), p) == b
        assert refc.get_bit(C.byref(rgb), p) == b


@pytest.mark.parametrize("n_symb", [2, 3, 256, 1000])
def test_symbol_coder_matches_reference_and_round_trips(refc, hostc, pkg_mod, n_symb):
    rng = np.random.default_rng(n_symb)
    n = 300
    probs = rng.dirichlet(np.full(n_symb, 0.3), size=n).astype(np.float32)
    probs[0] = 0
    probs[0, n_symb // 2] = 1.0  # one-hot: clamps to [1, 32767]
    syms = [int(rng.choice(n_symb, p=p.astype(np.float64) / p.astype(np.float64).sum())) for p in probs]
    ref = RefEncoder(refc)
    st, buf = _host_encoder(pkg_mod, hostc, n * 8 + 64)
    for p, s in zip(probs, syms):
        refc.write_sym(C.byref(ref.st), p.ctypes.data_as(C.POINTER(C.c_float)), n_symb, s)
        hostc.lib.nncp_write_sym(C.byref(st), p.ctypes.data, n_symb, s)
    expect = ref.finish()
    got = bytes(buf[:hostc.lib.nncp_put_bit_flush(C.byref(st))])
    assert got == expect
    gb = pkg_mod.host.NNCPGetBit()
    data = np.frombuffer(got, dtype=np.uint8).copy()
    hostc.lib.nncp_get_bit_init(C.byref(gb), data.ctypes.data, data.size)
    for p, s in zip(probs, syms):
        assert hostc.lib.nncp_read_sym(C.byref(gb), p.ctypes.data, n_symb) == s
    # code length is close to the ideal -sum log2 p
    ideal = -sum(np.log2(max(float(p[s]), 2.0 ** -15)) for p, s in zip(probs[1:], syms[1:]))
    assert len(got) * 8 <= ideal + 0.02 * ideal + 64


@pytest.mark.parametrize("V", [2, 256, 16384])
def test_cdf_symbol_coder_round_trip_and_length(ref, hostc, pkg_mod, V):
    rng = np.random.default_rng(V)
    n = 200
    logits = (rng.standard_normal((n, V)) * 3).astype(np.float32)
    cdf = ref.numpy(ref.nc_soft_max_cdf16(ref.tensor(logits)), free=True)
    p = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    syms = [int(rng.choice(V, p=row)) for row in p]
    st, buf = _host_encoder(pkg_mod, hostc, n * 8 + 64)
    for row, s in zip(cdf, syms):
        hostc.lib.nncp_write_sym_cdf(C.byref(st), row.ctypes.data, V, s)
    got = buf[:hostc.lib.nncp_put_bit_flush(C.byref(st))].copy()
    gb = pkg_mod.host.NNCPGetBit()
    hostc.lib.nncp_get_bit_init(C.byref(gb), got.ctypes.data, got.size)
    for row, s in zip(cdf, syms):
        assert hostc.lib.nncp_read_sym_cdf(C.byref(gb), row.ctypes.data, V) == s
    ideal = -sum(np.log2(row[s]) for row, s in zip(p, syms))
    assert got.size * 8 <= ideal * 1.02 + 64


@pytest.mark.parametrize("V", [2, 3, 256, 1000, 16384, 65535])
def test_cdf_path_holds_what_the_coder_reads_and_codes_the_same_bytes(ref, hostc, pkg_mod, V):
    """nc_cdf_path against a walk of the tree written here (the split point of every level,
    zero below the leaf), and nncp_write_sym_cdf_path on its columns against nncp_write_sym_cdf
    on the whole rows: the same bytes.  Symbols include both ends and, for the kernel's sake,
    values outside the alphabet (they index nothing outside the column)."""
    rng = np.random.default_rng(V + 1)
    n = 120
    logits = (rng.standard_normal((n, V)) * 3).astype(np.float32)
    cdf_t = ref.nc_soft_max_cdf16(ref.tensor(logits))
    cdf = ref.numpy(ref.dup(cdf_t))
    syms = rng.integers(0, V, n).astype(np.int32)
    syms[:2] = [0, V - 1]
    wild = syms.copy()
    wild[5:9] = [-1, V, 2 ** 31 - 1, -2 ** 31]
    levels = max(1, int(np.ceil(np.log2(V))))

    def walk(row, s):
        out, start, m = [], 0, V
        while m > 1:
            m0 = m >> 1
            out.append(int(row[start + m0]))
            if s >= start + m0:
                start, m = start + m0, m - m0
            else:
                m = m0
        return out + [0] * (levels - len(out))
    path = ref.numpy(ref.nc_cdf_path(ref.dup(cdf_t), ref.tensor(wild)), free=True)
    ref.free(cdf_t)
    assert path.shape == (n, levels) and path.dtype == np.uint16
    for c in range(n):
        assert path[c].tolist() == walk(cdf[c], int(wild[c])), c
    path = np.ascontiguousarray(path)
    a, abuf = _host_encoder(pkg_mod, hostc, n * 8 + 64)
    b, bbuf = _host_encoder(pkg_mod, hostc, n * 8 + 64)
    for c in range(n):
        if wild[c] != syms[c]:
            continue
        hostc.lib.nncp_write_sym_cdf(C.byref(a), cdf[c].ctypes.data, V, int(syms[c]))
        hostc.lib.nncp_write_sym_cdf_path(C.byref(b), path[c].ctypes.data, V, int(syms[c]))
    na, nb = hostc.lib.nncp_put_bit_flush(C.byref(a)), hostc.lib.nncp_put_bit_flush(C.byref(b))
    assert na == nb and bytes(abuf[:na]) == bytes(bbuf[:nb]) and na > 0


def test_interp_matches_reference(refc, hostc, pkg_mod):
    class RefInterp(C.Structure):  # cp_utils.h:60-67
        _fields_ = [("n_steps", C.c_int), ("val", C.c_float * 9), ("pos", C.c_int64 * 8),
                    ("decay_power", C.c_float)]
    for power in (0.0, 0.5, 0.7):
        a, b = RefInterp(), pkg_mod.host.NNCPInterp()
        for s in (a, b):
            s.n_steps = 2
            s.val[0], s.val[1], s.val[2] = 3e-4, 1e-4, 5e-5
            s.pos[0], s.pos[1] = 1000, 5000
            s.decay_power = power
        refc.get_interp_param.argtypes = [C.POINTER(RefInterp), C.c_int64]
        for pos in (0, 1, 999, 1000, 3000, 4999, 5000, 123456):
            assert refc.get_interp_param(C.byref(a), pos) == hostc.lib.nncp_interp(C.byref(b), pos)


GOLDEN = os.path.join(ROOT, "tests", "golden", "coder_vectors.npz")


def test_coders_reproduce_committed_reference_vectors(hostc, pkg_mod):
    """The same comparison without the reference tree: tests/golden/coder_vectors.npz holds
    inputs and the bytes / values that the reference's arith.c and cp_utils.c gave for them
    (written by tests/golden/make_coder_vectors.py)."""
    g = np.load(GOLDEN)
    for kind in ("uniform", "skewed", "carry"):
        probs, bits = g["rc_%s_prob0" % kind], g["rc_%s_bits" % kind]
        st, buf = _host_encoder(pkg_mod, hostc, probs.size * 2 + 64)
        for p, b in zip(probs.tolist(), bits.tolist()):
            hostc.lib.nncp_put_bit(C.byref(st), p, b)
        got = buf[:hostc.lib.nncp_put_bit_flush(C.byref(st))].copy()
        assert np.array_equal(got, g["rc_%s_bytes" % kind]), kind
        gb = pkg_mod.host.NNCPGetBit()
        hostc.lib.nncp_get_bit_init(C.byref(gb), got.ctypes.data, got.size)
        assert [hostc.lib.nncp_get_bit(C.byref(gb), p) for p in probs.tolist()] == bits.tolist(), kind
    for n_symb in (2, 3, 256, 1000):
        probs, syms = g["sym_%d_probs" % n_symb], g["sym_%d_syms" % n_symb]
        st, buf = _host_encoder(pkg_mod, hostc, syms.size * 8 + 64)
        for p, s in zip(probs, syms.tolist()):
            hostc.lib.nncp_write_sym(C.byref(st), np.ascontiguousarray(p).ctypes.data, n_symb, s)
        got = buf[:hostc.lib.nncp_put_bit_flush(C.byref(st))].copy()
        assert np.array_equal(got, g["sym_%d_bytes" % n_symb]), n_symb
        gb = pkg_mod.host.NNCPGetBit()
        hostc.lib.nncp_get_bit_init(C.byref(gb), got.ctypes.data, got.size)
        for p, s in zip(probs, syms.tolist()):
            assert hostc.lib.nncp_read_sym(C.byref(gb), np.ascontiguousarray(p).ctypes.data, n_symb) == s
    for i, power in enumerate(g["interp_power"]):
        s = pkg_mod.host.NNCPInterp(n_steps=2, decay_power=float(power))
        for k, v in enumerate(g["interp_val"]):
            s.val[k] = float(v)
        for k, v in enumerate(g["interp_pos"]):
            s.pos[k] = int(v)
        got = [hostc.lib.nncp_interp(C.byref(s), int(p)) for p in g["interp_at"]]
        assert np.array_equal(np.array(got, dtype=np.float32), g["interp_out"][i]), power
