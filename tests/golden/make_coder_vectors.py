"""Writes tests/golden/coder_vectors.npz: inputs and the bytes / values that the
reference's own coders produce for them.  The coders are arith.c, cp_utils.c and
cutils.c of the reference tree, compiled in place into
oracle/_ref/libnncp_coder_ref.so by oracle/Makefile (`make -C oracle ref`); this
script only calls that library.  Run it where the reference tree is present:

    python tests/golden/make_coder_vectors.py

Contents (all little-endian numpy arrays):
  rc_<kind>_prob0, rc_<kind>_bits, rc_<kind>_bytes   put_bit / put_bit_flush (arith.c:122-207)
  sym_<V>_probs, sym_<V>_syms, sym_<V>_bytes         write_sym (cp_utils.c:299-323)
  interp_val, interp_pos, interp_power, interp_at, interp_out   get_interp_param (cp_utils.c:381-410)
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import test_coder as T  # noqa: E402  (structures and the reference encoder wrapper)


def range_coder_case(kind, n=4000):
    rng = np.random.default_rng({"uniform": 11, "skewed": 12, "carry": 13}[kind])
    if kind == "uniform":
        probs = rng.integers(1, 32768, n)
        bits = rng.integers(0, 2, n)
    elif kind == "skewed":
        probs = np.where(rng.random(n) < 0.5, 32767, 1)
        bits = (rng.random(n) < probs / 32768.0).astype(int) ^ 1
    else:  # runs of the likely bit at the extreme probability: 0xff carry chains
        probs = np.full(n, 32767)
        bits = np.zeros(n, dtype=int)
        bits[::977] = 1
    return probs.astype(np.uint16), bits.astype(np.uint8)


def symbol_case(n_symb, rows):
    rng = np.random.default_rng(100 + n_symb)
    probs = rng.dirichlet(np.full(n_symb, 0.3), size=rows).astype(np.float32)
    probs[0] = 0
    probs[0, n_symb // 2] = 1.0  # one-hot row: every decision clamps to [1, 32767]
    syms = [int(rng.choice(n_symb, p=p.astype(np.float64) / p.astype(np.float64).sum())) for p in probs]
    return probs, np.array(syms, dtype=np.int32)


def main():
    if not os.path.exists(T.REF_CODER):
        sys.exit("oracle/_ref/libnncp_coder_ref.so missing: make -C oracle ref")
    lib = C.CDLL(T.REF_CODER)
    lib.put_bit_init.argtypes = [C.POINTER(T.RefPutBit), C.POINTER(C.c_uint8), C.c_int, T.WRITE_FUNC, C.c_void_p]
    lib.put_bit.argtypes = [C.POINTER(T.RefPutBit), C.c_int, C.c_int]
    lib.put_bit_flush.restype = C.c_int64
    lib.put_bit_flush.argtypes = [C.POINTER(T.RefPutBit)]
    lib.write_sym.argtypes = [C.POINTER(T.RefPutBit), C.POINTER(C.c_float), C.c_int, C.c_int]
    lib.get_interp_param.restype = C.c_float
    out = {}
    for kind in ("uniform", "skewed", "carry"):
        probs, bits = range_coder_case(kind)
        enc = T.RefEncoder(lib)
        for p, b in zip(probs.tolist(), bits.tolist()):
            lib.put_bit(C.byref(enc.st), p, b)
        out["rc_%s_prob0" % kind], out["rc_%s_bits" % kind] = probs, bits
        out["rc_%s_bytes" % kind] = np.frombuffer(enc.finish(), dtype=np.uint8)
    for n_symb, rows in ((2, 100), (3, 100), (256, 40), (1000, 20)):
        probs, syms = symbol_case(n_symb, rows)
        enc = T.RefEncoder(lib)
        for p, s in zip(probs, syms.tolist()):
            lib.write_sym(C.byref(enc.st), p.ctypes.data_as(C.POINTER(C.c_float)), n_symb, s)
        out["sym_%d_probs" % n_symb], out["sym_%d_syms" % n_symb] = probs, syms
        out["sym_%d_bytes" % n_symb] = np.frombuffer(enc.finish(), dtype=np.uint8)

    class RefInterp(C.Structure):  # cp_utils.h:60-67
        _fields_ = [("n_steps", C.c_int), ("val", C.c_float * 9), ("pos", C.c_int64 * 8),
                    ("decay_power", C.c_float)]
    lib.get_interp_param.argtypes = [C.POINTER(RefInterp), C.c_int64]
    val = np.array([3e-4, 1e-4, 5e-5], dtype=np.float32)
    pos = np.array([1000, 5000], dtype=np.int64)
    powers = np.array([0.0, 0.5, 0.7], dtype=np.float32)
    at = np.array([0, 1, 999, 1000, 1001, 3000, 4999, 5000, 5001, 123456, 10 ** 9], dtype=np.int64)
    res = np.zeros((powers.size, at.size), dtype=np.float32)
    for i, power in enumerate(powers):
        s = RefInterp(n_steps=2, decay_power=float(power))
        for k, v in enumerate(val):
            s.val[k] = float(v)
        for k, v in enumerate(pos):
            s.pos[k] = int(v)
        for j, p in enumerate(at):
            res[i, j] = lib.get_interp_param(C.byref(s), int(p))
    out.update(interp_val=val, interp_pos=pos, interp_power=powers, interp_at=at, interp_out=res)
    path = os.path.join(HERE, "coder_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
