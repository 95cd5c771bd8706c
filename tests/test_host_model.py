"""Parameter files of the host mirror (nc_save_coefs / nc_load_coefs, libnc.h:530, 536) on
the CPU checker; the GPU side of the same round trip is in tests/test_gpu_zz_new_paths.py."""
import os

import numpy as np

import modelutil as M


def test_parameter_file_round_trip_on_the_checker(tmp_path):
    """nc_save_coefs / nc_load_coefs (libnc.h:530, 536): a trained model's parameters
    written to a file and read into a freshly initialised model of the same configuration
    are the same bits, and the two models then evaluate identically; a file that is not a
    parameter file, or that names a parameter the model lacks, ends the process with a
    message (libnc's error model), which a child process shows."""
    import subprocess, sys, textwrap
    pkg = M.load_pkg()
    cfg = dict(M.TINY)
    a = pkg.host.Model(M.ref_host(), pkg.host.make_config(**dict(cfg, use_device=0, nb_threads=2, sgd_opt=M.rmsprop(3e-3))))
    syms = M.markov1(cfg["batch_size"] * cfg["seg_len"] * 3, cfg["n_symbols"], seed=5)
    for tok, tgt in M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], 3):
        a.train_step(tok, tgt, 3e-3)
    path = tmp_path / "coefs.bin"
    a.save_coefs(str(path))
    b = pkg.host.Model(M.ref_host(), pkg.host.make_config(**dict(cfg, seed=99, use_device=0, nb_threads=2, sgd_opt=M.rmsprop(3e-3))))
    assert any(not np.array_equal(a.get_param(n), b.get_param(n)) for n in a.param_names())
    b.load_coefs(str(path))
    for n in a.param_names():
        assert np.array_equal(a.get_param(n), b.get_param(n)), n
    # file layout as documented: magic, version, empty configuration, first record's name
    raw = path.read_bytes()
    assert raw[:4] == b"NCPF" and int.from_bytes(raw[4:8], "little") == 1 and int.from_bytes(raw[8:12], "little") == 0
    nl = int.from_bytes(raw[12:16], "little")
    assert raw[16:16 + nl].decode() == a.param_names()[0]
    a.close(); b.close()
    bad = tmp_path / "bad.bin"
    bad.write_bytes(b"not a parameter file")
    code = textwrap.dedent('''
        import sys; sys.path.insert(0, %r)
        import modelutil as M
        pkg = M.load_pkg()
        m = pkg.host.Model(M.ref_host(), pkg.host.make_config(**dict(M.TINY, use_device=0, nb_threads=1)))
        m.load_coefs(%r)
    ''') % (os.path.dirname(os.path.abspath(__file__)), str(bad))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "not a parameter file" in r.stderr


# ---- malformed parameter files ---------------------------------------------------------
def malformed_parameter_files(tmp_path):
    """name -> (path, message expected on stderr).  The model these are fed to holds a
    parameter `embed`; every file starts with a valid header."""
    import struct
    head = b"NCPF" + struct.pack("<II", 1, 0)

    def rec(name, type_, dims, payload, name_len=None):
        nl = len(name) if name_len is None else name_len
        return (struct.pack("<I", nl) + name + struct.pack("<II", type_, len(dims)) +
                b"".join(struct.pack("<Q", d) for d in dims) + payload)

    files = {
        # a name length of 2^32 - 1: nl + 1 wraps to 0 in 32 bits
        "name_wraps": (head + rec(b"embed", 0, [4], b"\0" * 16, name_len=0xFFFFFFFF) + b"x" * 4096, "does not fit"),
        "name_too_long": (head + rec(b"e" * 300, 0, [4], b"\0" * 16), "does not fit"),
        "name_cut": (head + struct.pack("<I", 5) + b"em", "truncated"),
        "dims_cut": (head + struct.pack("<I", 5) + b"embed" + struct.pack("<II", 0, 2) + struct.pack("<Q", 4), "truncated"),
        "too_many_dims": (head + rec(b"embed", 0, [2] * 9, b""), "bad record"),
        "unknown_type": (head + rec(b"embed", 99, [4], b"\0" * 16), "bad record"),
        "zero_dim": (head + rec(b"embed", 0, [4, 0], b""), "more elements than the file holds"),
        "huge_dims": (head + rec(b"embed", 0, [1 << 40, 1 << 40], b"\0" * 64), "more elements than the file holds"),
        "overflowing_dims": (head + rec(b"embed", 0, [1 << 33, 1 << 33], b"\0" * 64), "more elements than the file holds"),
        "payload_cut": (head + rec(b"embed", 0, [64], b"\0" * 100), "more elements than the file holds"),
    }
    out = {}
    for name, (raw, msg) in files.items():
        p = tmp_path / (name + ".bin")
        p.write_bytes(raw)
        out[name] = (str(p), msg)
    return out


LOAD_IN_CHILD = '''
import sys; sys.path.insert(0, %r)
import modelutil as M
pkg = M.load_pkg()
m = pkg.host.Model(%s, pkg.host.make_config(**dict(M.TINY, use_device=%d, nb_threads=1)))
m.load_coefs(%r)
'''


def check_malformed_files_end_cleanly(tmp_path, host_expr, use_device, env=None):
    import signal, subprocess, sys
    for name, (path, msg) in malformed_parameter_files(tmp_path).items():
        code = LOAD_IN_CHILD % (os.path.dirname(os.path.abspath(__file__)), host_expr, use_device, path)
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120, env=env)
        # nc_fatal: a message and abort(); never a segmentation fault or a silent success
        assert r.returncode == -signal.SIGABRT, (name, r.returncode, r.stderr[-500:])
        assert "parameter file" in r.stderr and msg in r.stderr, (name, r.stderr[-500:])


def test_malformed_parameter_files_end_with_a_message_on_the_checker(tmp_path):
    """Parameter files are user input (--load_coefs): a record whose name length wraps in 32
    bits, is longer than the caller's buffer or is cut short, a record with too many
    dimensions, an unknown element type, a zero extent, extents whose product overflows or
    exceeds what the file still holds, and a payload cut short each end the process through
    nc_fatal - nothing is written past the name buffer and nothing is allocated first."""
    check_malformed_files_end_cleanly(tmp_path, "M.ref_host()", 0)
